"""ctypes binding of libats_gfx950.so.

The library is the only compute path of this package: if it is missing or a
call fails, an exception is raised.  There is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_uint64, c_size_t, c_void_p

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libats_gfx950.so")

ATS_F32, ATS_BF16 = 0, 1
ROUTE_SOFTMAX_TOPK, ROUTE_TOPK_SOFTMAX = 0, 1
IDX_I32, IDX_I64 = 0, 1


class AtsError(RuntimeError):
    """A libats_gfx950 entry point returned an error code."""


_SIGNATURES = {
    "ats_version": (c_int, []),
    "ats_last_error_string": (c_char_p, []),
    "ats_rmsnorm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_int, c_int, c_void_p]),
    "ats_rope_table": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_double, c_double, c_void_p]),
    "ats_rope_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int,
                             c_void_p]),
    "ats_rope_fwd_append": (c_int, [c_void_p] * 8 + [c_int] * 8 + [c_int64] * 14 + [c_int, c_void_p]),
    "ats_router_logits": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "ats_route_topk_workspace": (c_size_t, [c_int64, c_int]),
    "ats_route_topk": (c_int, [c_void_p, c_int64, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_float, c_void_p, c_size_t, c_void_p]),
    "ats_dispatch_plan_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "ats_dispatch_plan": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ats_dispatch_plan_static": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ats_gather_rows": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "ats_invert_token_map": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "ats_grouped_gateup_swiglu": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                          c_int64, c_int, c_int, c_int, c_void_p]),
    "ats_grouped_down_dgrad_dsilu_supported": (c_int, [c_int, c_int64, c_int, c_int, c_int]),
    "ats_grouped_down_dgrad_dsilu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64,
                                             c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p]),
    "ats_grouped_down_dgrad_dsilu_nn_supported": (c_int, [c_int, c_int64, c_int, c_int, c_int]),
    "ats_grouped_down_dgrad_dsilu_nn": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64,
                                                c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p]),
    "ats_grouped_gemm_nn_supported": (c_int, [c_int, c_int64, c_int, c_int, c_int64, c_int]),
    "ats_grouped_gemm_nn": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_void_p, c_int64,
                                    c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "ats_grouped_gateup_swiglu_save_supported": (c_int, [c_int64, c_int, c_int64, c_int, c_int, c_int]),
    "ats_grouped_gateup_swiglu_save": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_int64,
                                               c_void_p, c_void_p]),
    "ats_grouped_down": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int,
                                 c_int, c_int, c_void_p]),
    "ats_grouped_down_splitk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                        c_int, c_int, c_int, c_int, c_void_p]),
    "ats_sum_partials": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "ats_swiglu_partials": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "ats_combine_partials": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                     c_int, c_int, c_void_p]),
    "ats_rmsnorm_bwd_workspace": (c_size_t, [c_int64, c_int]),
    "ats_rmsnorm_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_int, c_int,
                                c_void_p, c_size_t, c_void_p]),
    "ats_rope_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int,
                             c_void_p]),
    "ats_silu_mul_fwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                 c_int, c_void_p]),
    "ats_silu_mul_bwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                 c_int64, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "ats_combine_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int,
                                c_int, c_int, c_int, c_void_p]),
    "ats_route_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_float,
                              c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "ats_router_bwd_dx": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "ats_router_bwd_dw_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "ats_router_bwd_dw": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_size_t,
                                  c_void_p]),
    "ats_transpose_batched": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "ats_wgrad_padded_rows": (c_int64, [c_int64, c_int]),
    "ats_wgrad_plan": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p]),
    "ats_transposed_zero_empty_groups": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "ats_transpose_grouped_rows": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                           c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "ats_grouped_gemm_nt": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                    c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int,
                                    c_int, c_int, c_void_p]),
    "ats_cross_entropy_fwd": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_int64, c_int, c_int, c_void_p]),
    "ats_cross_entropy_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int64, c_int, c_int, c_void_p]),
    "ats_grad_clip_chunk_elems": (c_int, []),
    "ats_grad_norm_clip": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                   c_float, c_int, c_void_p]),
    "ats_attention_fwd_workspace": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "ats_attention_fwd": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                  c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p,
                                  c_size_t, c_void_p]),
    "ats_attention_fwd_ex": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                     c_void_p, c_int64, c_int64, c_float, c_uint64, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p]),
    "ats_attention_bwd_ex": (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_float, c_uint64] + [c_void_p] * 3 + [c_int] * 6 +
                             [c_float, c_void_p]),
    "ats_attention_bwd_out": (c_int, [c_void_p] * 9 + [c_int64, c_int64, c_float, c_uint64] + [c_void_p] * 3 + [c_int] * 6 +
                              [c_float, c_void_p]),
    "ats_attention_softmax_f32": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p,
                                          c_void_p, c_int64, c_int64, c_float, c_uint64, c_void_p]),
    "ats_attention_softmax_bwd_f32": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                                              c_float, c_uint64, c_void_p]),
    "ats_attention_delta": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "ats_attention_bwd": (c_int, [c_void_p] * 10 + [c_int] * 6 + [c_float, c_void_p]),
    "ats_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                            c_void_p]),
    "ats_combine_scatter_add": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                                        c_int, c_void_p]),
    "ats_row_dot": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int, c_int,
                            c_void_p]),
    "ats_row_dot_copy": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int64, c_int,
                                 c_int, c_void_p]),
    "ats_select_topk_per_sequence": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ats_scatter_add_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "ats_kth_value_workspace": (ctypes.c_size_t, [c_int64]),
    "ats_kth_value_mask": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ats_topk_mask_ste": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ats_mod_route_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int64, c_void_p]),
    "ats_swiglu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    # the reference's launcher names (void return, float32 only)
    "rms_norm_launcher": (None, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "rope_precompute_launcher": (None, [c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "rope_apply_launcher": (None, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                   c_void_p]),
    "swiglu_launcher": (None, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "swiglu_fused_launcher": (None, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                     ctypes.c_bool, c_void_p]),
    "fused_cross_entropy_accuracy_launcher": (None, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                                     c_void_p]),
    "fused_grad_clip_launcher": (c_float, [c_void_p, c_void_p, c_int, c_float, c_void_p]),
    "ats_legacy_last_status": (c_int, []),
    "ats_calibrate_copy": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "ats_calibrate_read": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "ats_calibrate_mfma": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "ats_debug_decode_tile": (c_int, [c_int64, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "ats_debug_decode_tiles_device": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64,
                                              c_void_p, c_void_p]),
    "ats_debug_grid_blocks": (c_int64, [c_int64, c_int, c_int, c_int, c_int, c_int, c_int]),
}

_lib = None


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def load() -> ctypes.CDLL:
    """Loads the library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not is_built():
            raise AtsError(
                f"{LIB_PATH} is missing: build it with `python -m adaptivetrainingsystem_amd.build` "
                "(needs hipcc); this package has no fallback path")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().ats_last_error_string().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise AtsError(f"{what} failed with code {rc}: {last_error()}")
