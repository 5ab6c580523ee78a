"""Tensor-level wrappers of the libats_gfx950 entry points.

PyTorch is used for device memory and streams only: every function here
validates shapes on the host, allocates outputs with torch, and enqueues the
hand-written HIP kernels on torch's current stream.  Tensors must live on the
GPU; there is no CPU path.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import ATS_BF16, ATS_F32, IDX_I32, IDX_I64, ROUTE_SOFTMAX_TOPK, ROUTE_TOPK_SOFTMAX, AtsError, check

_DT = {torch.float32: ATS_F32, torch.bfloat16: ATS_BF16}


def _tag(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise AtsError(f"unsupported dtype {t.dtype}: the gfx950 kernels take float32 or bfloat16") from None


def _need_gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise AtsError("tensor is not on the GPU: the gfx950 path has no CPU fallback")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device.  The raw accessors skip the Stream object
    and the device bookkeeping of torch.cuda.current_stream (8 us a call, a tenth of a decode step)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------------- RMSNorm
def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float = 1e-6) -> torch.Tensor:
    _need_gpu(x, weight)
    H = x.shape[-1]
    xc = x.contiguous()
    if weight is not None:
        if weight.numel() != H:
            raise AtsError(f"rmsnorm: weight has {weight.numel()} elements, hidden size is {H}")
        weight = weight.contiguous()
    y = torch.empty_like(xc)
    rows = xc.numel() // H if H else 0
    check(_lib.load().ats_rmsnorm_fwd(xc.data_ptr(), _ptr(weight), y.data_ptr(), rows, H, float(eps), _tag(xc),
                                      _tag(weight) if weight is not None else ATS_F32, _stream()), "ats_rmsnorm_fwd")
    return y.view(x.shape)


# --------------------------------------------------------------------------- RoPE
def rope_table(seq_len: int, dim: int, theta: float = 10000.0, scaling_factor: Optional[float] = None,
               half: bool = False, device=None) -> Tuple[torch.Tensor, torch.Tensor]:
    device = torch.device("cuda") if device is None else torch.device(device)
    if device.type != "cuda":
        raise AtsError("rope_table: the table is built by a GPU kernel; pass a cuda device")
    cols = dim // 2 if half else dim
    cos = torch.empty(seq_len, cols, dtype=torch.float32, device=device)
    sin = torch.empty(seq_len, cols, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        check(_lib.load().ats_rope_table(cos.data_ptr(), sin.data_ptr(), seq_len, dim, cols, float(theta),
                                         1.0 if scaling_factor is None else float(scaling_factor), _stream()),
              "ats_rope_table")
    return cos, sin


def _bhl_strides(t: torch.Tensor):
    if t.stride(3) != 1:
        t = t.contiguous()
    return t, t.stride(0), t.stride(1), t.stride(2)


def rope(q: torch.Tensor, k: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
         position_offset: int = 0, inverse: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q [B,Hq,L,D], k [B,Hkv,L,D] (any batch/head/position strides), cos/sin float32
    [>= offset+L, D or D/2].  Returns new contiguous tensors.  inverse=True applies the
    inverse rotation, i.e. the gradient of the forward rotation."""
    _need_gpu(q, k, cos, sin)
    if q.dim() != 4 or (k is not None and k.dim() != 4):
        raise AtsError("rope: q and k must be [batch, heads, seq, head_dim]")
    B, Hq, L, D = q.shape
    Hkv = 0
    if k is not None:
        if k.shape[0] != B or k.shape[2] != L or k.shape[3] != D or k.dtype != q.dtype:
            raise AtsError(f"rope: k {tuple(k.shape)}/{k.dtype} does not match q {tuple(q.shape)}/{q.dtype}")
        Hkv = k.shape[1]
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2:
        raise AtsError("rope: cos/sin must be float32 2-D tables of equal shape")
    if cos.stride(1) != 1 or sin.stride(1) != 1 or cos.stride(0) != sin.stride(0):
        cos, sin = cos.contiguous(), sin.contiguous()
    q, qsb, qsh, qsl = _bhl_strides(q)
    q_out = torch.empty((B, Hq, L, D), dtype=q.dtype, device=q.device)
    k_out = None
    ksb = ksh = ksl = 0
    if k is not None:
        k, ksb, ksh, ksl = _bhl_strides(k)
        k_out = torch.empty((B, Hkv, L, D), dtype=k.dtype, device=k.device)
    name = "ats_rope_bwd" if inverse else "ats_rope_fwd"
    check(getattr(_lib.load(), name)(q.data_ptr(), _ptr(k), q_out.data_ptr(), _ptr(k_out), cos.data_ptr(),
                                     sin.data_ptr(), cos.stride(0), cos.shape[0], B, Hq, Hkv, L, D,
                                     int(position_offset), qsb, qsh, qsl, ksb, ksh, ksl, _tag(q), _stream()), name)
    return q_out, k_out


def rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                k_cache: torch.Tensor, v_cache: torch.Tensor, cache_pos: int,
                position_offset: int = 0) -> torch.Tensor:
    """rope(q, k) with the rotated keys, and the values beside them, written into the cache buffers
    k_cache / v_cache [B, Hkv, capacity, D] at positions cache_pos .. cache_pos + L - 1 (one launch instead of the
    rotation and two strided copies).  Returns the rotated q as a new contiguous tensor."""
    _need_gpu(q, k, v, cos, sin, k_cache, v_cache)
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise AtsError("rope_append: q, k, v [batch, heads, seq, head_dim] and two caches of one shape")
    B, Hq, L, D = q.shape
    Hkv = k.shape[1]
    if (k.shape[0] != B or k.shape[2] != L or k.shape[3] != D or k.dtype != q.dtype or v.dtype != q.dtype
            or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype or k_cache.shape[0] != B
            or k_cache.shape[1] != Hkv or k_cache.shape[3] != D or k_cache.stride() != v_cache.stride()
            or k_cache.stride(3) != 1):
        raise AtsError(f"rope_append: k/v {tuple(k.shape)}, caches {tuple(k_cache.shape)} do not match q {tuple(q.shape)}")
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2:
        raise AtsError("rope_append: cos/sin must be float32 2-D tables of equal shape")
    if cos.stride(1) != 1 or sin.stride(1) != 1 or cos.stride(0) != sin.stride(0):
        cos, sin = cos.contiguous(), sin.contiguous()
    q, qsb, qsh, qsl = _bhl_strides(q)
    k, ksb, ksh, ksl = _bhl_strides(k)
    v, vsb, vsh, vsl = _bhl_strides(v)
    q_out = torch.empty((B, Hq, L, D), dtype=q.dtype, device=q.device)
    check(_lib.load().ats_rope_fwd_append(q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(),
                                          k_cache.data_ptr(), v_cache.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                          cos.stride(0), cos.shape[0], B, Hq, Hkv, L, D, int(position_offset),
                                          qsb, qsh, qsl, ksb, ksh, ksl, vsb, vsh, vsl, k_cache.stride(0),
                                          k_cache.stride(1), k_cache.stride(2), int(cache_pos), k_cache.shape[2],
                                          _tag(q), _stream()), "ats_rope_fwd_append")
    return q_out


# --------------------------------------------------------------------------- router
def router_logits(x: torch.Tensor, gate_weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T,H], gate_weight [E,H] (same dtype) -> float32 logits [T,E]."""
    _need_gpu(x, gate_weight, bias)
    if x.dim() != 2 or gate_weight.dim() != 2 or x.shape[1] != gate_weight.shape[1] or x.dtype != gate_weight.dtype:
        raise AtsError(f"router_logits: x {tuple(x.shape)}/{x.dtype} vs weight {tuple(gate_weight.shape)}/{gate_weight.dtype}")
    T, H = x.shape
    E = gate_weight.shape[0]
    x, gate_weight = x.contiguous(), gate_weight.contiguous()
    if bias is not None:
        if bias.numel() != E:
            raise AtsError("router_logits: bias must have one entry per expert")
        bias = bias.to(torch.float32).contiguous()
    logits = torch.empty(T, E, dtype=torch.float32, device=x.device)
    check(_lib.load().ats_router_logits(x.data_ptr(), gate_weight.data_ptr(), _ptr(bias), logits.data_ptr(), T, H, E,
                                        _tag(x), _stream()), "ats_router_logits")
    return logits


def route_topk(logits: torch.Tensor, k: int, temperature: float = 1.0, variant: int = ROUTE_SOFTMAX_TOPK,
               load_balancing_weight: float = 0.01, with_stats: bool = True):
    """float32 logits [T,E] -> dict(indices int32 [T,k], weights f32 [T,k], hist int32 [E],
    prob_colsum f32 [E], aux f32 [1])."""
    _need_gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.float32:
        raise AtsError("route_topk: logits must be a float32 [tokens, experts] tensor")
    logits = logits.contiguous()
    T, E = logits.shape
    dev = logits.device
    idx = torch.empty(T, k, dtype=torch.int32, device=dev)
    w = torch.empty(T, k, dtype=torch.float32, device=dev)
    hist = colsum = aux = ws = None
    ws_bytes = 0
    lib = _lib.load()
    if with_stats:
        # one buffer for the three outputs; the finalize kernel writes every element (nothing runs for T == 0)
        stats = (torch.empty if T > 0 else torch.zeros)(2 * E + 1, dtype=torch.int32, device=dev)
        hist = stats[:E]
        colsum = stats[E:2 * E].view(torch.float32)
        aux = stats[2 * E:].view(torch.float32)
        ws_bytes = lib.ats_route_topk_workspace(T, E)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    check(lib.ats_route_topk(logits.data_ptr(), T, E, int(k), float(temperature), int(variant), idx.data_ptr(),
                             w.data_ptr(), _ptr(hist), _ptr(colsum), _ptr(aux), float(load_balancing_weight),
                             _ptr(ws), ws_bytes, _stream()), "ats_route_topk")
    return {"indices": idx, "weights": w, "hist": hist, "prob_colsum": colsum, "aux": aux}


def aux_loss_clean_logits(clean_logits: torch.Tensor, hist: torch.Tensor, k: int, variant: int,
                          load_balancing_weight: float) -> torch.Tensor:
    """Load-balancing loss when routing ran on noisy logits: usage from the routed histogram, importance from
    the noise-free, un-tempered logits (MS/core/model.py:1190-1192, 1244-1263).  Returns a float32 scalar."""
    T, E = clean_logits.shape
    colsum = route_topk(clean_logits, k, 1.0, variant, load_balancing_weight)["prob_colsum"]
    usage = hist.float() / (T * k + 1e-9)
    return torch.clamp((usage * (colsum / T)).sum() * (E * load_balancing_weight), max=1.0)


# --------------------------------------------------------------------------- dispatch
def expert_capacity(total_tokens: int, top_k: int, num_experts: int, capacity_factor: float) -> int:
    """Host-side integer, in double arithmetic then truncated, exactly as the reference computes it."""
    return int((total_tokens * top_k / num_experts) * capacity_factor)


def dispatch_plan(indices: torch.Tensor, num_experts: int, capacity: int):
    """indices [T,k] int32/int64 -> dict of int32 tensors: slot [T*k], token_map [E,C], hist [E],
    kept [E], offsets [E+1], row_src [min(T*k,E*C)], row_of [T*k], status [1]."""
    _need_gpu(indices)
    if indices.dim() != 2 or indices.dtype not in (torch.int32, torch.int64):
        raise AtsError("dispatch_plan: indices must be an int32/int64 [tokens, k] tensor")
    indices = indices.contiguous()
    T, k = indices.shape
    E, C = int(num_experts), int(capacity)
    dev = indices.device
    i32 = dict(dtype=torch.int32, device=dev)
    n = T * k
    out = {
        "slot": torch.empty(n, **i32), "token_map": torch.empty(E, C, **i32), "hist": torch.empty(E, **i32),
        "kept": torch.empty(E, **i32), "offsets": torch.empty(E + 1, **i32),
        "row_src": torch.empty(max(1, min(n, E * C)), **i32), "row_of": torch.empty(n, **i32),
        "status": torch.empty(1, **i32),
    }
    lib = _lib.load()
    ws_bytes = max(lib.ats_dispatch_plan_workspace(max(T, 1), k, E), 4 * E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    check(lib.ats_dispatch_plan(indices.data_ptr(), IDX_I64 if indices.dtype == torch.int64 else IDX_I32, T, k, E, C,
                                out["slot"].data_ptr(), out["token_map"].data_ptr(), out["hist"].data_ptr(),
                                out["kept"].data_ptr(), out["offsets"].data_ptr(), out["row_src"].data_ptr(),
                                out["row_of"].data_ptr(), out["status"].data_ptr(), ws.data_ptr(), ws_bytes,
                                _stream()), "ats_dispatch_plan")
    return out


def gather_rows(src: torch.Tensor, row_map: torch.Tensor, div: int = 1) -> torch.Tensor:
    """out[r] = src[row_map[r] // div] (zeros where row_map[r] < 0)."""
    _need_gpu(src, row_map)
    if src.dim() != 2 or row_map.dtype != torch.int32:
        raise AtsError("gather_rows: src must be 2-D and row_map int32")
    src, row_map = src.contiguous(), row_map.contiguous()
    n, H = row_map.numel(), src.shape[1]
    out = torch.empty(n, H, dtype=src.dtype, device=src.device)
    check(_lib.load().ats_gather_rows(src.data_ptr(), row_map.data_ptr(), int(div), out.data_ptr(), n, H, _tag(src),
                                      _stream()), "ats_gather_rows")
    return out


def invert_token_map(token_map: torch.Tensor, n_assign: int) -> torch.Tensor:
    _need_gpu(token_map)
    if token_map.dtype != torch.int32:
        raise AtsError("invert_token_map: token_map must be int32")
    token_map = token_map.contiguous()
    row_of = torch.empty(n_assign, dtype=torch.int32, device=token_map.device)
    check(_lib.load().ats_invert_token_map(token_map.data_ptr(), token_map.numel(), row_of.data_ptr(), n_assign,
                                           _stream()), "ats_invert_token_map")
    return row_of


# --------------------------------------------------------------------------- expert FFN
_pointer_table_cache: dict = {}


def weight_pointer_table(weights: Sequence[torch.Tensor]) -> torch.Tensor:
    """Device array of the experts' weight base addresses (int64)."""
    for w in weights:
        _need_gpu(w)
        if not w.is_contiguous():
            raise AtsError("expert weights must be contiguous")
    # the table holds nothing but the addresses it is keyed by, so an entry can never go stale
    key = (weights[0].device,) + tuple(w.data_ptr() for w in weights)
    table = _pointer_table_cache.get(key)
    if table is None:
        if len(_pointer_table_cache) > 256:
            _pointer_table_cache.clear()
        table = torch.tensor(key[1:], dtype=torch.int64, device=weights[0].device)
        _pointer_table_cache[key] = table
    return table


def grouped_gateup_swiglu(a: torch.Tensor, w_gu_ptrs: torch.Tensor, row_start: torch.Tensor, row_count: torch.Tensor,
                          n_rows_out: int, max_rows: int, H: int, I: int, a_rows: Optional[torch.Tensor] = None,
                          a_row_div: int = 1) -> torch.Tensor:
    _need_gpu(a, w_gu_ptrs, row_start, row_count, a_rows)
    if a.dim() != 2 or a.shape[1] != H or not a.is_contiguous():
        raise AtsError("grouped_gateup_swiglu: activations must be a contiguous [rows, H] tensor")
    E = w_gu_ptrs.numel()
    if row_start.numel() < E or row_count.numel() < E or row_start.dtype != torch.int32 or row_count.dtype != torch.int32:
        raise AtsError("grouped_gateup_swiglu: row_start/row_count must be int32 with one entry per expert")
    h = torch.empty(n_rows_out, I, dtype=a.dtype, device=a.device)
    check(_lib.load().ats_grouped_gateup_swiglu(a.data_ptr(), int(a.shape[0]), _ptr(a_rows), int(a_row_div), w_gu_ptrs.data_ptr(),
                                                h.data_ptr(), row_start.data_ptr(), row_count.data_ptr(), E,
                                                int(max_rows), H, I, _tag(a), _stream()), "ats_grouped_gateup_swiglu")
    return h


def grouped_gateup_swiglu_save(a: torch.Tensor, w_gu_ptrs: torch.Tensor, row_start: torch.Tensor,
                               row_count: torch.Tensor, n_rows_out: int, max_rows: int, H: int, I: int,
                               a_rows: Optional[torch.Tensor] = None, a_row_div: int = 1,
                               t_col0: Optional[torch.Tensor] = None
                               ) -> Optional[Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]]:
    """Training forward of the gate/up projection: (gu [rows, 2I], h [rows, I], hT) from one kernel, or None when
    the sizes are not prefill-sized (the caller then runs the plain product and silu_mul).  hT is None unless
    t_col0 (the k_start of wgrad_plan) is given and the dtype is bfloat16: then it is h transposed into the
    weight-gradient layout [I, wgrad_padded_rows] (see transpose_grouped_rows), written by the same kernel."""
    _need_gpu(a, w_gu_ptrs, row_start, row_count, a_rows)
    if a.dim() != 2 or a.shape[1] != H or not a.is_contiguous():
        raise AtsError("grouped_gateup_swiglu_save: activations must be a contiguous [rows, H] tensor")
    E = w_gu_ptrs.numel()
    if row_start.numel() < E or row_count.numel() < E or row_start.dtype != torch.int32 or row_count.dtype != torch.int32:
        raise AtsError("grouped_gateup_swiglu_save: row_start/row_count must be int32 with one entry per expert")
    lib = _lib.load()
    if not lib.ats_grouped_gateup_swiglu_save_supported(int(a.shape[0]), E, int(max_rows), H, I, _tag(a)):
        return None
    h = torch.empty(n_rows_out, I, dtype=a.dtype, device=a.device)
    gu = torch.empty(n_rows_out, 2 * I, dtype=a.dtype, device=a.device)
    hT, ld = _transposed_copy_buffer(I, row_count, t_col0, max_rows, E, a.dtype, a.device)
    check(lib.ats_grouped_gateup_swiglu_save(a.data_ptr(), int(a.shape[0]), _ptr(a_rows), int(a_row_div),
                                             w_gu_ptrs.data_ptr(), h.data_ptr(), gu.data_ptr(), row_start.data_ptr(),
                                             row_count.data_ptr(), E, int(max_rows), H, I, _tag(a), _ptr(hT), ld,
                                             _ptr(t_col0) if hT is not None else None, _stream()),
          "ats_grouped_gateup_swiglu_save")
    return gu, h, hT


def _transposed_copy_buffer(C: int, row_count: torch.Tensor, t_col0: Optional[torch.Tensor], max_rows: int, E: int,
                            dtype: torch.dtype, device) -> Tuple[Optional[torch.Tensor], int]:
    """The [C, padded rows] buffer that a training launch fills with the transposed copy of its result (bfloat16
    launches with the experts' first columns given), the columns of experts without rows already cleared."""
    if t_col0 is None or dtype != torch.bfloat16:
        return None, 0
    _need_gpu(t_col0)
    if t_col0.dtype != torch.int32 or t_col0.numel() < E:
        raise AtsError("transposed copy: t_col0 must be int32 with one entry per expert")
    ld = wgrad_padded_rows(max_rows, E)
    out = torch.empty(C, ld, dtype=dtype, device=device)
    check(_lib.load().ats_transposed_zero_empty_groups(out.data_ptr(), ld, C, row_count.data_ptr(), t_col0.data_ptr(), E,
                                                       _tag(out), _stream()), "ats_transposed_zero_empty_groups")
    return out, ld


def grouped_down_dgrad_dsilu_supported(E: int, max_rows: int, H: int, I: int, dtype: torch.dtype,
                                       transposed_weights: bool = True) -> bool:
    """Whether grouped_down_dgrad_dsilu has a kernel for these sizes (with the transposed, or the forward's own, weights)."""
    lib = _lib.load()
    fn = lib.ats_grouped_down_dgrad_dsilu_supported if transposed_weights else lib.ats_grouped_down_dgrad_dsilu_nn_supported
    return bool(fn(int(E), int(max_rows), int(H), int(I), _DT[dtype]))


def grouped_down_dgrad_dsilu(dy: torch.Tensor, w_dT_ptrs: torch.Tensor, gu: torch.Tensor, row_start: torch.Tensor,
                             row_count: torch.Tensor, max_rows: int, H: int, I: int,
                             t_col0: Optional[torch.Tensor] = None, transposed_weights: bool = True
                             ) -> Optional[Tuple[torch.Tensor, Optional[torch.Tensor]]]:
    """Training backward of the down projection and of silu(g) * u in one kernel: (dgu [rows, 2I], dguT) from
    dy [rows, H], the transposed down weights ([I, H] per expert) and the saved gu; None when the groups are not
    prefill-sized (the caller then runs the plain product and silu_mul_bwd).  dguT is None unless t_col0 (the
    k_start of wgrad_plan) is given and the dtype is bfloat16: then it is dgu transposed into the weight-gradient
    layout [2I, wgrad_padded_rows], written by the same kernel.  transposed_weights=False: the pointer table holds
    the forward's own down weights ([H, I] per expert; bfloat16, ats_grouped_down_dgrad_dsilu_nn)."""
    _need_gpu(dy, w_dT_ptrs, gu, row_start, row_count)
    if dy.dim() != 2 or dy.shape[1] != H or not dy.is_contiguous():
        raise AtsError("grouped_down_dgrad_dsilu: dy must be a contiguous [rows, H] tensor")
    if gu.dim() != 2 or gu.shape[1] != 2 * I or not gu.is_contiguous() or gu.dtype != dy.dtype or gu.shape[0] < dy.shape[0]:
        raise AtsError("grouped_down_dgrad_dsilu: gu must be a contiguous [rows, 2I] tensor of dy's dtype")
    E = w_dT_ptrs.numel()
    if row_start.numel() < E or row_count.numel() < E or row_start.dtype != torch.int32 or row_count.dtype != torch.int32:
        raise AtsError("grouped_down_dgrad_dsilu: row_start/row_count must be int32 with one entry per expert")
    lib = _lib.load()
    if not grouped_down_dgrad_dsilu_supported(E, max_rows, H, I, dy.dtype, transposed_weights):
        return None
    dgu = torch.empty_like(gu)
    dguT, ld = _transposed_copy_buffer(2 * I, row_count, t_col0, max_rows, E, dy.dtype, dy.device)
    fn = lib.ats_grouped_down_dgrad_dsilu if transposed_weights else lib.ats_grouped_down_dgrad_dsilu_nn
    check(fn(dy.data_ptr(), w_dT_ptrs.data_ptr(), gu.data_ptr(), dgu.data_ptr(), row_start.data_ptr(),
             row_count.data_ptr(), E, int(max_rows), H, I, _tag(dy), _ptr(dguT), ld,
             _ptr(t_col0) if dguT is not None else None, _stream()),
          "ats_grouped_down_dgrad_dsilu" if transposed_weights else "ats_grouped_down_dgrad_dsilu_nn")
    return dgu, dguT


def grouped_down(h: torch.Tensor, w_d_ptrs: torch.Tensor, row_start: torch.Tensor, row_count: torch.Tensor,
                 max_rows: int, H: int, I: int, out: Optional[torch.Tensor] = None,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    _need_gpu(h, w_d_ptrs, row_start, row_count, out)
    if h.dim() != 2 or h.shape[1] != I or not h.is_contiguous():
        raise AtsError("grouped_down: h must be a contiguous [rows, I] tensor")
    E = w_d_ptrs.numel()
    if out is None:
        out = torch.empty(h.shape[0], H, dtype=out_dtype or h.dtype, device=h.device)
    check(_lib.load().ats_grouped_down(h.data_ptr(), w_d_ptrs.data_ptr(), out.data_ptr(), row_start.data_ptr(),
                                       row_count.data_ptr(), E, int(max_rows), H, I, _tag(h), _tag(out), _stream()),
          "ats_grouped_down")
    return out


def down_k_splits(E: int, max_rows: int, N: int, K: int, dtype: torch.dtype) -> int:
    """Slices of K for a projection with few rows per expert.  Such a product streams its weights, and
    it takes several hundred workgroups to keep the memory system busy; the plain tilings give
    E * ceil(N / 128) of them up to 32 rows per expert and E * ceil(rows / 128) * ceil(N / 256) above.
    When that is under 384, 32-row tiles (64-row tiles above 32 rows) with K cut into slices are used
    instead, if two or more slices are needed to fill the chip (measured on MI355X: 8 x [4096, 14336]
    weights x 16 rows 199 -> 160 us with 2 slices; one [4096, 4096] weight x 64 rows 50 -> 10 us with 8,
    x 256 rows 51 -> 23 us with 2; [4096, 14336] x 64 rows 156 -> 22 us with 8).
    Powers of two up to 16, slices of at least 512 columns, at most 256 rows per expert."""
    slab = 64 if dtype == torch.bfloat16 else 32
    if E <= 0 or max_rows <= 0:
        return 1
    rows = -(-max_rows // E)
    if rows > 256:
        return 1
    n128 = (N + 127) // 128
    plain = E * n128 if max_rows // E <= 32 else E * ((rows + 127) // 128) * ((N + 255) // 256)
    if plain >= 384:
        return 1
    # 32-row tiles (three workgroups per CU) up to 32 rows, 64-row tiles (two per CU) above
    groups = E * (1 if rows <= 32 else (rows + 63) // 64) * n128
    enough = 384 if rows <= 32 else 256
    s = 1
    while s < 16 and groups * s < enough and K % (2 * s * slab) == 0 and K // (2 * s) >= 512:
        s *= 2
    return s


def grouped_down_splitk(h: torch.Tensor, w_d_ptrs: torch.Tensor, row_start: torch.Tensor, row_count: torch.Tensor,
                        max_rows: int, H: int, I: int, k_splits: int) -> torch.Tensor:
    """Float32 partial results [k_splits, rows, H] of grouped_down with K cut into k_splits slices
    (decode sizes only); sum_partials or combine_partials add them up."""
    _need_gpu(h, w_d_ptrs, row_start, row_count)
    if h.dim() != 2 or h.shape[1] != I or not h.is_contiguous():
        raise AtsError("grouped_down_splitk: h must be a contiguous [rows, I] tensor")
    E = w_d_ptrs.numel()
    parts = torch.empty(k_splits, h.shape[0], H, dtype=torch.float32, device=h.device)
    check(_lib.load().ats_grouped_down_splitk(h.data_ptr(), w_d_ptrs.data_ptr(), parts.data_ptr(), row_start.data_ptr(),
                                              row_count.data_ptr(), E, int(max_rows), h.shape[0], H, I, int(k_splits),
                                              _tag(h), _stream()), "ats_grouped_down_splitk")
    return parts


def sum_partials(parts: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """parts float32 [S, ...] -> their sum over S in slice order, rounded once to out_dtype."""
    _need_gpu(parts)
    if parts.dtype != torch.float32 or parts.dim() < 2 or not parts.is_contiguous():
        raise AtsError("sum_partials: parts must be a contiguous float32 [slices, ...] tensor")
    out = torch.empty(parts.shape[1:], dtype=out_dtype, device=parts.device)
    check(_lib.load().ats_sum_partials(parts.data_ptr(), parts.shape[0], out.numel(), out.data_ptr(), out.numel(),
                                       _tag(out), _stream()), "ats_sum_partials")
    return out


def swiglu_partials(parts: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """parts float32 [S, rows, 2I] (a gate/up projection cut along K, gate columns first) ->
    silu(sum gate) * (sum up) as [rows, I] of out_dtype."""
    _need_gpu(parts)
    if parts.dtype != torch.float32 or parts.dim() != 3 or parts.shape[2] % 8 or not parts.is_contiguous():
        raise AtsError("swiglu_partials: parts must be a contiguous float32 [slices, rows, 2I] tensor")
    S, rows, two_i = parts.shape
    out = torch.empty(rows, two_i // 2, dtype=out_dtype, device=parts.device)
    check(_lib.load().ats_swiglu_partials(parts.data_ptr(), S, rows * two_i, out.data_ptr(), rows, two_i // 2, _tag(out),
                                          _stream()), "ats_swiglu_partials")
    return out


# --------------------------------------------------------------------------- combine
def combine(y: torch.Tensor, row_of: torch.Tensor, weights: torch.Tensor, num_tokens: int, k: int,
            out_dtype: Optional[torch.dtype] = None, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y [rows, H] (any leading shape); row_of int32 [T*k]; weights f32 [T,k] -> out [T,H]."""
    _need_gpu(y, row_of, weights, residual)
    if row_of.dtype != torch.int32 or weights.dtype != torch.float32:
        raise AtsError("combine: row_of must be int32 and weights float32")
    if row_of.numel() != num_tokens * k or weights.numel() != num_tokens * k:
        raise AtsError("combine: row_of/weights must have tokens*k entries")
    y2 = y.reshape(-1, y.shape[-1]).contiguous()
    H = y2.shape[1]
    out = torch.empty(num_tokens, H, dtype=out_dtype or y.dtype, device=y.device)
    if residual is not None:
        residual = residual.reshape(num_tokens, H).contiguous()
        if residual.dtype != out.dtype:
            raise AtsError("combine: residual must have the output dtype")
    check(_lib.load().ats_combine(y2.data_ptr(), row_of.contiguous().data_ptr(), weights.contiguous().data_ptr(),
                                  _ptr(residual), out.data_ptr(), num_tokens, int(k), H, _tag(y2), _tag(out),
                                  _stream()), "ats_combine")
    return out


def combine_scatter_add(y: torch.Tensor, row_of: torch.Tensor, weights: torch.Tensor, num_tokens: int, k: int,
                        out: torch.Tensor, out_rows: torch.Tensor) -> bool:
    """combine whose result is added onto rows out_rows[t] (int32, distinct, negative = skip) of `out` [N, H] in
    place, with the bits of combine followed by scatter_add_rows.  Returns False (nothing done) when the sizes
    are outside the vector kernel (k > 8, H not a multiple of 8, unaligned views)."""
    _need_gpu(y, row_of, weights, out, out_rows)
    if row_of.dtype != torch.int32 or weights.dtype != torch.float32 or out_rows.dtype != torch.int32:
        raise AtsError("combine_scatter_add: row_of / out_rows must be int32 and weights float32")
    if row_of.numel() != num_tokens * k or weights.numel() != num_tokens * k or out_rows.numel() != num_tokens:
        raise AtsError("combine_scatter_add: row_of/weights must have tokens*k entries, out_rows one per token")
    y2 = y.reshape(-1, y.shape[-1]).contiguous()
    H = y2.shape[1]
    if out.dim() != 2 or out.shape[1] != H or not out.is_contiguous():
        raise AtsError("combine_scatter_add: out must be a contiguous [rows, H] tensor")
    if k > 8 or H % 8 or y2.data_ptr() % 16 or out.data_ptr() % 16:
        return False
    check(_lib.load().ats_combine_scatter_add(y2.data_ptr(), row_of.contiguous().data_ptr(),
                                              weights.contiguous().data_ptr(), out_rows.contiguous().data_ptr(),
                                              out.data_ptr(), num_tokens, int(k), H, _tag(y2), _tag(out), _stream()),
          "ats_combine_scatter_add")
    return True


def combine_partials(parts: torch.Tensor, row_of: torch.Tensor, weights: torch.Tensor, num_tokens: int, k: int,
                     out_dtype: torch.dtype, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """combine over the float32 partial results [S, rows, H] of grouped_down_splitk: an expert row is their
    sum in slice order, rounded to out_dtype like the unsplit projection's result, before the weighting."""
    _need_gpu(parts, row_of, weights, residual)
    if row_of.dtype != torch.int32 or weights.dtype != torch.float32:
        raise AtsError("combine_partials: row_of must be int32 and weights float32")
    if row_of.numel() != num_tokens * k or weights.numel() != num_tokens * k:
        raise AtsError("combine_partials: row_of/weights must have tokens*k entries")
    if parts.dim() != 3 or parts.dtype != torch.float32 or not parts.is_contiguous():
        raise AtsError("combine_partials: partial results must be a contiguous float32 [slices, rows, H] tensor")
    S, rows, H = parts.shape
    out = torch.empty(num_tokens, H, dtype=out_dtype, device=parts.device)
    if residual is not None:
        residual = residual.reshape(num_tokens, H).contiguous()
        if residual.dtype != out.dtype:
            raise AtsError("combine_partials: residual must have the output dtype")
    check(_lib.load().ats_combine_partials(parts.data_ptr(), S, rows * H, row_of.contiguous().data_ptr(),
                                           weights.contiguous().data_ptr(), _ptr(residual), out.data_ptr(),
                                           num_tokens, int(k), H, _tag(out), _stream()), "ats_combine_partials")
    return out


# --------------------------------------------------------------------------- MoD helpers
def row_dot(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, temperature: float = 1.0,
            want_prob: bool = False, want_copy: bool = False):
    """score[t] = x[t,:] . w (+ bias); optionally sigmoid(score / temperature).  want_copy: the same pass also
    writes a copy of the rows ([T, H], returned last), the start of a residual output."""
    _need_gpu(x, w, bias)
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    T, H = x2.shape
    w = w.reshape(-1).contiguous()
    if w.numel() != H or w.dtype != x2.dtype:
        raise AtsError("row_dot: weight must have H elements of x's dtype")
    if bias is not None:
        bias = bias.reshape(-1).to(torch.float32).contiguous()
    score = torch.empty(T, dtype=torch.float32, device=x.device)
    prob = torch.empty(T, dtype=torch.float32, device=x.device) if want_prob else None
    copy = torch.empty_like(x2) if want_copy else None
    check(_lib.load().ats_row_dot_copy(x2.data_ptr(), w.data_ptr(), _ptr(bias), score.data_ptr(), _ptr(prob),
                                       float(temperature), _ptr(copy), T, H, _tag(x2), _stream()), "ats_row_dot_copy")
    res = (score, prob) if want_prob else (score,)
    if want_copy:
        res = res + (copy,)
    return res if len(res) > 1 else res[0]


def select_topk_per_sequence(scores: torch.Tensor, keep: int) -> torch.Tensor:
    """scores f32 [B,L] -> flat token ids (b*L+pos) of the `keep` best per sequence, ascending, int32 [B*keep]."""
    _need_gpu(scores)
    if scores.dim() != 2 or scores.dtype != torch.float32:
        raise AtsError("select_topk_per_sequence: scores must be float32 [batch, seq]")
    scores = scores.contiguous()
    B, L = scores.shape
    sel = torch.empty(B * keep, dtype=torch.int32, device=scores.device)
    check(_lib.load().ats_select_topk_per_sequence(scores.data_ptr(), B, L, int(keep), sel.data_ptr(), _stream()),
          "ats_select_topk_per_sequence")
    return sel


def scatter_add_rows(base: torch.Tensor, rows: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    """base[rows[i]] += delta[i] in place (rows distinct); returns base."""
    _need_gpu(base, rows, delta)
    if not base.is_contiguous() or base.dim() != 2 or rows.dtype != torch.int32 or delta.dtype != base.dtype:
        raise AtsError("scatter_add_rows: base must be contiguous 2-D, rows int32, delta of base's dtype")
    delta = delta.reshape(-1, base.shape[1]).contiguous()
    check(_lib.load().ats_scatter_add_rows(base.data_ptr(), rows.contiguous().data_ptr(), delta.data_ptr(),
                                           rows.numel(), base.shape[1], _tag(base), _stream()),
          "ats_scatter_add_rows")
    return base


def kth_value_mask(values: torch.Tensor, kth: int, return_count: bool = False):
    """float32 mask of values >= the kth smallest value (1-based), same shape as `values`; with
    `return_count` also the number of ones as a one-element int64 device tensor (written by the kernel)."""
    _need_gpu(values)
    if values.dtype != torch.float32:
        raise AtsError("kth_value_mask: values must be float32")
    v = values.contiguous()
    mask = torch.empty_like(v)
    lib = _lib.load()
    ws_bytes = int(lib.ats_kth_value_workspace(v.numel()))       # 16 bytes, or with room for the digit histograms
    ws = torch.zeros(ws_bytes // 8, dtype=torch.int64, device=v.device) if v.numel() == 0 else \
        torch.empty(ws_bytes // 8, dtype=torch.int64, device=v.device)
    check(lib.ats_kth_value_mask(v.data_ptr(), v.numel(), int(kth), mask.data_ptr(), ws.data_ptr(), ws_bytes,
                                 _stream()), "ats_kth_value_mask")
    return (mask, ws[1:2]) if return_count else mask


def topk_mask_ste(values: torch.Tensor, k: int, want_ste: bool = True):
    """float32 mask with exactly min(k, n) ones at the k largest of `values` (lower index first among equals)
    and, with `want_ste`, the straight-through weights (mask - values) + values; both of `values`' shape."""
    _need_gpu(values)
    if values.dtype != torch.float32:
        raise AtsError("topk_mask_ste: values must be float32")
    v = values.contiguous()
    mask = torch.empty_like(v)
    ste = torch.empty_like(v) if want_ste else None
    lib = _lib.load()
    ws_bytes = int(lib.ats_kth_value_workspace(v.numel()))
    ws = torch.empty(max(ws_bytes // 8, 2), dtype=torch.int64, device=v.device)
    check(lib.ats_topk_mask_ste(v.data_ptr(), v.numel(), int(k), mask.data_ptr(), _ptr(ste), ws.data_ptr(), ws_bytes,
                                _stream()), "ats_topk_mask_ste")
    return (mask, ste) if want_ste else mask


def mod_route_bwd(prob: torch.Tensor, grad_weights: Optional[torch.Tensor], grad_probs: Optional[torch.Tensor],
                  temperature: float = 1.0, need_bias: bool = True):
    """Gradient of the MoD router's logits, float32 [n], and of its bias, float32 [1] (or None)."""
    _need_gpu(prob, grad_weights, grad_probs)
    p = prob.reshape(-1).contiguous()
    n = p.numel()
    for g in (grad_weights, grad_probs):
        if g is not None and (g.dtype != torch.float32 or g.numel() != n):
            raise AtsError("mod_route_bwd: gradients must be float32 with one value per token")
    if p.dtype != torch.float32:
        raise AtsError("mod_route_bwd: probabilities must be float32")
    gw = None if grad_weights is None else grad_weights.reshape(-1).contiguous()
    gp = None if grad_probs is None else grad_probs.reshape(-1).contiguous()
    gl = torch.empty(n, dtype=torch.float32, device=p.device)
    db = torch.empty(1, dtype=torch.float32, device=p.device) if need_bias else None
    check(_lib.load().ats_mod_route_bwd(_ptr(gw), _ptr(gp), p.data_ptr(), float(temperature), gl.data_ptr(), _ptr(db), n,
                                        _stream()), "ats_mod_route_bwd")
    return gl, db


def swiglu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """gate * silu(up) (dense-FFN convention of the fused wrapper)."""
    _need_gpu(gate, up)
    if gate.shape != up.shape or gate.dtype != up.dtype:
        raise AtsError("swiglu_mul: gate and up must match")
    g, u = gate.contiguous(), up.contiguous()
    out = torch.empty_like(g)
    check(_lib.load().ats_swiglu_mul(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _tag(g), _stream()),
          "ats_swiglu_mul")
    return out


# --------------------------------------------------------------------------- backward pass
def rmsnorm_bwd(x: torch.Tensor, weight: Optional[torch.Tensor], dy: torch.Tensor, eps: float = 1e-6,
                need_dw: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Gradients of rmsnorm: dx (x's shape and dtype) and dw (float32 [H]) or None."""
    _need_gpu(x, weight, dy)
    H = x.shape[-1]
    if dy.shape != x.shape or dy.dtype != x.dtype:
        raise AtsError(f"rmsnorm_bwd: dy {tuple(dy.shape)}/{dy.dtype} does not match x {tuple(x.shape)}/{x.dtype}")
    xc, dyc = x.contiguous(), dy.contiguous()
    if weight is not None:
        weight = weight.contiguous()
    rows = xc.numel() // H if H else 0
    dx = torch.empty_like(xc)
    lib = _lib.load()
    dw = ws = None
    ws_bytes = 0
    if need_dw and weight is not None:
        dw = torch.empty(H, dtype=torch.float32, device=x.device)
        ws_bytes = lib.ats_rmsnorm_bwd_workspace(rows, H)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    check(lib.ats_rmsnorm_bwd(xc.data_ptr(), _ptr(weight), dyc.data_ptr(), dx.data_ptr(), _ptr(dw), rows, H,
                              float(eps), _tag(xc), _tag(weight) if weight is not None else ATS_F32, _ptr(ws),
                              ws_bytes, _stream()), "ats_rmsnorm_bwd")
    return dx.view(x.shape), dw


def _rows_2d(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dim() != 2 or t.stride(1) != 1:
        raise AtsError(f"{name}: operands must be 2-D with contiguous rows")
    return t


def silu_mul(a: torch.Tensor, b: torch.Tensor, rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(a) * b for 2-D operands that may be column slices of a wider matrix.  rows_dev: optional
    int32 device scalar; rows at or beyond it are left untouched."""
    _need_gpu(a, b, rows_dev)
    a, b = _rows_2d(a, "silu_mul"), _rows_2d(b, "silu_mul")
    if a.shape != b.shape or a.dtype != b.dtype:
        raise AtsError("silu_mul: operand shapes / dtypes differ")
    out = torch.empty(a.shape, dtype=a.dtype, device=a.device)
    check(_lib.load().ats_silu_mul_fwd(a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), out.data_ptr(),
                                       out.stride(0) if out.numel() else a.shape[1], a.shape[0], _ptr(rows_dev),
                                       a.shape[1], _tag(a), _stream()), "ats_silu_mul_fwd")
    return out


def silu_mul_bwd(a: torch.Tensor, b: torch.Tensor, dout: torch.Tensor, da: Optional[torch.Tensor] = None,
                 db: Optional[torch.Tensor] = None,
                 rows_dev: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gradients of silu(a) * b; da/db may be preallocated (e.g. the two halves of one matrix)."""
    _need_gpu(a, b, dout, da, db)
    a, b, dout = _rows_2d(a, "silu_mul_bwd"), _rows_2d(b, "silu_mul_bwd"), _rows_2d(dout, "silu_mul_bwd")
    if a.shape != b.shape or a.shape != dout.shape or a.dtype != b.dtype or a.dtype != dout.dtype:
        raise AtsError("silu_mul_bwd: operand shapes / dtypes differ")
    if da is None:
        da = torch.empty(a.shape, dtype=a.dtype, device=a.device)
    if db is None:
        db = torch.empty(a.shape, dtype=a.dtype, device=a.device)
    da, db = _rows_2d(da, "silu_mul_bwd"), _rows_2d(db, "silu_mul_bwd")
    cols = a.shape[1]
    st = lambda t: t.stride(0) if t.shape[0] > 1 else max(t.stride(0), cols)
    check(_lib.load().ats_silu_mul_bwd(a.data_ptr(), st(a), b.data_ptr(), st(b), dout.data_ptr(), st(dout),
                                       da.data_ptr(), st(da), db.data_ptr(), st(db), a.shape[0], _ptr(rows_dev), cols,
                                       _tag(a), _stream()), "ats_silu_mul_bwd")
    return da, db


def combine_bwd(dout: torch.Tensor, y: torch.Tensor, token_map: torch.Tensor, w: torch.Tensor,
                k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gradients of combine: dy (y's shape/dtype) and dw float32 [T, k]."""
    _need_gpu(dout, y, token_map, w)
    if dout.dim() != 2 or y.dim() != 2 or dout.shape[1] != y.shape[1] or token_map.dtype != torch.int32:
        raise AtsError("combine_bwd: dout [T,H], y [rows,H], token_map int32 [rows]")
    T, H = dout.shape
    n_rows = y.shape[0]
    if token_map.numel() < n_rows or w.numel() != T * k or w.dtype != torch.float32:
        raise AtsError("combine_bwd: token_map / weights do not match the row and token counts")
    dout, y, w = dout.contiguous(), y.contiguous(), w.contiguous()
    dy = torch.empty_like(y)
    dw = torch.empty(T, k, dtype=torch.float32, device=y.device)
    check(_lib.load().ats_combine_bwd(dout.data_ptr(), y.data_ptr(), token_map.data_ptr(), w.data_ptr(), dy.data_ptr(),
                                      dw.data_ptr(), n_rows, T, int(k), H, _tag(y), _tag(dout), _stream()),
          "ats_combine_bwd")
    return dy, dw


def route_bwd(logits_route: torch.Tensor, idx: torch.Tensor, w: torch.Tensor, dw: torch.Tensor,
              temperature: float = 1.0, mode: int = ROUTE_SOFTMAX_TOPK, logits_aux: Optional[torch.Tensor] = None,
              usage: Optional[torch.Tensor] = None, aux_scale: float = 0.0,
              aux_scale_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dlogits [T,E] float32 of the routing rule (and of the load-balancing loss when usage is given;
    its factor is aux_scale times the optional float32 device scalar aux_scale_dev)."""
    _need_gpu(logits_route, idx, w, dw, logits_aux, usage, aux_scale_dev)
    if aux_scale_dev is not None and (aux_scale_dev.dtype != torch.float32 or aux_scale_dev.numel() != 1):
        raise AtsError("route_bwd: aux_scale_dev must be a float32 scalar tensor")
    T, E = logits_route.shape
    k = idx.shape[1]
    if (logits_route.dtype != torch.float32 or idx.dtype != torch.int32 or w.dtype != torch.float32
            or dw.dtype != torch.float32 or w.shape != idx.shape or dw.shape != idx.shape):
        raise AtsError("route_bwd: logits float32 [T,E], idx int32 [T,k], w/dw float32 [T,k]")
    logits_route, idx, w, dw = logits_route.contiguous(), idx.contiguous(), w.contiguous(), dw.contiguous()
    if usage is not None:
        usage = usage.contiguous().float()
        logits_aux = (logits_route if logits_aux is None else logits_aux).contiguous()
    out = torch.empty(T, E, dtype=torch.float32, device=logits_route.device)
    check(_lib.load().ats_route_bwd(logits_route.data_ptr(), _ptr(logits_aux), idx.data_ptr(), w.data_ptr(),
                                    dw.data_ptr(), _ptr(usage), float(aux_scale), _ptr(aux_scale_dev),
                                    float(temperature), int(mode), out.data_ptr(), T, E, k, _stream()),
          "ats_route_bwd")
    return out


def router_bwd(dlogits: torch.Tensor, x: torch.Tensor, gate_weight: torch.Tensor,
               base: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
               need_dx: bool = True, need_dw: bool = True) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Gradients of router_logits: dx = base + dlogits @ Wg (x's dtype) and dWg float32 [E,H]."""
    _need_gpu(dlogits, x, gate_weight, base, out)
    T, H = x.shape
    E = gate_weight.shape[0]
    if dlogits.shape != (T, E) or dlogits.dtype != torch.float32 or gate_weight.dtype != x.dtype:
        raise AtsError("router_bwd: dlogits float32 [T,E]; x and the gate weight share a dtype")
    dlogits, xc, wg = dlogits.contiguous(), x.contiguous(), gate_weight.contiguous()
    lib = _lib.load()
    dx = dwg = None
    if need_dx:
        if base is not None:
            base = base.contiguous()
        dx = out if out is not None else torch.empty_like(xc)
        check(lib.ats_router_bwd_dx(dlogits.data_ptr(), wg.data_ptr(), _ptr(base), dx.data_ptr(), T, E, H, _tag(xc),
                                    _stream()), "ats_router_bwd_dx")
    if need_dw:
        dwg = torch.empty(E, H, dtype=torch.float32, device=x.device)
        ws_bytes = lib.ats_router_bwd_dw_workspace(T, E, H)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
        check(lib.ats_router_bwd_dw(dlogits.data_ptr(), xc.data_ptr(), dwg.data_ptr(), T, E, H, _tag(xc),
                                    ws.data_ptr(), ws_bytes, _stream()), "ats_router_bwd_dw")
    return dx, dwg


def transpose_batched(mats: Sequence[torch.Tensor]) -> Tuple[list, torch.Tensor]:
    """Transposes E equally shaped contiguous matrices [R,C]; returns the list of [C,R] views of one
    buffer and the device pointer table over them."""
    _need_gpu(*mats)
    R, C = mats[0].shape
    for m in mats:
        if m.shape != (R, C) or m.dtype != mats[0].dtype or not m.is_contiguous():
            raise AtsError("transpose_batched: matrices must be contiguous and share shape and dtype")
    E = len(mats)
    buf = torch.empty(E, C, R, dtype=mats[0].dtype, device=mats[0].device)
    outs = [buf[e] for e in range(E)]
    in_tab = weight_pointer_table(list(mats))
    out_tab = weight_pointer_table(outs)
    aligned = all(m.data_ptr() % 16 == 0 for m in mats) and all(o.data_ptr() % 16 == 0 for o in outs)
    check(_lib.load().ats_transpose_batched(in_tab.data_ptr(), out_tab.data_ptr(), E, R, C, _tag(mats[0]), int(aligned),
                                            _stream()), "ats_transpose_batched")
    return outs, out_tab


def wgrad_plan(row_count: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per expert: first column and padded width of its slice in the transposed activations."""
    _need_gpu(row_count)
    E = row_count.numel()
    k_start = torch.empty(E, dtype=torch.int32, device=row_count.device)
    k_count = torch.empty(E, dtype=torch.int32, device=row_count.device)
    check(_lib.load().ats_wgrad_plan(row_count.data_ptr(), E, k_start.data_ptr(), k_count.data_ptr(), _stream()),
          "ats_wgrad_plan")
    return k_start, k_count


def wgrad_padded_rows(max_rows: int, E: int) -> int:
    return int(_lib.load().ats_wgrad_padded_rows(int(max_rows), int(E)))


def transpose_grouped_rows(src: torch.Tensor, row_start: torch.Tensor, row_count: torch.Tensor, max_rows: int,
                           gather: Optional[torch.Tensor] = None, gather_div: int = 1) -> torch.Tensor:
    """[rows, C] -> [C, padded] with expert e in columns k_start[e] .. (see wgrad_plan), zero padded."""
    _need_gpu(src, row_start, row_count, gather)
    src = _rows_2d(src, "transpose_grouped_rows")
    E = row_count.numel()
    C = src.shape[1]
    ld = wgrad_padded_rows(max_rows, E)
    out = torch.empty(C, ld, dtype=src.dtype, device=src.device)
    check(_lib.load().ats_transpose_grouped_rows(src.data_ptr(), src.stride(0), C, _ptr(gather), int(gather_div),
                                                 row_start.data_ptr(), row_count.data_ptr(), E, int(max_rows),
                                                 out.data_ptr(), ld, _tag(src), _stream()),
          "ats_transpose_grouped_rows")
    return out


def grouped_gemm_nt(b_ptrs: torch.Tensor, ldb: int, b_rows: int, row_start: torch.Tensor, row_count: torch.Tensor,
                    n_rows_out: int, max_rows: int, N: int, K: int, a: Optional[torch.Tensor] = None,
                    a_ptrs: Optional[torch.Tensor] = None, lda: Optional[int] = None,
                    a_rows: Optional[torch.Tensor] = None, a_row_div: int = 1, k_count: Optional[torch.Tensor] = None,
                    dtype: Optional[torch.dtype] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[row_start[e]+m, :N] = A_e[m, :K_e] @ B_e[:N, :K_e]^T (see ats_grouped_gemm_nt)."""
    _need_gpu(a, a_ptrs, b_ptrs, row_start, row_count, a_rows, k_count)
    if (a is None) == (a_ptrs is None):
        raise AtsError("grouped_gemm_nt: give either a or a_ptrs")
    if a is not None:
        a = _rows_2d(a, "grouped_gemm_nt")
        dtype = a.dtype
        lda = a.stride(0)
    elif dtype is None or lda is None:
        raise AtsError("grouped_gemm_nt: a_ptrs needs dtype and lda")
    out_dtype = dtype if out_dtype is None else out_dtype
    E = b_ptrs.numel()
    out = torch.empty(n_rows_out, N, dtype=out_dtype, device=b_ptrs.device)
    check(_lib.load().ats_grouped_gemm_nt(_ptr(a), _ptr(a_ptrs), int(lda), int(a.shape[0]) if a is not None else 0,
                                          _ptr(a_rows), int(a_row_div), b_ptrs.data_ptr(), int(ldb), int(b_rows),
                                          out.data_ptr(), N, row_start.data_ptr(), row_count.data_ptr(), _ptr(k_count),
                                          E, int(max_rows), int(N), int(K), _DT[dtype], _DT[out_dtype], _stream()),
          "ats_grouped_gemm_nt")
    return out


def grouped_gemm_nn_supported(E: int, max_rows: int, N: int, K: int, ldb: int, dtype: torch.dtype) -> bool:
    """Whether grouped_gemm_nn has a kernel for these sizes (bfloat16, prefill-sized groups)."""
    if dtype not in _DT:
        return False
    return bool(_lib.load().ats_grouped_gemm_nn_supported(int(E), int(max_rows), int(N), int(K), int(ldb), _DT[dtype]))


def grouped_gemm_nn(b_ptrs: torch.Tensor, ldb: int, row_start: torch.Tensor, row_count: torch.Tensor, n_rows_out: int,
                    max_rows: int, N: int, K: int, a: torch.Tensor, a_rows: Optional[torch.Tensor] = None,
                    a_row_div: int = 1, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[row_start[e]+m, :N] = A_e[m, :K] @ B_e[:K, :N] with B_e = b_ptrs[e] stored [K, ldb] (see
    ats_grouped_gemm_nn): the data gradient of a linear layer against the weights as the forward holds them."""
    _need_gpu(a, b_ptrs, row_start, row_count, a_rows)
    a = _rows_2d(a, "grouped_gemm_nn")
    out_dtype = a.dtype if out_dtype is None else out_dtype
    E = b_ptrs.numel()
    out = torch.empty(n_rows_out, N, dtype=out_dtype, device=b_ptrs.device)
    check(_lib.load().ats_grouped_gemm_nn(a.data_ptr(), int(a.stride(0)), int(a.shape[0]), _ptr(a_rows), int(a_row_div),
                                          b_ptrs.data_ptr(), int(ldb), out.data_ptr(), N, row_start.data_ptr(),
                                          row_count.data_ptr(), E, int(max_rows), int(N), int(K), _DT[a.dtype],
                                          _DT[out_dtype], _stream()),
          "ats_grouped_gemm_nn")
    return out


# --------------------------------------------------------------------------- attention
def _key_bias(key_bias, B: int, Lk: int, q: torch.Tensor, who: str):
    if key_bias is None:
        return None
    if key_bias.shape != (B, Lk) or key_bias.dtype != torch.float32 or key_bias.device != q.device:
        raise AtsError(f"{who}: key_bias must be float32 [batch, keys] = [{B}, {Lk}] on the inputs' device")
    return key_bias.contiguous()


def _pair_bias(pair_bias, B: int, Hq: int, L: int, Lk: int, q: torch.Tensor, who: str):
    """Checks a pair bias, float32 [batch or 1, queries, keys] or [batch or 1, heads or 1, queries, keys], and
    returns it as a contiguous 4-D tensor with its batch and head strides in floats (0 where it is shared)."""
    if pair_bias.dim() == 3:
        pair_bias = pair_bias[:, None]
    if pair_bias.dim() != 4 or pair_bias.shape[0] not in (1, B) or pair_bias.shape[1] not in (1, Hq) \
            or tuple(pair_bias.shape[2:]) != (L, Lk) or pair_bias.dtype != torch.float32 or pair_bias.device != q.device:
        raise AtsError(f"{who}: pair_bias must be float32 [batch or 1, (heads or 1,) queries, keys] = "
                       f"[{B}, {Hq}, {L}, {Lk}] on the inputs' device")
    pair_bias = pair_bias.contiguous()
    heads = pair_bias.shape[1]
    return pair_bias, (0 if pair_bias.shape[0] == 1 else heads * L * Lk), (0 if heads == 1 else L * Lk)


def _attention_extras(key_bias, pair_bias, dropout_p: float, B: int, Hq: int, L: int, Lk: int, q: torch.Tensor, who: str):
    """Arguments of the extended entry points.  Returns (key_bias, pair_bias, batch stride, head stride): with a
    pair bias or dropout a per-key bias is folded into the pair bias (the kernels take one or the other)."""
    key_bias = _key_bias(key_bias, B, Lk, q, who)
    if not 0.0 <= dropout_p < 1.0:
        raise AtsError(f"{who}: dropout_p {dropout_p} must be in [0, 1)")
    sb = sh = 0
    if pair_bias is not None:
        pair_bias, sb, sh = _pair_bias(pair_bias, B, Hq, L, Lk, q, who)
        if key_bias is not None:
            pair_bias, sb, sh = _pair_bias(pair_bias + key_bias[:, None, None, :], B, Hq, L, Lk, q, who)
            key_bias = None
    elif dropout_p > 0.0 and key_bias is not None:
        pair_bias, sb, sh = key_bias[:, None, None, :].expand(B, 1, L, Lk).contiguous(), L * Lk, 0
        key_bias = None
    return key_bias, pair_bias, sb, sh


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None,
                     return_lse: bool = False, key_bias: Optional[torch.Tensor] = None, split_keys: bool = True,
                     pair_bias: Optional[torch.Tensor] = None, dropout_p: float = 0.0, dropout_seed: int = 0):
    """Causal grouped-query attention.  q [B,Hq,L,D]; k [B,Hkv,Lk,D] with a head's rows one after the other
    and any batch/head strides (e.g. a view of a larger cache buffer); v [B,Hkv,Lk,D] in any batch/head/position
    strides (e.g. a view of a fused projection output); bf16, D 64 or 128, Lk >= L.
    With Lk > L the leading Lk - L keys are a cache: query i sits at position i + Lk - L.
    key_bias [B, Lk] float32 (optional) is added to the scaled scores of a key for every query and head;
    (1 - attention_mask) * -1e4 is the reference's padding mask (MS/core/model.py:819-824).
    pair_bias [B or 1, L, Lk] or [B or 1, Hq or 1, L, Lk] float32 (optional) is added to the scaled scores of
    a (query, key) pair, for every head or per head: (1 - mask) * -1e4 for the reference's 4-D masks (same lines).
    dropout_p > 0 drops attention weights (model.py:831-833) by a hash of (dropout_seed, batch, head, query,
    key); causal_attention_bwd given the same seed sees the same mask.
    split_keys=False keeps the single-pass kernel where few rows against many keys would otherwise be cut
    into key ranges.  Returns out [B, L, Hq*D] (and lse [B,Hq,L] float32 if asked)."""
    _need_gpu(q, k, v)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or q.dtype != torch.bfloat16 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise AtsError("causal_attention: q, k, v must be 4-D bfloat16 tensors [batch, heads, seq, head_dim]")
    B, Hq, L, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    if k.shape != (B, Hkv, Lk, D) or v.shape != (B, Hkv, Lk, D) or Hq % Hkv != 0 or Lk < L:
        raise AtsError(f"causal_attention: shapes q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    q = q.contiguous()
    if k.stride(3) != 1 or k.stride(2) != D or k.stride(0) % 8 or k.stride(1) % 8 or k.data_ptr() % 16:
        k = k.contiguous()        # rows of a head must follow one another; batch and head strides are free
    key_bias, pair_bias, pair_sb, pair_sh = _attention_extras(key_bias, pair_bias, dropout_p, B, Hq, L, Lk, q,
                                                              "causal_attention")
    if v.stride(3) != 1 or any(st % 8 for st in v.stride()[:3]) or v.stride(2) < D or v.data_ptr() % 16:
        v = v.contiguous()
    lib = _lib.load()
    out = torch.empty(B, L, Hq * D, dtype=q.dtype, device=q.device)
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=q.device) if return_lse else None
    # decoding a few sequences: scratch for the partial results of key ranges that run side by side
    ws_bytes = lib.ats_attention_fwd_workspace(B, Hq, Hkv, L, Lk, D) if split_keys else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    check(lib.ats_attention_fwd_ex(q.data_ptr(), k.data_ptr(), k.stride(0), k.stride(1), v.data_ptr(), v.stride(0),
                                   v.stride(2), v.stride(1), _ptr(key_bias), _ptr(pair_bias), pair_sb, pair_sh,
                                   float(dropout_p), int(dropout_seed) & 0xFFFFFFFFFFFFFFFF, out.data_ptr(), _ptr(lse),
                                   B, Hq, Hkv, L, Lk, D, float(D ** -0.5 if scale is None else scale), _ptr(ws),
                                   ws_bytes, _stream()),
          "ats_attention_fwd_ex")
    return (out, lse) if return_lse else out


def causal_attention_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
                         dout: torch.Tensor, scale: Optional[float] = None, key_bias: Optional[torch.Tensor] = None,
                         pair_bias: Optional[torch.Tensor] = None, dropout_p: float = 0.0, dropout_seed: int = 0):
    """Gradients of causal_attention: q [B,Hq,L,D], k, v [B,Hkv,Lk,D], out, dout [B,L,Hq*D], lse [B,Hq,L],
    key_bias, pair_bias, dropout_p and dropout_seed as in the forward.  Returns (dq, dk, dv) shaped like q, k, v."""
    _need_gpu(q, k, v, out, lse, dout)
    B, Hq, L, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    if (q.dtype != torch.bfloat16 or k.shape != (B, Hkv, Lk, D) or v.shape != k.shape or out.shape != (B, L, Hq * D)
            or dout.shape != out.shape or lse.shape != (B, Hq, L) or lse.dtype != torch.float32):
        raise AtsError("causal_attention_bwd: shapes or dtypes do not match the forward's")
    q, k, v, out = q.contiguous(), k.contiguous(), v.contiguous(), out.contiguous()
    dout = dout.to(q.dtype).contiguous()
    lse = lse.contiguous()
    key_bias, pair_bias, pair_sb, pair_sh = _attention_extras(key_bias, pair_bias, dropout_p, B, Hq, L, Lk, q,
                                                              "causal_attention_bwd")
    lib = _lib.load()
    # delta = rowsum(dO * O) is formed inside the dQ kernel and handed to the dK/dV kernel through this buffer
    delta = torch.empty(B, Hq, L, dtype=torch.float32, device=q.device)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    check(lib.ats_attention_bwd_out(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(),
                                    lse.data_ptr(), delta.data_ptr(), _ptr(key_bias), _ptr(pair_bias), pair_sb, pair_sh,
                                    float(dropout_p), int(dropout_seed) & 0xFFFFFFFFFFFFFFFF, dq.data_ptr(), dk.data_ptr(),
                                    dv.data_ptr(), B, Hq, Hkv, L, Lk, D, float(D ** -0.5 if scale is None else scale),
                                    _stream()),
          "ats_attention_bwd_out")
    return dq, dk, dv


# --------------------------------------------------------------------------- float32 attention
def _ptr_table(t: torch.Tensor, index: torch.Tensor, stride_elems: int) -> torch.Tensor:
    """Device table of addresses t.data_ptr() + index * stride_elems * itemsize (no host round trip)."""
    return index.to(torch.int64) * (stride_elems * t.element_size()) + t.data_ptr()


def _transpose_to(src: torch.Tensor, src_index: torch.Tensor, dst: torch.Tensor, dst_index: torch.Tensor, R: int, C: int):
    """Matrix src_index[n] ([R, C] contiguous inside src) -> matrix dst_index[n] ([C, R] inside dst)."""
    n = src_index.numel()
    in_tab, out_tab = _ptr_table(src, src_index, R * C), _ptr_table(dst, dst_index, R * C)   # both alive at the launch
    check(_lib.load().ats_transpose_batched(in_tab.data_ptr(), out_tab.data_ptr(), n, R, C, _tag(src), 1, _stream()),
          "ats_transpose_batched")


def _pad_rows(t: torch.Tensor, rows: int) -> torch.Tensor:
    """[..., r, D] -> [..., rows, D] contiguous, zero rows appended."""
    if t.shape[-2] == rows:
        return t.contiguous()
    out = t.new_zeros(*t.shape[:-2], rows, t.shape[-1])
    out[..., :t.shape[-2], :] = t
    return out


def _f32_groups(B: int, Hq: int, Hkv: int, dev):
    e = torch.arange(B * Hq, device=dev)
    kv_of = (e // Hq) * Hkv + (e % Hq) // (Hq // Hkv)            # the (batch, kv head) matrix of group (batch, q head)
    return e, kv_of


def attention_f32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None,
                  key_bias: Optional[torch.Tensor] = None, pair_bias: Optional[torch.Tensor] = None,
                  dropout_p: float = 0.0, dropout_seed: int = 0, return_weights: bool = False):
    """Causal grouped-query attention on float32 tensors the way the reference's _standard_attention runs it
    (MS/core/model.py:807-839): the scores of every (batch, head) are materialised by a grouped product
    (float32 MFMA kernels), softmaxed in place (ats_attention_softmax_f32: scale, causal fill, masks, dropout)
    and multiplied with V by a second grouped product.  q [B,Hq,L,D], k, v [B,Hkv,Lk,D], D a multiple of 4;
    key_bias / pair_bias / dropout as in causal_attention.  Returns out [B, L, Hq*D]; with return_weights also
    the state the backward needs (padded weights before and after dropout)."""
    _need_gpu(q, k, v)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or q.dtype != torch.float32 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise AtsError("attention_f32: q, k, v must be 4-D float32 tensors [batch, heads, seq, head_dim]")
    B, Hq, L, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    if k.shape != (B, Hkv, Lk, D) or v.shape != (B, Hkv, Lk, D) or Hq % Hkv != 0 or Lk < L or D % 4 or B * Hq > 4096:
        raise AtsError(f"attention_f32: shapes q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} "
                       "(head_dim a multiple of 4, at most 4096 (batch, head) pairs)")
    key_bias = _key_bias(key_bias, B, Lk, q, "attention_f32")
    if not 0.0 <= dropout_p < 1.0:
        raise AtsError(f"attention_f32: dropout_p {dropout_p} must be in [0, 1)")
    pair_sb = pair_sh = 0
    if pair_bias is not None:
        pair_bias, pair_sb, pair_sh = _pair_bias(pair_bias, B, Hq, L, Lk, q, "attention_f32")
    scale = float(D ** -0.5 if scale is None else scale)
    dev = q.device
    lib = _lib.load()
    Lp, Lkp = (L + 3) // 4 * 4, (Lk + 3) // 4 * 4
    E = B * Hq
    qp, kp, vp = _pad_rows(q, Lp), _pad_rows(k, Lkp), _pad_rows(v, Lkp)
    e, kv_of = _f32_groups(B, Hq, Hkv, dev)
    row_start = (e * Lp).to(torch.int32)
    row_count = torch.full((E,), Lp, dtype=torch.int32, device=dev)
    # scores[e] = q[e] . k[kv_of[e]]^T
    w = grouped_gemm_nt(_ptr_table(kp, kv_of, Lkp * D), D, Lkp, row_start, row_count, E * Lp, E * Lp, Lkp, D,
                        a=qp.view(E * Lp, D))
    w_drop = torch.empty_like(w) if dropout_p > 0 else None
    check(lib.ats_attention_softmax_f32(w.data_ptr(), _ptr(w_drop), B, Hq, L, Lp, Lk, Lkp, scale, _ptr(key_bias),
                                        _ptr(pair_bias), pair_sb, pair_sh, float(dropout_p),
                                        int(dropout_seed) & 0xFFFFFFFFFFFFFFFF, _stream()), "ats_attention_softmax_f32")
    # out[e] = weights[e] . v[kv_of[e]]  (NT product against v^T)
    vT = torch.empty(B * Hkv, D, Lkp, dtype=q.dtype, device=dev)
    every_kv = torch.arange(B * Hkv, device=dev)
    _transpose_to(vp, every_kv, vT, every_kv, Lkp, D)
    used = w_drop if w_drop is not None else w
    o = grouped_gemm_nt(_ptr_table(vT, kv_of, D * Lkp), Lkp, D, row_start, row_count, E * Lp, E * Lp, D, Lkp, a=used)
    out = o.view(B, Hq, Lp, D)[:, :, :L].transpose(1, 2).reshape(B, L, Hq * D)
    if return_weights:
        return out, (w, w_drop, qp, kp, vp)
    return out


def attention_f32_bwd(state, dout: torch.Tensor, B: int, Hq: int, Hkv: int, L: int, Lk: int, D: int,
                      scale: Optional[float] = None, dropout_p: float = 0.0, dropout_seed: int = 0):
    """Gradients of attention_f32 from the state its forward returned: dV = P'^T.dO, dP' = dO.V^T, dS through
    ats_attention_softmax_bwd_f32, dQ = dS.K, dK = dS^T.Q, each a grouped float32 product (transposed operands
    are written by ats_transpose_batched; the query heads of a kv head are summed by ats_sum_partials).
    Returns (dq [B,Hq,L,D], dk, dv [B,Hkv,Lk,D])."""
    w, w_drop, qp, kp, vp = state
    _need_gpu(w, dout)
    dev = w.device
    lib = _lib.load()
    scale = float(D ** -0.5 if scale is None else scale)
    Lp, Lkp = qp.shape[2], kp.shape[2]
    E, rep = B * Hq, Hq // Hkv
    e, kv_of = _f32_groups(B, Hq, Hkv, dev)
    row_start = (e * Lp).to(torch.int32)
    row_count = torch.full((E,), Lp, dtype=torch.int32, device=dev)
    do = _pad_rows(dout.to(torch.float32).view(B, L, Hq, D).permute(0, 2, 1, 3), Lp)          # [B, Hq, Lp, D]
    # dP' = dO . V^T, then in place to dS (gradient of the raw scores)
    ds = grouped_gemm_nt(_ptr_table(vp, kv_of, Lkp * D), D, Lkp, row_start, row_count, E * Lp, E * Lp, Lkp, D,
                         a=do.view(E * Lp, D))
    check(lib.ats_attention_softmax_bwd_f32(w.data_ptr(), ds.data_ptr(), B, Hq, L, Lp, Lk, Lkp, scale, float(dropout_p),
                                            int(dropout_seed) & 0xFFFFFFFFFFFFFFFF, _stream()),
          "ats_attention_softmax_bwd_f32")
    # dQ = dS . K  (NT product against K^T)
    every_kv = torch.arange(B * Hkv, device=dev)
    kT = torch.empty(B * Hkv, D, Lkp, dtype=w.dtype, device=dev)
    _transpose_to(kp, every_kv, kT, every_kv, Lkp, D)
    dq = grouped_gemm_nt(_ptr_table(kT, kv_of, D * Lkp), Lkp, D, row_start, row_count, E * Lp, E * Lp, D, Lkp, a=ds)
    dq = dq.view(B, Hq, Lp, D)[:, :, :L].contiguous()
    # dV and dK: per query head a product over the queries, written so that the `rep` heads of a kv head are
    # `rep` slices of one buffer: group (b, hq) goes to slot (hq % rep) * (B * Hkv) + its kv matrix
    slot = (e % Hq % rep) * (B * Hkv) + kv_of
    slot_count = torch.full((E,), Lkp, dtype=torch.int32, device=dev)
    order = torch.empty(E, dtype=torch.int64, device=dev)
    order[slot] = e                                   # group that owns slot s
    doT = torch.empty(E, D, Lp, dtype=w.dtype, device=dev)
    _transpose_to(do, e, doT, e, Lp, D)
    qT = torch.empty(E, D, Lp, dtype=w.dtype, device=dev)
    _transpose_to(qp, e, qT, e, Lp, D)

    def over_queries(mat: torch.Tensor, rhsT: torch.Tensor) -> torch.Tensor:
        """sum over the heads of a kv group of mat[e]^T . rhs[e]: mat [E*Lp, Lkp], rhsT [E, D, Lp] -> [B,Hkv,Lkp,D]."""
        matT = torch.empty(E, Lkp, Lp, dtype=w.dtype, device=dev)
        _transpose_to(mat, e, matT, slot, Lp, Lkp)
        # b_ptrs and row tables are read in group order 0..E-1 = slot order here
        parts = grouped_gemm_nt(_ptr_table(rhsT, order, D * Lp), Lp, D, (torch.arange(E, device=dev) * Lkp).to(torch.int32),
                                slot_count, E * Lkp, E * Lkp, D, Lp, a=matT.view(E * Lkp, Lp))
        parts = parts.view(rep, B * Hkv * Lkp * D)
        total = sum_partials(parts, torch.float32) if rep > 1 else parts[0]
        return total.view(B, Hkv, Lkp, D)[:, :, :Lk].contiguous()

    dv = over_queries(w_drop if w_drop is not None else w, doT)
    dk = over_queries(ds, qT)
    return dq, dk, dv


_single_group_cache: dict = {}


def _single_group(T: int, device: torch.device):
    """row_start = [0], row_count = [T] of a one-group GEMM, kept per (T, device): two fill launches
    per call are a visible share of a small projection."""
    key = (T, device)
    hit = _single_group_cache.get(key)
    if hit is None:
        if len(_single_group_cache) > 64:
            _single_group_cache.clear()
        hit = (torch.zeros(1, dtype=torch.int32, device=device), torch.full((1,), T, dtype=torch.int32, device=device))
        _single_group_cache[key] = hit
    return hit


def linear_nt(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x [T, K] @ weight[N, K]^T through the grouped GEMM kernels with a single group."""
    _need_gpu(x, weight)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1] or x.dtype != weight.dtype:
        raise AtsError("linear_nt: x [T,K], weight [N,K], same dtype")
    T, K = x.shape
    N = weight.shape[0]
    x, weight = x.contiguous(), weight.contiguous()
    start, count = _single_group(T, x.device)
    splits = down_k_splits(1, T, N, K, x.dtype) if K % 8 == 0 and N % 8 == 0 else 1
    if splits > 1:      # a few rows against a whole weight matrix: slices of K keep every CU streaming
        return sum_partials(grouped_down_splitk(x, weight_pointer_table([weight]), start, count, T, N, K, splits),
                            x.dtype)
    return grouped_gemm_nt(weight_pointer_table([weight]), K, N, start, count, T, T, N, K, a=x)
