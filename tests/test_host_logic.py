"""CPU-side checks: the C-ABI library loads and exports every declared symbol, the tile
schedule covers every tile exactly once, host-side integer logic, error behaviour without a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "ats_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ats_[a-z0-9_]+|[a-z_]+_launcher)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from adaptivetrainingsystem_amd import _lib
    assert _lib.is_built(), "build the library first: python -m adaptivetrainingsystem_amd.build"
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
        assert n in _lib._SIGNATURES, f"{n} has no ctypes signature"
    assert lib.ats_version() >= 100
    assert set(_lib._SIGNATURES) == set(names)


def test_reference_launcher_names_are_exported_and_never_exit():
    """The four launcher names the reference's ctypes loader binds (cuda_opt_wrapper.py:98-108, 156-169,
    219-228, 337-344) exist with void returns; a bad argument leaves a status and a text, not an exit()."""
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    raw = ctypes.CDLL(_lib.LIB_PATH)        # as the reference binds it: no argtypes, explicit ctypes wrappers
    for n in ("rms_norm_launcher", "rope_precompute_launcher", "rope_apply_launcher", "swiglu_launcher", "swiglu_fused_launcher",
              "fused_cross_entropy_accuracy_launcher", "fused_grad_clip_launcher"):      # training/cuda_kernels.py:60-78
        assert hasattr(raw, n), n
    raw.rms_norm_launcher(ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_int(4), ctypes.c_int(0),
                          ctypes.c_float(1e-6), ctypes.c_void_p(0))
    assert lib.ats_legacy_last_status() == -1 and b"hidden" in lib.ats_last_error_string()
    raw.rope_apply_launcher(ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_void_p(0),
                            ctypes.c_int(1), ctypes.c_int(1), ctypes.c_int(4), ctypes.c_int(7), ctypes.c_int(0),
                            ctypes.c_void_p(0))
    assert lib.ats_legacy_last_status() == -1           # odd head_dim
    raw.swiglu_launcher(ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_int(0), ctypes.c_int(16),
                        ctypes.c_void_p(0))
    assert lib.ats_legacy_last_status() == 0            # nothing to do is not an error
    raw.rope_precompute_launcher(ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_int(8), ctypes.c_int(16),
                                 ctypes.c_float(10000.0), ctypes.c_void_p(0))
    assert lib.ats_legacy_last_status() == -1 and b"null" in lib.ats_last_error_string()


def test_argument_errors_return_codes_not_exits():
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    # invalid arguments are rejected on the host before any device work
    assert lib.ats_rmsnorm_fwd(None, None, None, 4, 0, 1e-6, 0, 0, None) == -1
    assert b"hidden" in lib.ats_last_error_string()
    assert lib.ats_rmsnorm_fwd(None, None, None, 4, 8, 1e-6, 7, 0, None) != 0
    assert lib.ats_route_topk(None, 4, 8, 9, 1.0, 0, None, None, None, None, None, 0.01, None, 0, None) == -1
    assert lib.ats_dispatch_plan(None, 0, 4, 2, 5000, 3, None, None, None, None, None, None, None, None, None, 0,
                                 None) == -1
    assert lib.ats_rope_fwd(None, None, None, None, None, None, 4, 4, 1, 1, 1, 4, 7, 0, 0, 0, 0, 0, 0, 0, 0,
                            None) == -1       # odd head_dim
    assert lib.ats_select_topk_per_sequence(None, 1, 10000, 5, None, None) == -1
    # attention: head_dim outside {64, 128}, fewer keys than queries, query heads not a multiple of kv heads
    assert lib.ats_attention_fwd(None, None, 0, 0, None, 0, 96, 0, None, None, None, 1, 4, 2, 16, 16, 96, 0.1, None, 0, None) == -2
    assert b"head_dim" in lib.ats_last_error_string()
    assert lib.ats_attention_fwd(None, None, 0, 0, None, 0, 128, 0, None, None, None, 1, 4, 2, 16, 8, 128, 0.1, None, 0, None) == -1
    assert lib.ats_attention_fwd(None, None, 0, 0, None, 0, 128, 0, None, None, None, 1, 3, 2, 16, 16, 128, 0.1, None, 0, None) == -1
    assert lib.ats_attention_fwd(None, None, 0, 0, None, 0, 128, 0, None, None, None, 1, 4, 2, 16, 16, 128, 0.1, None, 0, None) == -1     # null pointers
    assert lib.ats_attention_fwd(None, None, 0, 0, None, 0, 128, 0, None, None, None, 0, 4, 2, 16, 16, 128, 0.1, None, 0, None) == 0      # empty batch
    assert lib.ats_attention_bwd(*([None] * 10), 1, 4, 2, 16, 8, 128, 0.1, None, 0, None) == -1
    assert lib.ats_attention_bwd(*([None] * 10), 1, 4, 2, 16, 16, 32, 0.1, None) == -2
    assert lib.ats_attention_delta(None, None, None, 1, 4, 16, 80, None) == -2
    assert lib.ats_attention_bwd_out(*([None] * 9), 0, 0, 0.0, 0, None, None, None, 1, 4, 2, 16, 16, 128, 0.1, None) == -1
    assert lib.ats_attention_bwd_out(*([None] * 9), 0, 0, 0.0, 0, None, None, None, 0, 4, 2, 16, 16, 128, 0.1, None) == 0
    # K slices: I must be k_splits whole slabs, and only weight-streaming sizes (<= 48 rows per expert)
    one = ctypes.c_void_p(16)
    assert lib.ats_grouped_down_splitk(one, one, one, one, one, 8, 128, 128, 4096, 14336, 3, 1, None) == -2
    assert b"slices" in lib.ats_last_error_string()
    assert lib.ats_grouped_down_splitk(one, one, one, one, one, 8, 4096, 4096, 4096, 14336, 2, 1, None) == -2   # 512 rows per expert
    assert lib.ats_grouped_down_splitk(one, one, one, one, one, 8, 128, 128, 4096, 14336, 0, 1, None) == -1
    assert lib.ats_sum_partials(one, 2, 10, one, 8, 1, None) == -1          # stride not a multiple of 4
    assert lib.ats_sum_partials(None, 2, 16, None, 0, 1, None) == 0         # nothing to add
    assert lib.ats_combine_partials(one, 2, 64, one, one, None, one, 4, 9, 64, 1, None) == -1   # k > 8
    assert lib.ats_route_topk_workspace(16384, 8) > 0
    assert lib.ats_dispatch_plan_workspace(16384, 2, 8) == (32768 // 256) * 8 * 4


@pytest.mark.parametrize("aligned", [0, 1])
@pytest.mark.parametrize("counts,BM,n_tiles,SM,SN,slices", [
    ([5120, 4000, 300, 0, 1, 256, 257, 77], 256, 112, 4, 8, 1),
    ([20, 16, 0, 3], 32, 112, 1, 32, 1),
    ([130, 90, 576, 1], 128, 11, 8, 4, 1),
    ([0, 0, 0], 128, 5, 4, 8, 1),
    ([1000] * 64, 128, 11, 4, 8, 1),
    ([384] * 70, 256, 11, 8, 4, 1),
    ([20, 16, 0, 3], 32, 32, 1, 32, 3),
    ([64, 33, 1], 64, 40, 1, 32, 2),
])
def test_tile_schedule_covers_each_tile_once(counts, BM, n_tiles, SM, SN, slices, aligned):
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    rc = np.asarray(counts, dtype=np.int32)
    E = len(counts)
    blocks = lib.ats_debug_grid_blocks(int(rc.sum()) * slices, E * slices, BM, n_tiles, SM, SN, aligned)
    assert blocks % 256 == 0
    seen = {}
    out = np.zeros(4, dtype=np.int32)
    for b in range(blocks):
        if lib.ats_debug_decode_tile(b, rc.ctypes.data, E, BM, n_tiles, SM, SN, aligned, slices, out.ctypes.data):
            key = tuple(out.tolist())
            assert key not in seen, f"tile {key} given to blocks {seen[key]} and {b}"
            seen[key] = b
    expect = {(e, mt, nt, ks) for ks in range(slices) for e in range(E) for mt in range(-(-counts[e] // BM))
              for nt in range(n_tiles)}
    assert set(seen) == expect
    # blocks of one supertile land on one XCD (ids congruent mod 8) and cover SN neighbouring n-tiles of one band:
    # SM consecutive entries of the m-tile list (group 0's tiles, then group 1's, ...; a group is an expert or one
    # K slice of it; with `aligned` every group's tile count is rounded up to a multiple of SM)
    if expect:
        per = [-(-c // BM) for c in counts] * slices
        if aligned:
            per = [-(-t // SM) * SM for t in per]
        first = np.concatenate([[0], np.cumsum(per)])
        by_xcd = {}
        for key, b in seen.items():
            by_xcd.setdefault((b % 8, (b // 8) // 32), []).append(key)
        order = []
        for (xcd, li), keys in sorted(by_xcd.items(), key=lambda kv: kv[0][1] * 8 + kv[0][0]):
            pos = {int(first[ks * E + e]) + mt for e, mt, _, ks in keys}
            assert len({q // SM for q in pos}) == 1
            assert len({k[2] // SN for k in keys}) == 1
            if aligned:
                assert len({(k[0], k[3]) for k in keys}) == 1      # one expert's weight panels per supertile
            order.append((min(pos) // SM, keys[0][2] // SN))
        # supertiles go group by group (by the group a band starts in), n-group by n-group, band by band
        owner = lambda band: int(np.searchsorted(first, band * SM, side="right") - 1)
        assert order == sorted(order, key=lambda t: (owner(t[0]), t[1], t[0]))


def test_capacity_is_python_double_arithmetic():
    from adaptivetrainingsystem_amd import ops
    assert ops.expert_capacity(512, 2, 8, 1.25) == 160
    assert ops.expert_capacity(64, 2, 8, 1.25) == 20
    assert ops.expert_capacity(16384, 2, 8, 1.25) == 5120
    assert ops.expert_capacity(4096, 6, 64, 1.5) == 576
    assert ops.expert_capacity(512, 2, 8, 1.1) == 140


def test_no_cpu_fallback_and_module_surface():
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    with pytest.raises(A.AtsError):
        A.RMSNorm(16)(torch.randn(2, 16))
    with pytest.raises(A.AtsError):
        A.apply_rotary_pos_emb(torch.randn(1, 1, 4, 8), torch.randn(1, 1, 4, 8), torch.ones(4, 8), torch.zeros(4, 8))
    layer = A.MoEFFNLayer(LayerConfig(32, 64, 4, 2))
    with pytest.raises(A.AtsError):
        layer(torch.randn(1, 3, 32))
    # parameter names and shapes that checkpoints of the reference model carry
    sd = layer.state_dict()
    assert sd["gate.weight"].shape == (4, 32)
    assert sd["experts.0.gate_up_proj.weight"].shape == (128, 32)
    assert sd["experts.3.down_proj.weight"].shape == (32, 64)
    assert set(sd) == {"gate.weight"} | {f"experts.{i}.{n}.weight" for i in range(4)
                                         for n in ("gate_up_proj", "down_proj")}
    for attr in ("num_experts", "top_k", "capacity_factor", "routing_temperature", "noise_std",
                 "load_balancing_weight", "use_cuda_ops", "get_routing_stats", "reset_routing_stats"):
        assert hasattr(layer, attr)
    assert layer.get_routing_stats() == {"error": "No routing statistics available"}
    assert A.RMSNorm(8).state_dict()["weight"].shape == (8,)
    assert list(A.RotaryEmbedding(8).state_dict()) == []           # buffers are non-persistent
    assert A.MoECUDAOps.should_use_cuda(1, 1, 1, True, False) is False
    # attention sub-layer and block: the reference's parameter names; CPU tensors are refused
    cfg = LayerConfig(64, 128, 4, 2, num_heads=4, num_kv_heads=2, seq_length=32, use_moe=True)
    att = A.GroupedQueryAttention(cfg)
    assert {k: tuple(v.shape) for k, v in att.state_dict().items()} == {
        "q_proj.weight": (64, 64), "k_proj.weight": (32, 64), "v_proj.weight": (32, 64), "o_proj.weight": (64, 64)}
    with pytest.raises(A.AtsError):
        att(torch.randn(1, 4, 64).bfloat16())
    # attention dropout (model.py:831-833) is part of the kernel path: with or without it a CPU tensor is refused
    drop = A.GroupedQueryAttention(LayerConfig(64, 128, 4, 2, num_heads=4, num_kv_heads=2, seq_length=32, dropout=0.1))
    assert drop.dropout_p == pytest.approx(0.1)
    for mode in (drop.train(), drop.eval()):
        with pytest.raises(A.AtsError, match="GPU"):
            mode(torch.randn(1, 4, 64).bfloat16())
    blk = A.TransformerBlock(cfg, layer_idx=0)
    names = set(blk.state_dict())
    assert {"input_norm.weight", "post_attn_norm.weight", "self_attn.o_proj.weight", "ffn.gate.weight",
            "ffn.experts.3.down_proj.weight"} <= names
    dense = A.TransformerBlock(LayerConfig(64, 128, 1, 1, num_heads=4, num_kv_heads=2, seq_length=32), layer_idx=0)
    assert {"ffn.gate_up_proj.weight", "ffn.down_proj.weight"} <= set(dense.state_dict())
    assert A.DenseGroupedQueryAttention is A.GroupedQueryAttention


def test_workloads_are_reproducible():
    from adaptivetrainingsystem_amd import workloads as W
    a = W.make_moe_workload("c1_cpu_reference", device="cpu")
    b = W.make_moe_workload("c1_cpu_reference", device="cpu")
    assert torch.equal(a.x, b.x) and torch.equal(a.down[7], b.down[7])
    assert a.x.shape == (2, 256, 512) and a.gate_up[0].shape == (2816, 512) and a.gate.shape == (8, 512)
    c = W.make_moe_workload("c4_prefill", device="cpu", scale_tokens=16, overrides={"hidden": 64, "intermediate": 64})
    assert torch.allclose(c.logit_bias, 1.5 * torch.log(1.0 / torch.arange(1, 9).float()))
    n = W.make_norm_rope_workload(device="cpu", batch=1, seq=8)
    assert n.q.shape == (1, 16, 8, 128) and n.k.shape == (1, 4, 8, 128) and n.norm_weight.dtype == torch.float32


def test_bench_refuses_more_than_one_gpu():
    """The path runs on one GPU: asking the benchmark for more exits with a message instead of measuring."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for argv, env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "2"})):
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *argv], capture_output=True, text=True,
                           env={**os.environ, **env}, timeout=300)
        assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""
