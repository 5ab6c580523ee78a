"""Writes the golden fixtures of this directory from the CPU oracle (oracle/sparse_layer_oracle.py).

    python tests/golden/make_fixtures.py

The reference repository holds no numeric fixtures for this path (its tests assert shapes and
finiteness only) and its Python was not imported: every vector here comes from the oracle, whose
functions are pinned independently by tests/test_oracle_pinning.py.  The fixtures freeze those
results so that (a) a later change of the oracle or of torch is noticed and (b) the GPU tests have
fixed integer artefacts (indices, token maps, dropped sets) to compare with bit for bit.
Inputs are regenerated from seeds by adaptivetrainingsystem_amd.workloads; only outputs are stored.
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from adaptivetrainingsystem_amd import workloads as W  # noqa: E402
from oracle import sparse_layer_oracle as O  # noqa: E402


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(np.ascontiguousarray(t.numpy()).tobytes()).hexdigest()


def tiny_cases():
    """Full tensors for tiny layers (T <= 16) with drops, all in float32."""
    out = {}
    for name, (T, H, I, E, k, cf, routing) in {
        "t16_e4_k2_cf0.75": (16, 8, 12, 4, 2, 0.75, "softmax_topk"),
        "t12_e8_k3_cf1.0": (12, 8, 12, 8, 3, 1.0, "topk_softmax"),
        "t9_e4_k1_cf1.25": (9, 8, 12, 4, 1, 1.25, "softmax_topk"),
    }.items():
        g = torch.Generator().manual_seed(1234 + T)
        x = torch.randn(T, H, generator=g)
        wg = torch.randn(E, H, generator=g) * 0.5
        wgu = [torch.randn(2 * I, H, generator=g) * 0.2 for _ in range(E)]
        wd = [torch.randn(H, I, generator=g) * 0.2 for _ in range(E)]
        r = O.moe_forward_capacity(x, wg, wgu, wd, k=k, capacity_factor=cf, routing=routing, literal_loops=True)
        out[name] = {
            "shape": [T, H, I, E, k], "capacity_factor": cf, "routing": routing, "seed": 1234 + T,
            "capacity": r["capacity"], "indices": r["indices"].tolist(), "weights": r["weights"].tolist(),
            "token_map": r["token_map"].tolist(), "slot": r["slot"].tolist(), "hist": r["hist"].tolist(),
            "kept": r["kept"].tolist(), "aux": float(r["aux"]), "out": r["out"].tolist(),
        }
    return out


def config1():
    """Benchmark config 1 at full size (512 tokens, H 512, 8 experts top-2, I 1408, cf 1.25, float32,
    pre-norm): integer artefacts in full, floats as a strided sample plus a digest."""
    w = W.make_moe_workload("c1_cpu_reference", device="cpu")
    xn = O.rmsnorm(w.x, w.norm_weight, 1e-6)
    r = O.moe_forward_capacity(xn, w.gate, w.gate_up, w.down, k=2, capacity_factor=1.25)
    flat = r["out"].reshape(-1, 512)
    return {
        "capacity": r["capacity"], "indices": r["indices"].tolist(), "hist": r["hist"].tolist(),
        "kept": r["kept"].tolist(), "dropped": (r["slot"] < 0).nonzero().flatten().tolist(),
        "token_map": r["token_map"].tolist(), "aux": float(r["aux"]),
        "out_sample_rows": list(range(0, 512, 37)), "out_sample_cols": list(range(0, 512, 61)),
        "out_sample": flat[0:512:37, 0:512:61].tolist(), "out_abs_max": float(flat.abs().max()),
        "out_sha256_f32": sha(flat), "xn_sha256_f32": sha(xn),
    }


def rope_rows():
    cos, sin = O.rope_table(8192, 128, 10000.0)
    rows = [0, 1, 2047, 8191]
    return {"dim": 128, "theta": 10000.0, "rows": rows, "cos": cos[rows, :64].tolist(), "sin": sin[rows, :64].tolist()}


def main():
    fixtures = {"tiny": tiny_cases(), "config1": config1(), "rope_table": rope_rows(),
                "torch_version": torch.__version__}
    path = os.path.join(HERE, "sparse_layer_fixtures.json")
    with open(path, "w") as f:
        json.dump(fixtures, f)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
