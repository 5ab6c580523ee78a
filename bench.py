#!/usr/bin/env python3
"""Benchmark of the sparse-layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
    (NAME_train, e.g. c4_prefill_train, times forward + backward of the same layer)

A step is one forward pass of the MoE layer (router GEMM -> softmax/top-k ->
capacity dispatch plan -> grouped gate/up GEMM + SwiGLU -> grouped down GEMM ->
weighted combine) over one batch of synthetic tokens that is already resident
in HBM.  The default workload is the prefill configuration the headline metric
is quoted on: 8 x 2048 = 16384 tokens, hidden 4096, 8 experts, top-2,
intermediate 14336, capacity factor 1.25, Zipf-skewed router logits, bf16.

Prints one JSON line: whole-job tokens/s, the roofline position of the dominant
kernel (grouped gate/up GEMM: algorithmic flops of the kept assignments over its
mean duration, measured with HIP events on the launch stream inside the timed
region) and the CPU baseline (the oracle's restatement of the reference path on
a bounded sample of the same workload, on this machine's host cores).
Everything else (per-stage times) goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0   # MI355X dense bf16
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f32": 157.3}   # MI355X dense MFMA peaks by arithmetic type
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E


def profile_traffic(workload: str, kernel: str):
    """HBM-side bytes per launch of a kernel, from the tracked hardware-counter summaries: lines
    `bench-traffic <workload> <kernel> <bytes>` in profiles/*hbm_traffic.txt (None when no summary has one)."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_traffic.txt"))):
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 4 and parts[0] == "bench-traffic" and parts[1] == workload and parts[2] == kernel:
                    return float(parts[3])
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(w, sample_tokens: int):
    """Times the oracle (CPU restatement of the reference path, float32) on the first
    `sample_tokens` tokens of the workload with the workload's own weights."""
    from oracle import sparse_layer_oracle as O
    # converted on the host: float32 copies on the GPU would be 3.8 GB of temporaries at the headline shape
    x = w.x.reshape(-1, w.hidden)[:sample_tokens].cpu().float()
    gate = w.gate.cpu().float()
    gu = [t.cpu().float() for t in w.gate_up]
    dn = [t.cpu().float() for t in w.down]
    bias = None if w.logit_bias is None else w.logit_bias.cpu().float()
    kw = dict(k=w.top_k, capacity_factor=w.capacity_factor, routing=w.routing, logit_bias=bias)
    O.moe_forward_capacity(x[:64], gate, gu, dn, **kw)   # touch the weights once
    t0 = time.perf_counter()
    r = O.moe_forward_capacity(x, gate, gu, dn, **kw)
    dt = time.perf_counter() - t0
    kept = int(r["kept"].sum())
    out = {"value": sample_tokens / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"first {sample_tokens} tokens of the workload, same weights, float32, one pass "
                     f"({dt:.2f} s, {kept} kept assignments)"}
    if w.name == "c1_cpu_reference":
        # the reference's own per-token / per-expert Python loops (moe_cuda_wrapper.py:316-324, 343-357), once
        t0 = time.perf_counter()
        O.moe_forward_capacity(x, gate, gu, dn, literal_loops=True, **kw)
        out["literal_loops_c1"] = sample_tokens / (time.perf_counter() - t0)
    return out


def gemm_calibration(w, moe, plan, kept: int, gu_ms: float):
    """What bounds the grouped GEMM on this machine, measured in the same process: MFMA-only loops with zero
    and with random operands (the gap is the board's power limit), this library's gate/up kernel on all-zero
    operands with the same row plan (its schedule without the power limit), and the vendor library's dense
    bf16 matmul of the same M x N x K."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd.profiling import StageTimer, calibrate_mfma
    H, I, E, k = w.hidden, w.intermediate, w.num_experts, w.top_k
    out = {"mfma_only": {}}
    for shape in ("16x16x32", "32x32x16"):
        for rnd in (False, True):
            r = calibrate_mfma(shape, rnd)
            out["mfma_only"][f"{shape}_{'random' if rnd else 'zero'}_operands"] = {
                "tflops": round(r["tflops"], 1), "core_clock_mhz": round(r["core_clock_mhz"])}
    rows = min(plan["row_of"].numel(), E * plan["capacity"])
    # the same launch on zero operands: the tile schedule, loads and barriers without operand-dependent power
    x0 = torch.zeros(w.tokens, H, dtype=w.dtype, device=w.x.device)
    wz = [torch.zeros(2 * I, H, dtype=w.dtype, device=w.x.device) for _ in range(E)]
    ptrs = ops.weight_pointer_table(wz)
    timer = StageTimer()
    for i in range(6):
        with timer.range("z" if i >= 2 else "warm"):
            ops.grouped_gateup_swiglu(x0, ptrs, plan["offsets"], plan["kept"], rows, rows, H, I,
                                      a_rows=plan["row_src"], a_row_div=k)
    z_ms = timer.summary()["z"]["mean_ms"]
    del wz, ptrs, x0
    out["gateup_zero_operands"] = {"tflops": round(4.0 * H * I * kept / (z_ms * 1e-3) / 1e12, 1), "ms": round(z_ms, 4)}
    out["gateup_random_operands"] = {"tflops": round(4.0 * H * I * kept / (gu_ms * 1e-3) / 1e12, 1), "ms": round(gu_ms, 4)}
    # vendor BLAS, dense, same M x N x K as the grouped launch (M = kept rows)
    a = torch.randn(kept, H, device=w.x.device).to(w.dtype)
    ref = {}
    for key, wt, flop in (("gateup_shape", w.gate_up[0], 4.0 * H * I * kept), ("down_shape", None, 2.0 * H * I * kept)):
        if wt is None:
            a = torch.randn(kept, I, device=w.x.device).to(w.dtype) * 0.1
            wt = w.down[0]
        timer = StageTimer()
        for i in range(8):
            with timer.range("m" if i >= 3 else "warm"):
                torch.matmul(a, wt.t())
        ms = timer.summary()["m"]["mean_ms"]
        ref[key] = {"m_n_k": [kept, wt.shape[0], wt.shape[1]], "tflops": round(flop / (ms * 1e-3) / 1e12, 1),
                    "ms": round(ms, 4)}
    out["gemm_reference"] = {"what": "torch.matmul (vendor BLAS) on one dense bf16 problem of the grouped launch's "
                                     "M x N x K, random operands, same process", **ref}
    return out


def stream_read_yardstick(nbytes, dev, reps=10):
    """What a kernel that only reads `nbytes`, front to back, reaches (the library's plain streaming read)."""
    from adaptivetrainingsystem_amd import profiling
    nbytes -= nbytes % 16
    buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).random_(0, 1 << 30)
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    for _ in range(2):
        profiling.stream_read(buf, sink)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(reps):
        profiling.stream_read(buf, sink)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / reps
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"what": "this library's plain streaming read kernel (16 bytes per lane, eight loads in flight per lane, "
                    "non-temporal) over as many bytes as the gate/up launch streams: what a kernel that only reads "
                    "them reaches", "achieved": gbs, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "ms": ms}


def run_moe(args):
    from adaptivetrainingsystem_amd import workloads as W
    from adaptivetrainingsystem_amd.profiling import StageTimer

    dev = torch.device("cuda:0")
    name = args.workload
    # CPU-seeded generator where the tensors are small enough to draw on the host in seconds
    gen_device = "cpu" if name in ("c1_cpu_reference", "c3_decode") else "cuda"
    w = W.make_moe_workload(name, device=dev, gen_device=gen_device)
    layer = W.build_layer(w, "fcfs")
    moe = layer.moe if hasattr(layer, "moe") else layer
    T_in = w.tokens
    log(f"workload {name}: tokens={T_in} H={w.hidden} E={w.num_experts} k={w.top_k} I={w.intermediate} "
        f"cf={w.capacity_factor} dtype={w.dtype} (inputs drawn on {gen_device})")

    with torch.no_grad():
        for _ in range(args.warmup):
            layer(w.x)
        torch.cuda.synchronize()
        # timed region: only the dominant kernel is bracketed by events (a pair costs the stream ~10 us)
        timer = StageTimer(only=("gateup_swiglu",))
        moe.stage_timer = timer
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out, aux = layer(w.x)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # afterwards, untimed: the same steps with every stage bracketed, for the stage table
        full = StageTimer()
        moe.stage_timer = full
        for _ in range(args.steps):
            layer(w.x)
        stages = full.summary()
        moe.stage_timer = None
    stages["gateup_swiglu"] = timer.summary()["gateup_swiglu"]      # the figure of the timed region
    plan = moe.last_plan
    kept = int(plan["kept"].sum().item())
    hist = plan["hist"].cpu().tolist()
    T_moe = plan["row_of"].numel() // w.top_k
    dropped = T_moe * w.top_k - kept
    for s, v in stages.items():
        log(f"  stage {s:14s} mean {v['mean_ms']:9.4f} ms  median {v['median_ms']:9.4f}  p10 {v['p10_ms']:9.4f}  "
            f"p90 {v['p90_ms']:9.4f}  min {v['min_ms']:9.4f} ms  ({v['calls']} calls)")
    log(f"  kept assignments {kept} of {T_moe * w.top_k} (dropped {dropped}); capacity {plan['capacity']}; hist {hist}")
    log(f"  finite output: {bool(torch.isfinite(out.float()).all())}, aux {float(aux):.6f}")

    H, I = w.hidden, w.intermediate
    dtype_name = "bf16" if w.dtype == torch.bfloat16 else "f32"
    gu_ms = stages["gateup_swiglu"]["mean_ms"]
    gu_flops = 4.0 * H * I * kept
    achieved = gu_flops / (gu_ms * 1e-3) / 1e12
    dn_ms = stages["down"]["mean_ms"]
    log(f"  gate/up GEMM {achieved:.1f} TFLOP/s; down GEMM {2.0 * H * I * kept / (dn_ms * 1e-3) / 1e12:.1f} TFLOP/s")
    ms_per_step = dt / args.steps * 1e3
    es = 2 if w.dtype == torch.bfloat16 else 4
    mfma_bound = kept / w.num_experts > 48
    if not mfma_bound:
        # decode-sized groups: the gate/up kernel streams the weights of the active experts once
        active = sum(1 for c in plan["kept"].cpu().tolist() if c > 0)
        gu_bytes = active * 2.0 * I * H * es + kept * (H + I) * es
        gbs = gu_bytes / (gu_ms * 1e-3) / 1e9
        roofline = {"kernel": "grouped gate/up GEMM + SwiGLU (weight streaming)", "bound": "hbm", "achieved": gbs,
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                    "traffic": profile_traffic(name, "gateup")}
        stream_read_reference = stream_read_yardstick(int(gu_bytes), dev)
        stream_read_reference["gateup_vs_read"] = gbs / stream_read_reference["achieved"]
        log(f"  plain streaming read of the same {gu_bytes / 1e9:.2f} GB: {stream_read_reference['achieved']:.0f} GB/s; "
            f"the gate/up kernel reaches {stream_read_reference['gateup_vs_read']:.3f} of it")
    else:
        peak = PEAK_MFMA_TFLOPS[dtype_name]
        roofline = {"kernel": "grouped gate/up GEMM + SwiGLU", "bound": "mfma", "achieved": achieved,
                    "peak": peak, "unit": "TFLOP/s", "frac": achieved / peak,
                    "traffic": profile_traffic(name, "gateup")}
    result = {
        "metric": f"MoE-layer tokens/s (h{H}, {w.num_experts}e top-{w.top_k}, {dtype_name}) + % of MFMA/HBM roofline",
        "value": T_in * args.steps / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_name, "data": "synthetic",
        "config": {"workload": f"{name}: MoE layer forward, {T_in} tokens, hidden {H}, {w.num_experts} experts, "
                               f"top-{w.top_k}, intermediate {I}, capacity_factor {w.capacity_factor}"
                               + (", Zipf-skewed router logits" if w.zipf_bias else "")
                               + (f", MoD keeps {w.mod_keep_fraction:.3f} of each sequence" if w.mod_keep_fraction else ""),
                   "kept_assignments": kept, "dropped_assignments": dropped, "inputs_drawn_on": gen_device},
        "roofline": roofline,
        "stages_ms": {s: round(v["mean_ms"], 4) for s, v in stages.items()},
        "stages_median_p10_p90_ms": {s: [round(v["median_ms"], 4), round(v["p10_ms"], 4), round(v["p90_ms"], 4)]
                                     for s, v in stages.items()},
    }
    if not mfma_bound:
        result["stream_read_reference"] = stream_read_reference
    if mfma_bound and w.dtype == torch.bfloat16 and not args.no_calibration:
        with torch.no_grad():
            result["calibration"] = gemm_calibration(w, moe, plan, kept, gu_ms)
        log(f"  calibration: {json.dumps(result['calibration'])}")
    if not args.no_cpu_baseline:
        sample = min(args.cpu_sample_tokens, T_moe)
        src = w
        if hasattr(layer, "moe"):
            log("  cpu baseline: MoE part only, on the first tokens of the batch")
        if getattr(args, "defer_cpu_baseline", False):
            result["_cpu_leg"] = (src, sample)      # main() runs it after the secondary records
        else:
            result["cpu_baseline"] = cpu_baseline(src, sample)
            log(f"  cpu baseline: {result['cpu_baseline']}")
    return result


def run_train(args):
    """Forward + backward of the MoE layer through the autograd path (all steps are HIP kernels)."""
    from adaptivetrainingsystem_amd import workloads as W

    dev = torch.device("cuda:0")
    name = args.workload[:-len("_train")]
    w = W.make_moe_workload(name, device=dev, gen_device="cuda")
    layer = W.build_layer(w, "fcfs")
    for p in layer.parameters():
        p.requires_grad_(True)
    x = w.x.clone().requires_grad_(True)
    cot = torch.randn_like(x)
    T_in = w.tokens
    log(f"workload {name} (training step): tokens={T_in} H={w.hidden} E={w.num_experts} k={w.top_k} "
        f"I={w.intermediate} cf={w.capacity_factor} dtype={w.dtype}")

    def step():
        for p in layer.parameters():
            p.grad = None
        x.grad = None
        out, aux = layer(x)
        torch.autograd.backward([out, aux], [cot, torch.ones_like(aux)])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    kept = int(layer.last_plan["kept"].sum().item())
    H, I = w.hidden, w.intermediate
    flops = 18.0 * H * I * kept            # forward 6*H*I per kept row, backward twice that
    achieved = flops / (dt / args.steps) / 1e12
    finite = all(p.grad is not None and bool(torch.isfinite(p.grad.float()).all()) for p in layer.parameters())
    log(f"  kept assignments {kept}; gradients finite: {finite}; {achieved:.1f} TFLOP/s over the whole step; "
        f"peak memory {torch.cuda.max_memory_allocated() / 2**30:.1f} GiB")
    result = {
        "metric": "MoE-layer training tokens/s (forward + backward, h4096, 8e top-2, bf16)",
        "value": T_in * args.steps / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{name}: MoE layer forward + backward (gradients of x, gate and all expert weights), "
                               f"{T_in} tokens, hidden {H}, {w.num_experts} experts, top-{w.top_k}, intermediate {I}, "
                               f"capacity_factor {w.capacity_factor}", "kept_assignments": kept},
        "roofline": {"kernel": "whole step: 9 grouped GEMM passes (18*H*I flop per kept row) plus the HBM-bound kernels",
                     "bound": "mfma", "achieved": achieved, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_BF16_TFLOPS, "traffic": None},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        n = min(args.cpu_sample_tokens, 2048)
        xs = w.x.reshape(-1, H)[:n].float().cpu()
        bias = None if w.logit_bias is None else w.logit_bias.float().cpu()
        E = w.num_experts
        tens = [xs, w.gate.float().cpu()] + [t.float().cpu() for t in w.gate_up] + [t.float().cpu() for t in w.down]

        def fwd(xx, wgate, *ws):
            r = O.moe_forward_capacity(xx, wgate, list(ws[:E]), list(ws[E:]), k=w.top_k,
                                       capacity_factor=w.capacity_factor, routing=w.routing, logit_bias=bias)
            return r["out"], r["aux"]

        t0 = time.perf_counter()
        O.layer_grads(fwd, tens, [torch.ones(n, H), torch.tensor(1.0)])
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": n / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"first {n} tokens, same weights, float32 autograd over the oracle forward, "
                                            f"one pass ({cdt:.2f} s)"}
        log(f"  cpu baseline: {result['cpu_baseline']}")
    return result


def run_loss_clip(args):
    """Fused cross-entropy (forward + logits gradient) over [16384, 32000] bf16 logits, then gradient
    norm + clipping over the headline layer's 2.8 G bf16 gradient elements."""
    from adaptivetrainingsystem_amd.profiling import StageTimer
    from adaptivetrainingsystem_amd.training import FusedGradClip, FusedLoss
    dev = torch.device("cuda:0")
    T, V = 16384, 32000
    torch.manual_seed(5)
    logits = (torch.randn(T, V, device=dev) * 2).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), device=dev)
    grads = [torch.randn(2 * 14336, 4096, device=dev).bfloat16() for _ in range(8)] + \
            [torch.randn(4096, 14336, device=dev).bfloat16() for _ in range(8)] + [torch.randn(8, 4096, device=dev).bfloat16()]
    loss_fn, clip = FusedLoss(), FusedGradClip()
    timer = StageTimer()

    def step():
        logits.grad = None
        with timer.range("loss_fwd"):
            out = loss_fn(logits, labels)
        with timer.range("loss_bwd"):
            out["loss"].backward()
        with timer.range("grad_clip"):
            clip.norm_and_clip(grads, 1.0)
        return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = StageTimer()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    n_grad = sum(g.numel() for g in grads)
    # the gradients are already inside the norm after the first step, so the scaling pass returns at once:
    # the clip stage reads every gradient once
    bytes_ = {"loss_fwd": T * V * 2, "loss_bwd": 2 * T * V * 2, "grad_clip": n_grad * 2}
    for k, v in st.items():
        log(f"  {k:10s} {v['mean_ms']*1e3:9.1f} us -> {bytes_[k] / (v['mean_ms'] * 1e-3) / 1e9:.0f} GB/s "
            f"({bytes_[k] / (v['mean_ms'] * 1e-3) / 1e9 / PEAK_HBM_GBS:.1%}); median {v['median_ms']*1e3:.1f} us, "
            f"max {v['max_ms']*1e3:.1f} us")
    gbs = bytes_["loss_bwd"] / (st["loss_bwd"]["mean_ms"] * 1e-3) / 1e9
    result = {
        "metric": "fused cross-entropy + grad-clip tokens/s", "value": T * args.steps / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"loss_clip: cross-entropy + accuracy forward and logits gradient on [{T}, {V}] bf16 "
                               f"logits; norm + clip of {n_grad} bf16 gradient elements in 17 tensors"},
        "roofline": {"kernel": "cross_entropy_bwd", "bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "traffic": None},
        "stages_ms": {s_: round(v["mean_ms"], 4) for s_, v in st.items()},
        "loss": float(out["loss"].detach()),
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        n = 2048
        lg = logits.detach()[:n].float().cpu().requires_grad_()
        t0 = time.perf_counter()
        O.fused_loss(lg, labels[:n].cpu())["loss"].backward()
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": n / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"first {n} tokens: float32 cross-entropy forward + backward ({cdt:.2f} s)"}
    return result


def run_attention(args):
    """Causal GQA attention of the headline model shape: B 8, L 2048, 32 query / 8 kv heads, head_dim 128."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd.profiling import StageTimer
    dev = torch.device("cuda:0")
    B, L, Hq, Hkv, D = 8, 2048, 32, 8, 128
    torch.manual_seed(6)
    q = torch.randn(B, Hq, L, D, device=dev).bfloat16()
    k = torch.randn(B, Hkv, L, D, device=dev).bfloat16()
    v = torch.randn(B, L, Hkv, D, device=dev).bfloat16().transpose(1, 2)     # view of a projection output
    for _ in range(args.warmup):
        ops.causal_attention(q, k, v)
    torch.cuda.synchronize()
    timer = StageTimer()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        with timer.range("attention"):
            out = ops.causal_attention(q, k, v)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    flops = 4.0 * B * Hq * D * L * (L + 1) / 2
    achieved = flops / (st["attention"]["mean_ms"] * 1e-3) / 1e12
    log(f"  attention {st['attention']['mean_ms']*1e3:.1f} us -> {achieved:.1f} TFLOP/s "
        f"({achieved / PEAK_MFMA_BF16_TFLOPS:.1%} of the bf16 MFMA peak)")
    result = {
        "metric": "causal GQA attention tokens/s", "value": B * L * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"attention: causal GQA forward, batch {B}, seq {L}, {Hq} query / {Hkv} kv heads, head_dim {D}"},
        "roofline": {"kernel": "attention_fwd_kernel", "bound": "mfma", "achieved": achieved,
                     "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": None},
        "stages_ms": {s_: round(v_["mean_ms"], 4) for s_, v_ in st.items()},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        rep = Hq // Hkv
        qc, kc, vc = q[:1].float().cpu(), k[:1].float().cpu(), v[:1].float().cpu()
        t0 = time.perf_counter()
        O.attention_standard(qc, kc.repeat_interleave(rep, dim=1), vc.repeat_interleave(rep, dim=1), D ** -0.5)
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": L / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"one sequence of the batch ({L} tokens), float32, one pass ({cdt:.2f} s)"}
    return result


def run_attention_train(args):
    """Forward + backward of the causal GQA attention at the headline model shape (see run_attention)."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd.profiling import StageTimer
    dev = torch.device("cuda:0")
    B, L, Hq, Hkv, D = 8, 2048, 32, 8, 128
    torch.manual_seed(8)
    q = torch.randn(B, Hq, L, D, device=dev).bfloat16()
    k = torch.randn(B, Hkv, L, D, device=dev).bfloat16()
    v = torch.randn(B, Hkv, L, D, device=dev).bfloat16()
    dout = torch.randn(B, L, Hq * D, device=dev).bfloat16()

    def step(timer=None):
        if timer is None:
            out, lse = ops.causal_attention(q, k, v, return_lse=True)
            return ops.causal_attention_bwd(q, k, v, out, lse, dout)
        with timer.range("forward"):
            out, lse = ops.causal_attention(q, k, v, return_lse=True)
        with timer.range("backward"):
            return ops.causal_attention_bwd(q, k, v, out, lse, dout)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = StageTimer()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(timer)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    prod = 2.0 * B * Hq * D * L * (L + 1) / 2            # one causal [L, L] x D product
    # forward 2 products; backward 7 as computed here (scores and dP are formed in both backward kernels),
    # 5 by the textbook count, which is the one the rate is quoted on
    step_ms = st["forward"]["mean_ms"] + st["backward"]["mean_ms"]
    achieved = 7.0 * prod / (step_ms * 1e-3) / 1e12
    log(f"  forward {st['forward']['mean_ms']*1e3:.1f} us, backward {st['backward']['mean_ms']*1e3:.1f} us -> "
        f"{achieved:.1f} TFLOP/s over 2 + 5 products ({achieved / PEAK_MFMA_BF16_TFLOPS:.1%} of the bf16 MFMA peak)")
    result = {
        "metric": "causal GQA attention training tokens/s", "value": B * L * args.steps / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"attention_train: causal GQA forward + backward, batch {B}, seq {L}, {Hq} query / "
                               f"{Hkv} kv heads, head_dim {D}"},
        "roofline": {"kernel": "attention_fwd_kernel + attention_bwd_dq_kernel (forms delta) + "
                               "attention_bwd_dkv_kernel", "bound": "mfma", "achieved": achieved,
                     "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": None},
        "stages_ms": {s_: round(v_["mean_ms"], 4) for s_, v_ in st.items()},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        rep = Hq // Hkv
        qc, kc, vc = (t[:1].float().cpu().requires_grad_() for t in (q, k, v))
        t0 = time.perf_counter()
        o = O.attention_standard(qc, kc.repeat_interleave(rep, dim=1), vc.repeat_interleave(rep, dim=1), D ** -0.5)
        o.backward(dout[:1].float().cpu())
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": L / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"one sequence of the batch ({L} tokens), float32, forward + autograd "
                                            f"backward ({cdt:.2f} s)"}
    return result


def run_block_train(args):
    """One transformer block of the headline model (pre-norm, GQA attention, top-2 of 8 experts MoE FFN with
    FCFS capacity 1.25) on batch 8 x seq 2048: forward + backward with all gradients."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    from adaptivetrainingsystem_amd.profiling import StageTimer
    dev = torch.device("cuda:0")
    B, L, H, I, E, K, Hq, Hkv = 8, 2048, 4096, 14336, 8, 2, 32, 8
    torch.manual_seed(9)
    cfg = LayerConfig(H, I, E, K, 1.25, num_heads=Hq, num_kv_heads=Hkv, seq_length=L, use_moe=True,
                      moe_capacity_mode="fcfs", num_layers=32)
    with torch.device(dev):
        blk = A.TransformerBlock(cfg)
    blk = blk.to(torch.bfloat16).train()
    x = torch.randn(B, L, H, device=dev).bfloat16().requires_grad_()
    dy = torch.randn(B, L, H, device=dev).bfloat16()

    def step(timer=None):
        blk.zero_grad(set_to_none=True)
        x.grad = None
        if timer is None:
            out, aux = blk(x)
            torch.autograd.backward([out, aux], [dy, torch.ones_like(aux)])
            return
        with timer.range("forward"):
            out, aux = blk(x)
        with timer.range("backward"):
            torch.autograd.backward([out, aux], [dy, torch.ones_like(aux)])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = StageTimer()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(timer)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    T = B * L
    kept = int(blk.ffn.last_plan["kept"].sum().item())
    D = H // Hq
    proj = 2.0 * T * H * (Hq * D + 2 * Hkv * D + H)
    attn = 2.0 * B * Hq * D * L * (L + 1) / 2
    ffn = 6.0 * kept * H * I
    flops = 3.0 * (proj + ffn) + 7.0 * attn + 3.0 * 2.0 * T * H * E      # forward + dgrad + wgrad; attention 2 + 5
    step_ms = st["forward"]["mean_ms"] + st["backward"]["mean_ms"]
    achieved = flops / (step_ms * 1e-3) / 1e12
    log(f"  forward {st['forward']['mean_ms']:.3f} ms, backward {st['backward']['mean_ms']:.3f} ms; kept assignments "
        f"{kept} of {T * K}; {achieved:.1f} TFLOP/s over the step ({achieved / PEAK_MFMA_BF16_TFLOPS:.1%} of the bf16 MFMA peak); "
        f"peak memory {torch.cuda.max_memory_allocated() / 2**30:.1f} GiB")
    return {
        "metric": "transformer block training tokens/s", "value": T * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"block_train: pre-norm block, GQA {Hq}/{Hkv} heads + MoE {E} experts top-{K} (I {I}, cf 1.25), "
                               f"hidden {H}, batch {B}, seq {L}, forward + backward"},
        "roofline": {"kernel": "whole step (grouped GEMMs, attention, HBM-bound kernels)", "bound": "mfma",
                     "achieved": achieved, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_BF16_TFLOPS, "traffic": None},
        "stages_ms": {s_: round(v_["mean_ms"], 4) for s_, v_ in st.items()},
        "cpu_baseline": None,
    }


def run_attention_decode(args):
    """One decoding step of the causal GQA attention: 64 sequences, one new token each, against a cache of 2048
    keys (32 query / 8 kv heads, head_dim 128).  Bound by reading the cache once."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd.profiling import StageTimer
    dev = torch.device("cuda:0")
    B, Lk, Hq, Hkv, D = 64, 2048, 32, 8, 128
    torch.manual_seed(10)
    q = torch.randn(B, Hq, 1, D, device=dev).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, device=dev).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, device=dev).bfloat16()
    for _ in range(args.warmup):
        ops.causal_attention(q, k, v)
    torch.cuda.synchronize()
    timer = StageTimer()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        with timer.range("attention_decode"):
            ops.causal_attention(q, k, v)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    # K and V of the cache are each read once
    cache_bytes = 2.0 * B * Hkv * Lk * D * 2
    achieved = cache_bytes / (st["attention_decode"]["mean_ms"] * 1e-3) / 1e9
    log(f"  decode attention {st['attention_decode']['mean_ms']*1e3:.1f} us -> {achieved:.0f} GB/s of "
        f"cache ({achieved / PEAK_HBM_GBS:.1%} of the HBM peak)")
    result = {
        "metric": "causal GQA attention decode tokens/s", "value": B * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"attention_decode: {B} sequences x 1 new token against {Lk} cached keys, {Hq} query / "
                               f"{Hkv} kv heads, head_dim {D}"},
        "roofline": {"kernel": "attention_fwd_kernel, packed rows", "bound": "hbm", "achieved": achieved,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                     "traffic": profile_traffic("attention_decode", "attention")},
        "stages_ms": {s_: round(v_["mean_ms"], 4) for s_, v_ in st.items()},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        rep = Hq // Hkv
        n = 8
        qc, kc, vc = q[:n].float().cpu(), k[:n].float().cpu(), v[:n].float().cpu()
        t0 = time.perf_counter()
        O.attention_standard(qc, kc.repeat_interleave(rep, dim=1), vc.repeat_interleave(rep, dim=1), D ** -0.5)
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": n / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"{n} of the {B} sequences, float32, one pass ({cdt:.2f} s)"}
    return result


def run_gqa_layer(args):
    """The attention sub-layer of the headline model shape (hidden 4096, 32 query / 8 kv heads, head_dim 128) on
    batch 8 x seq 2048: q/k/v projections, RoPE, causal attention, output projection."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    from adaptivetrainingsystem_amd.profiling import StageTimer
    dev = torch.device("cuda:0")
    B, L, H, Hq, Hkv = 8, 2048, 4096, 32, 8
    D = H // Hq
    torch.manual_seed(7)
    cfg = LayerConfig(H, 14336, 8, 2, num_heads=Hq, num_kv_heads=Hkv, seq_length=L)
    att = A.GroupedQueryAttention(cfg).to(torch.bfloat16).to(dev).eval()
    x = torch.randn(B, L, H, device=dev).bfloat16()
    timer = StageTimer()
    with torch.no_grad():
        for _ in range(args.warmup):
            att(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            with timer.range("gqa_layer"):
                att(x)
        torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = timer.summary()
    T = B * L
    flops = 2.0 * T * H * (Hq * D + 2 * Hkv * D + H) + 4.0 * B * Hq * D * L * (L + 1) / 2
    achieved = flops / (st["gqa_layer"]["mean_ms"] * 1e-3) / 1e12
    log(f"  attention sub-layer {st['gqa_layer']['mean_ms']:.3f} ms -> {achieved:.1f} TFLOP/s over projections + attention "
        f"({achieved / PEAK_MFMA_BF16_TFLOPS:.1%} of the bf16 MFMA peak)")
    result = {
        "metric": "GQA attention sub-layer tokens/s", "value": T * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"gqa_layer: q/k/v/o projections + RoPE + causal attention, batch {B}, seq {L}, hidden {H}, "
                               f"{Hq} query / {Hkv} kv heads"},
        "roofline": {"kernel": "whole sub-layer (4 projection GEMMs + attention_fwd_kernel)", "bound": "mfma",
                     "achieved": achieved, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_BF16_TFLOPS, "traffic": None},
        "stages_ms": {s_: round(v_["mean_ms"], 4) for s_, v_ in st.items()},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        w = [getattr(att, n).weight.detach().float().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
        xc = x[:1].float().cpu()
        t0 = time.perf_counter()
        O.gqa_forward(xc, *w, Hq, Hkv)
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": L / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"one sequence of the batch ({L} tokens), float32, one pass ({cdt:.2f} s)"}
    return result


def run_gqa_decode(args):
    """Decoding steps of the attention sub-layer of the headline model shape (hidden 4096, 32 query / 8 kv heads,
    head_dim 128): 64 sequences, one new token each, starting from 2048 cached keys; every step feeds the cache
    the previous one returned (q/k/v projections of 64 rows, RoPE, cache append, attention, output projection)."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    dev = torch.device("cuda:0")
    B, L0, H, Hq, Hkv = 64, 2048, 4096, 32, 8
    D = H // Hq
    torch.manual_seed(11)
    cfg = LayerConfig(H, 14336, 8, 2, num_heads=Hq, num_kv_heads=Hkv, seq_length=8192)
    att = A.GroupedQueryAttention(cfg).to(torch.bfloat16).to(dev).eval()
    xs = torch.randn(8, B, 1, H, device=dev).bfloat16()

    def fresh_cache():
        return (torch.randn(B, Hkv, L0, D, device=dev).bfloat16(), torch.randn(B, Hkv, L0, D, device=dev).bfloat16())

    with torch.no_grad():
        cache = fresh_cache()
        for i in range(args.warmup):
            _, cache = att(xs[i % 8], past_key_value=cache, use_cache=True)
        cache = fresh_cache()
        _, cache = att(xs[0], past_key_value=cache, use_cache=True)       # moves the cache into a buffer with room
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        for i in range(args.steps):
            _, cache = att(xs[i % 8], past_key_value=cache, use_cache=True)
        ev1.record()
        torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    gpu_ms = ev0.elapsed_time(ev1) / args.steps
    keys_mid = L0 + 1 + args.steps / 2.0
    # a step streams the four projection weights once and the filled part of the cache once
    weight_bytes = 2.0 * H * (Hq * D + 2 * Hkv * D + H)
    cache_bytes = 2.0 * B * Hkv * keys_mid * D * 2
    achieved = (weight_bytes + cache_bytes) / (gpu_ms * 1e-3) / 1e9
    log(f"  attention sub-layer decode step {gpu_ms * 1e3:.1f} us (host clock {dt / args.steps * 1e6:.1f} us) -> "
        f"{achieved:.0f} GB/s of weights + cache ({achieved / PEAK_HBM_GBS:.1%} of the HBM peak)")
    result = {
        "metric": "GQA attention sub-layer decode tokens/s", "value": B * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"gqa_decode: q/k/v/o projections + RoPE + cache append + attention, {B} sequences x 1 new "
                               f"token, {L0} cached keys growing by one per step, hidden {H}, {Hq} query / {Hkv} kv heads"},
        "roofline": {"kernel": "whole sub-layer step (4 K-sliced projections + attention_fwd_kernel, packed rows)",
                     "bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM_GBS, "traffic": None},
        "stages_ms": {"gqa_decode_step": round(gpu_ms, 4)},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        w = [getattr(att, n).weight.detach().float().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
        n = 8
        kc, vc = (t[:n, :, :L0].float().cpu() for t in cache)
        xc = xs[0][:n].float().cpu()
        t0 = time.perf_counter()
        O.gqa_forward(xc, *w, Hq, Hkv, past_key_value=(kc, vc), use_cache=True)
        cdt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": n / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"{n} of the {B} sequences, float32, one step ({cdt:.2f} s)"}
    return result


def run_norm_rope(args):
    """Config 2: RMSNorm over x[8192, 2048] and RoPE over q[4,16,2048,128], k[4,4,2048,128], bf16."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd import workloads as W
    from adaptivetrainingsystem_amd.profiling import StageTimer, stream_copy
    dev = torch.device("cuda:0")
    w = W.make_norm_rope_workload(device=dev, gen_device="cpu")
    cos, sin = ops.rope_table(w.seq, w.head_dim, w.theta, device=dev)
    # The inputs of one step are 75 MB: repeated over the same buffers they would be served by the 256 MB
    # memory-side cache, not by HBM.  The calls therefore rotate over 16 copies (1.2 GB of inputs).
    n_sets = 16
    xs = [w.x] + [w.x.clone() for _ in range(n_sets - 1)]
    qs = [w.q] + [w.q.clone() for _ in range(n_sets - 1)]
    ks = [w.k] + [w.k.clone() for _ in range(n_sets - 1)]
    copy_dst = [torch.empty_like(w.x) for _ in range(n_sets)]
    turn = [0]
    keep = [None] * (4 * n_sets)      # results stay alive for a while, so outputs land in distinct blocks too

    def nxt():
        turn[0] = (turn[0] + 1) % n_sets
        return turn[0]

    def hold(result):
        keep[hold.at % len(keep)] = result
        hold.at += 1

    hold.at = 0

    # at least one pass over the ring of held results, so that the timed steps allocate nothing new
    for _ in range(max(args.warmup, len(keep) // 2)):
        i = nxt()
        hold(ops.rmsnorm(xs[i], w.norm_weight, w.eps))
        hold(ops.rope(qs[i], ks[i], cos, sin))
    torch.cuda.synchronize()
    # whole-step time: RMSNorm then RoPE, back to back
    t0 = time.perf_counter()
    for _ in range(args.steps):
        i = nxt()
        hold(ops.rmsnorm(xs[i], w.norm_weight, w.eps))
        hold(ops.rope(qs[i], ks[i], cos, sin))
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # per-kernel duration: these kernels run 10-20 us, shorter than the host's launch path, so each is
    # timed as a burst of launches between one pair of events (the queue stays full, the events see
    # kernel time plus the ~1 us gap between consecutive kernels)
    burst = 20

    def stage_round(timer):
        with timer.range("rmsnorm"):
            for _ in range(burst):
                hold(ops.rmsnorm(xs[nxt()], w.norm_weight, w.eps))
        with timer.range("rope"):
            for _ in range(burst):
                i = nxt()
                hold(ops.rope(qs[i], ks[i], cos, sin))
        # the gradients of the two kernels (another copy of x stands in for dy: same shape and type)
        with timer.range("rmsnorm_bwd"):
            for _ in range(burst):
                i = nxt()
                hold(ops.rmsnorm_bwd(xs[i], w.norm_weight, xs[(i + 1) % n_sets], w.eps))
        with timer.range("rope_bwd"):
            for _ in range(burst):
                i = nxt()
                hold(ops.rope(qs[i], ks[i], cos, sin, inverse=True))
        # yardsticks: torch's copy of x (the bytes of the RMSNorm) and this library's plain streaming copy kernel,
        # over the same rotating buffers
        with timer.range("copy_x"):
            for _ in range(burst):
                i = nxt()
                copy_dst[i].copy_(xs[i])
        with timer.range("stream_copy_x"):
            for _ in range(burst):
                i = nxt()
                stream_copy(xs[i], copy_dst[i])

    # two untimed rounds first: the ring of held results fills up and the allocator stops asking the driver
    # for new blocks, which would otherwise fall into the first timed bursts
    for _ in range(2):
        stage_round(StageTimer())
    torch.cuda.synchronize()
    timer = StageTimer()
    for _ in range(max(2, args.steps // burst)):
        stage_round(timer)
    torch.cuda.synchronize()
    st = timer.summary()
    for v in st.values():
        for key in ("mean_ms", "min_ms", "total_ms"):
            v[key] /= burst if key != "total_ms" else 1
    es = w.x.element_size()
    T = w.batch * w.seq
    rms_bytes = 2 * T * w.hidden * es + 4 * w.hidden
    rope_bytes = 2 * T * (w.q_heads + w.kv_heads) * w.head_dim * es + 2 * w.seq * (w.head_dim // 2) * 4
    rms_gbs = rms_bytes / (st["rmsnorm"]["mean_ms"] * 1e-3) / 1e9
    rope_gbs = rope_bytes / (st["rope"]["mean_ms"] * 1e-3) / 1e9
    log(f"  rmsnorm {st['rmsnorm']['mean_ms']*1e3:.1f} us -> {rms_gbs:.0f} GB/s ({rms_gbs/PEAK_HBM_GBS:.1%}); "
        f"rope {st['rope']['mean_ms']*1e3:.1f} us -> {rope_gbs:.0f} GB/s ({rope_gbs/PEAK_HBM_GBS:.1%})")
    copy_gbs = 2 * T * w.hidden * es / (st["copy_x"]["mean_ms"] * 1e-3) / 1e9
    log(f"  plain copy of x over the same buffers: {st['copy_x']['mean_ms']*1e3:.1f} us -> {copy_gbs:.0f} GB/s "
        f"({copy_gbs/PEAK_HBM_GBS:.1%})")
    scopy_gbs = 2 * T * w.hidden * es / (st["stream_copy_x"]["mean_ms"] * 1e-3) / 1e9
    log(f"  hand-written streaming copy of x: {st['stream_copy_x']['mean_ms']*1e3:.1f} us -> {scopy_gbs:.0f} GB/s "
        f"({scopy_gbs/PEAK_HBM_GBS:.1%}); rmsnorm reaches {rms_gbs / scopy_gbs:.3f} of it, rope {rope_gbs / scopy_gbs:.3f}")
    rmsb_bytes = 3 * T * w.hidden * es + 8 * w.hidden
    rmsb_gbs = rmsb_bytes / (st["rmsnorm_bwd"]["mean_ms"] * 1e-3) / 1e9
    ropeb_gbs = rope_bytes / (st["rope_bwd"]["mean_ms"] * 1e-3) / 1e9
    log(f"  rmsnorm_bwd {st['rmsnorm_bwd']['mean_ms']*1e3:.1f} us -> {rmsb_gbs:.0f} GB/s ({rmsb_gbs/PEAK_HBM_GBS:.1%}); "
        f"rope_bwd {st['rope_bwd']['mean_ms']*1e3:.1f} us -> {ropeb_gbs:.0f} GB/s ({ropeb_gbs/PEAK_HBM_GBS:.1%})")
    result = {
        "metric": "fused RMSNorm + RoPE tokens/s (config 2)", "value": T * args.steps / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c2_norm_rope: RMSNorm x[8192,2048] + RoPE q[4,16,2048,128] k[4,4,2048,128]"},
        "roofline": {"kernel": "rope", "bound": "hbm", "achieved": rope_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": rope_gbs / PEAK_HBM_GBS, "traffic": profile_traffic("c2_norm_rope", "rope")},
        "rmsnorm_roofline": {"bound": "hbm", "achieved": rms_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": rms_gbs / PEAK_HBM_GBS, "traffic": profile_traffic("c2_norm_rope", "rmsnorm")},
        "copy_reference": {"what": "torch copy of x over the same rotating buffers (1.2 GB of inputs, outputs in "
                                   "distinct blocks: nothing is served by the 256 MB memory-side cache)",
                           "achieved": copy_gbs, "unit": "GB/s", "frac": copy_gbs / PEAK_HBM_GBS},
        "stream_copy_reference": {"what": "this library's plain streaming copy kernel (16 bytes per lane, four loads in "
                                          "flight per lane, non-temporal) of x over the same rotating buffers: what a "
                                          "kernel that only moves the RMSNorm's bytes reaches at this size",
                                  "achieved": scopy_gbs, "unit": "GB/s", "frac": scopy_gbs / PEAK_HBM_GBS,
                                  "rmsnorm_vs_copy": rms_gbs / scopy_gbs, "rope_vs_copy": rope_gbs / scopy_gbs},
        "rmsnorm_bwd_roofline": {"bound": "hbm", "achieved": rmsb_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                 "frac": rmsb_gbs / PEAK_HBM_GBS,
                                 "traffic": profile_traffic("c2_norm_rope", "rmsnorm_bwd")},
        "rope_bwd_roofline": {"bound": "hbm", "achieved": ropeb_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": ropeb_gbs / PEAK_HBM_GBS,
                              "traffic": profile_traffic("c2_norm_rope", "rope_bwd")},
        "stages_ms": {s: round(v["mean_ms"], 5) for s, v in st.items()},
    }
    if not args.no_cpu_baseline:
        from oracle import sparse_layer_oracle as O
        x, nw, q, k = w.x.float().cpu(), w.norm_weight.cpu(), w.q.float().cpu(), w.k.float().cpu()
        c, s = O.rope_table(w.seq, w.head_dim, w.theta)
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            O.rmsnorm(x, nw, w.eps)
            O.rope_apply(q, k, c, s)
        cdt = (time.perf_counter() - t0) / reps
        result["cpu_baseline"] = {"value": T / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(),
                                  "kind": "port", "sample": f"whole config, float32, mean of {reps} passes"}
    return result


def _r(v, n=4):
    return round(float(v), n) if isinstance(v, (int, float)) else v


def _roof(r):
    return {"bound": r["bound"], "achieved": _r(r["achieved"], 1), "peak": r["peak"], "unit": r["unit"],
            "frac": _r(r["frac"]), "traffic": r.get("traffic")}


def secondary_records(args):
    """The other benchmark configurations, each from a short event-timed loop of its own in this process
    (their own step and warm-up counts; no CPU leg, no calibration): config 2's RMSNorm / RoPE against the HBM
    peak and against the streaming-copy yardstick, config 3's weight-streaming GEMMs against the HBM peak and the
    streaming-read yardstick, config 5's step time and grouped GEMM against the MFMA peak."""
    import copy
    out = {}
    sub = copy.copy(args)
    sub.no_cpu_baseline, sub.no_calibration = True, True
    sub.steps, sub.warmup = 200, 50

    sub.workload = "c2_norm_rope"
    r = run_norm_rope(sub)
    out["c2_norm_rope"] = {
        "workload": r["config"]["workload"], "ms_per_step": _r(r["ms_per_step"], 5),
        "rmsnorm": _roof(r["rmsnorm_roofline"]), "rope": _roof(r["roofline"]),
        "rmsnorm_bwd": _roof(r["rmsnorm_bwd_roofline"]), "rope_bwd": _roof(r["rope_bwd_roofline"]),
        "stream_copy_reference": {k: _r(v) for k, v in r["stream_copy_reference"].items() if k != "what"},
        "copy_reference": {k: _r(v) for k, v in r["copy_reference"].items() if k != "what"},
        "kernel_us": {k: _r(v * 1e3, 2) for k, v in r["stages_ms"].items()}}
    torch.cuda.empty_cache()

    sub.workload = "c3_decode"
    r = run_moe(sub)
    st = r["stages_ms"]
    H, I, es = 4096, 14336, 2
    kept = r["config"]["kept_assignments"]
    dn_bytes = 8 * H * I * es + kept * (H + I) * es            # every expert's down weight once + rows in and out
    dn_ms = st["down"]
    out["c3_decode"] = {
        "workload": r["config"]["workload"], "tokens_per_s": _r(r["value"], 0), "ms_per_step": _r(r["ms_per_step"]),
        "gateup": _roof(r["roofline"]),
        "down": {"bound": "hbm", "achieved": _r(dn_bytes / (dn_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                 "unit": "GB/s", "frac": _r(dn_bytes / (dn_ms * 1e-3) / 1e9 / PEAK_HBM_GBS),
                 "traffic": profile_traffic("c3_decode", "down")},
        "stream_read_reference": {k: _r(v) for k, v in r["stream_read_reference"].items() if k != "what"},
        "stages_ms": st}
    torch.cuda.empty_cache()

    sub.workload = "c5_finegrained_mod"
    r = run_moe(sub)
    st = r["stages_ms"]
    kept = r["config"]["kept_assignments"]
    dn_tf = 2.0 * 2048 * 1408 * kept / (st["down"] * 1e-3) / 1e12
    out["c5_finegrained_mod"] = {
        "workload": r["config"]["workload"], "tokens_per_s": _r(r["value"], 0), "ms_per_step": _r(r["ms_per_step"]),
        "gateup": _roof(r["roofline"]),
        "down": {"bound": "mfma", "achieved": _r(dn_tf, 1), "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                 "frac": _r(dn_tf / PEAK_MFMA_BF16_TFLOPS), "traffic": profile_traffic("c5_finegrained_mod", "down")},
        "stages_ms": st}
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 20; 200 for the workloads whose step is shorter than 2 ms)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps first (default 5; 50 for the short workloads: with fewer the core clock "
                         "has not settled and the first kernels run up to 20 %% slower)")
    ap.add_argument("--workload", default="c4_prefill",
                    choices=["c4_prefill", "c3_decode", "c5_finegrained_mod", "c1_cpu_reference", "c2_norm_rope",
                             "c4_prefill_train", "c1_cpu_reference_train", "loss_clip", "attention", "attention_train", "attention_decode", "gqa_layer", "gqa_decode", "block_train"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-calibration", action="store_true",
                    help="skip the MFMA-only loops, the zero-operand launch and the vendor-BLAS matmul")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 1 GiB device copy (known traffic) so hardware-counter runs can be scaled")
    ap.add_argument("--cpu-sample-tokens", type=int, default=16384)
    ap.add_argument("--no-secondary", action="store_true",
                    help="with the default workload: skip the short runs of the other configurations (c2, c3, c5) "
                         "that are appended as the `secondary` record")
    args = ap.parse_args()
    short = args.workload in ("c3_decode", "c5_finegrained_mod", "c2_norm_rope", "loss_clip", "attention",
                              "attention_train", "attention_decode", "gqa_layer", "gqa_decode")
    if args.steps is None:
        args.steps = 200 if short else 20
    if args.warmup is None:
        args.warmup = 50 if short else 5
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on one GPU (experts stay resident, no collectives); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from adaptivetrainingsystem_amd import _lib
    _lib.load()
    torch.cuda.set_device(0)
    # everything imported so far moves to the permanent generation: a full collection over torch's half a
    # million objects takes tens of milliseconds, longer than the queued GPU work of the short workloads
    import gc
    gc.collect()
    gc.freeze()
    if args.copy_probe:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.workload == "c2_norm_rope":
        result = run_norm_rope(args)
    elif args.workload == "loss_clip":
        result = run_loss_clip(args)
    elif args.workload == "attention":
        result = run_attention(args)
    elif args.workload == "attention_train":
        result = run_attention_train(args)
    elif args.workload == "block_train":
        result = run_block_train(args)
    elif args.workload == "attention_decode":
        result = run_attention_decode(args)
    elif args.workload == "gqa_layer":
        result = run_gqa_layer(args)
    elif args.workload == "gqa_decode":
        result = run_gqa_decode(args)
    elif args.workload.endswith("_train"):
        result = run_train(args)
    else:
        with_secondary = args.workload == "c4_prefill" and not args.no_secondary
        # The CPU leg comes after the short GPU runs: allocating and freeing gigabytes between the headline
        # measurement and theirs changes where the driver places the tensors they allocate, and the decode
        # shape's weight-streaming launch runs up to 10 % slower on weights placed that way.
        args.defer_cpu_baseline = with_secondary
        result = run_moe(args)
        cpu_leg = result.pop("_cpu_leg", None)
        if with_secondary:
            torch.cuda.empty_cache()
            log("secondary records (other configurations, short loops in this process):")
            try:
                result["secondary"] = secondary_records(args)
            except Exception as exc:       # the headline line is printed whatever happens to the short runs
                result["secondary"] = {"error": f"{type(exc).__name__}: {exc}"}
            for name, rec in result["secondary"].items():
                log(f"  secondary {name}: {json.dumps(rec)}")
        if cpu_leg is not None:
            result["cpu_baseline"] = cpu_baseline(*cpu_leg)
            log(f"  cpu baseline: {result['cpu_baseline']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
