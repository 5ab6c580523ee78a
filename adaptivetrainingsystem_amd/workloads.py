"""Synthetic inputs for the five benchmark configurations of the sparse-layer path.

Every tensor is drawn from a torch generator seeded with the configuration's
seed, in the fixed order written below (x, norm weight, gate, then per expert
gate_up followed by down; for the MoD block the MoD router weight comes right
after x), as float32 N(0,1) scaled, then cast.  `gen_device="cpu"` draws on the
host (bit-reproducible everywhere; used by the parity tests at small sizes);
`gen_device="cuda"` draws on the GPU (used for the multi-gigabyte weight sets).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

import torch


@dataclass
class MoEWorkload:
    name: str
    seed: int
    batch: int
    seq: int
    hidden: int
    num_experts: int
    top_k: int
    intermediate: int
    capacity_factor: float
    dtype: torch.dtype
    routing: str = "softmax_topk"
    zipf_bias: float = 0.0          # logits += zipf_bias * ln(1/rank)
    mod_keep_fraction: Optional[float] = None
    x: torch.Tensor = None
    norm_weight: torch.Tensor = None
    gate: torch.Tensor = None
    gate_up: List[torch.Tensor] = field(default_factory=list)
    down: List[torch.Tensor] = field(default_factory=list)
    mod_weight: Optional[torch.Tensor] = None
    logit_bias: Optional[torch.Tensor] = None

    @property
    def tokens(self) -> int:
        return self.batch * self.seq


CONFIGS = {
    # name: (seed, batch, seq, hidden, experts, top_k, intermediate, capacity_factor, dtype, zipf, mod_keep)
    "c1_cpu_reference": (0, 2, 256, 512, 8, 2, 1408, 1.25, torch.float32, 0.0, None),
    "c3_decode": (2, 1, 64, 4096, 8, 2, 14336, 1.25, torch.bfloat16, 0.0, None),
    "c4_prefill": (3, 8, 2048, 4096, 8, 2, 14336, 1.25, torch.bfloat16, 1.5, None),
    "c5_finegrained_mod": (4, 16, 2048, 2048, 64, 6, 1408, 1.5, torch.bfloat16, 0.0, 0.125),
}


def make_moe_workload(name: str, device="cuda", gen_device: str = "cpu", scale_tokens: Optional[int] = None,
                      overrides: Optional[dict] = None) -> MoEWorkload:
    """Builds the tensors of one MoE configuration.  `scale_tokens` replaces batch*seq by
    1 x scale_tokens (parity tests at reduced size); `overrides` replaces shape fields."""
    seed, B, L, H, E, k, I, cf, dtype, zipf, keep = CONFIGS[name]
    if scale_tokens is not None:
        B, L = 1, scale_tokens
    w = MoEWorkload(name, seed, B, L, H, E, k, I, cf, dtype, zipf_bias=zipf, mod_keep_fraction=keep)
    for key, val in (overrides or {}).items():
        setattr(w, key, val)
    B, L, H, E, I, dtype = w.batch, w.seq, w.hidden, w.num_experts, w.intermediate, w.dtype
    gdev = torch.device(gen_device)
    gen = torch.Generator(device=gdev).manual_seed(seed)

    def draw(*shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=gen, device=gdev, dtype=torch.float32)
        if std != 1.0:
            t.mul_(std)
        if mean != 0.0:
            t.add_(mean)
        return t.to(dtype).to(device)

    w.x = draw(B, L, H)
    if w.mod_keep_fraction is not None:
        w.mod_weight = draw(1, H, std=1.0 / math.sqrt(H))
    w.norm_weight = torch.ones(H, dtype=torch.float32, device=device)
    w.gate = draw(E, H, std=0.02)
    for _ in range(E):
        w.gate_up.append(draw(2 * I, H, std=0.02))
        w.down.append(draw(H, I, std=0.02))
    if w.zipf_bias:
        ranks = torch.arange(1, E + 1, dtype=torch.float64)
        w.logit_bias = (w.zipf_bias * torch.log(1.0 / ranks)).float().to(device)
    return w


@dataclass
class NormRopeWorkload:
    seed: int = 1
    batch: int = 4
    seq: int = 2048
    hidden: int = 2048
    q_heads: int = 16
    kv_heads: int = 4
    head_dim: int = 128
    theta: float = 10000.0
    eps: float = 1e-6
    dtype: torch.dtype = torch.bfloat16
    x: torch.Tensor = None
    norm_weight: torch.Tensor = None
    q: torch.Tensor = None
    k: torch.Tensor = None


def make_norm_rope_workload(device="cuda", gen_device: str = "cpu", **overrides) -> NormRopeWorkload:
    """Config 2: x ~ N(0,1) [B,L,H], w ~ N(1,0.1) [H] float32, q [B,Hq,L,D], k [B,Hkv,L,D], drawn in that order."""
    w = NormRopeWorkload(**overrides)
    gdev = torch.device(gen_device)
    gen = torch.Generator(device=gdev).manual_seed(w.seed)

    def draw(*shape):
        return torch.randn(*shape, generator=gen, device=gdev, dtype=torch.float32)

    w.x = draw(w.batch, w.seq, w.hidden).to(w.dtype).to(device)
    w.norm_weight = (draw(w.hidden) * 0.1 + 1.0).to(device)
    w.q = draw(w.batch, w.q_heads, w.seq, w.head_dim).to(w.dtype).to(device)
    w.k = draw(w.batch, w.kv_heads, w.seq, w.head_dim).to(w.dtype).to(device)
    return w


class LayerConfig:
    """Minimal config object with the fields the layer constructors read."""

    def __init__(self, hidden_size, intermediate_size, num_experts, moe_top_k, capacity_factor=1.25, **kw):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_experts = num_experts
        self.moe_top_k = moe_top_k
        self.capacity_factor = capacity_factor
        self.init_std = 0.02
        self.num_layers = 1
        for key, val in kw.items():
            setattr(self, key, val)


def build_layer(w: MoEWorkload, capacity_mode: str = "fcfs"):
    """A MoE layer (or MoD+MoE block) on w.x's device whose parameters ARE the workload tensors."""
    from .layers import MoDMoEBlock, MoEFFNLayer

    cfg = LayerConfig(w.hidden, w.intermediate, w.num_experts, w.top_k, w.capacity_factor,
                      moe_routing=w.routing, moe_capacity_mode=capacity_mode,
                      mod_keep_fraction=w.mod_keep_fraction or 0.125)
    dev = w.x.device
    with torch.device("meta"):
        block = MoDMoEBlock(cfg) if w.mod_keep_fraction is not None else None
        layer = MoEFFNLayer(cfg) if block is None else None
    top = block if block is not None else layer
    top = top.to_empty(device=dev)
    moe = top.moe if block is not None else top
    moe.routing, moe.capacity_mode = w.routing, capacity_mode
    moe._routing_stats["expert_usage"] = torch.zeros(w.num_experts)
    moe.gate.weight = torch.nn.Parameter(w.gate, requires_grad=False)
    for e, ex in enumerate(moe.experts):
        ex.gate_up_proj.weight = torch.nn.Parameter(w.gate_up[e], requires_grad=False)
        ex.down_proj.weight = torch.nn.Parameter(w.down[e], requires_grad=False)
    moe.router_logit_bias = w.logit_bias
    if block is not None:
        block.router.weight = torch.nn.Parameter(w.mod_weight, requires_grad=False)
    top.eval()
    return top
