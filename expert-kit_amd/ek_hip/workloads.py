"""Synthetic workloads: the five benchmark configurations, seeded.

All randomness is drawn from ``torch.Generator`` objects with fixed seeds:
weights ``1000 + layer`` (one stream per expert), activations ``2000``, router
logits ``3000 + layer``, hot-expert bias permutation ``4000``, request lengths
``5000``.  The router is the Qwen3 shim's softmax -> top-k -> renormalise ->
cast (ek-integration/expertkit_torch/expertkit_torch/models/qwen3_moe.py:161-169),
spelled with torch primitives: it produces the *inputs* of the expert path.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import List, Optional

import torch

from .backend import ExpertWeight


@dataclass(frozen=True)
class Workload:
    name: str
    hidden: int
    inter: int
    n_experts: int
    top_k: int
    tokens: int
    act_dtype: torch.dtype
    w8: bool = False              # int8 weights + per-output-channel bf16 scales
    zipf_s: float = 0.0           # hot-expert bias b_e = -s * ln(rank_e)
    n_layers: int = 1
    ragged: bool = False          # tokens come from a continuous-batching request mix
    fp8_block: bool = False       # with w8: fp8 e4m3fn weights + fp32 scales per 128x128 block, kept as stored

    @property
    def pairs(self) -> int:
        return self.tokens * self.top_k

    def expert_weight_bytes(self) -> int:
        wsz = 1 if self.w8 else 2
        scales = (2 * self.inter + self.hidden) * 2 if self.w8 else 0
        if self.fp8_block:
            scales = 3 * ((self.inter + 127) // 128) * ((self.hidden + 127) // 128) * 4
        return 3 * self.hidden * self.inter * wsz + scales

    def flops_per_pair(self) -> int:
        return 6 * self.hidden * self.inter


C1 = Workload("c1_tiny_bf16", 1024, 512, 16, 2, 64, torch.bfloat16)
C2 = Workload("c2_qwen3_fp16_decode", 2048, 768, 128, 8, 256, torch.float16, zipf_s=1.0)
C3 = Workload("c3_dsv3_w8a16_decode", 7168, 2048, 256, 8, 128, torch.bfloat16, w8=True)
C4 = Workload("c4_dsv3_w8a16_prefill", 7168, 2048, 256, 8, 8192, torch.bfloat16, w8=True, zipf_s=0.8)
C5 = Workload("c5_qwen3_fp16_ragged_x4", 2048, 768, 128, 8, 0, torch.float16, zipf_s=1.2, n_layers=4, ragged=True)
CONFIGS = {w.name.split("_")[0]: w for w in (C1, C2, C3, C4, C5)}


def request_lengths(n_decode: int = 40, n_prefill: int = 8, lo: int = 64, hi: int = 1024) -> List[int]:
    """C5's request mix: decode requests hold 1 token, prefill chunks ~U{lo..hi}."""
    g = torch.Generator().manual_seed(5000)
    pre = torch.randint(lo, hi + 1, (n_prefill,), generator=g).tolist()
    return [1] * n_decode + pre


def resolve(w: Workload) -> Workload:
    """Fills in the token count of a ragged workload from its request mix."""
    if w.ragged and w.tokens == 0:
        return replace(w, tokens=sum(request_lengths()))
    return w


def request_offsets() -> torch.Tensor:
    lens = request_lengths()
    return torch.tensor([0] + list(torch.tensor(lens).cumsum(0).tolist()), dtype=torch.int32)


def make_x(w: Workload) -> torch.Tensor:
    g = torch.Generator().manual_seed(2000)
    return torch.randn(w.tokens, w.hidden, generator=g).to(w.act_dtype)


def expert_bias(w: Workload) -> Optional[torch.Tensor]:
    if w.zipf_s == 0.0:
        return None
    g = torch.Generator().manual_seed(4000)
    rank = torch.randperm(w.n_experts, generator=g) + 1
    return -w.zipf_s * torch.log(rank.float())


def make_routing(w: Workload, layer: int = 0):
    """(ids int32 [T,K], gate weights [T,K] in the activation dtype)."""
    g = torch.Generator().manual_seed(3000 + layer)
    logits = torch.randn(w.tokens, w.n_experts, generator=g)
    b = expert_bias(w)
    if b is not None:
        logits = logits + b
    rw = torch.nn.functional.softmax(logits, dim=1, dtype=torch.float)
    rw, sel = torch.topk(rw, w.top_k, dim=-1)
    rw = rw / rw.sum(dim=-1, keepdim=True)
    return sel.to(torch.int32).contiguous(), rw.to(w.act_dtype).contiguous()


def make_expert(w: Workload, e: int, layer: int = 0, device: str = "cpu", std: float = 0.02) -> ExpertWeight:
    """One expert's weights.  Each expert has its own generator stream, so any
    subset can be reproduced without drawing the others.  CPU and GPU generators
    give different values for the same seed; parity tests always move the very
    tensors they loaded into the library over to the oracle."""
    seed = (1000 + layer) * 1_000_003 + e
    g = torch.Generator(device=device).manual_seed(seed)
    H, I = w.hidden, w.inter
    if w.fp8_block:
        def f8(r, c):       # a Gaussian scaled so that its tail reaches the format's 448, like a quantised block
            return (torch.randn(r, c, generator=g, device=device) * 110).clamp(-448, 448).to(torch.float8_e4m3fn)

        def sb(r, c):
            return torch.rand((r + 127) // 128, (c + 127) // 128, generator=g, device=device) * 3e-4 + 5e-5

        return ExpertWeight(up_w=f8(I, H), gate_w=f8(I, H), down_w=f8(H, I), up_scale=sb(I, H), gate_scale=sb(I, H),
                            down_scale=sb(H, I))
    if w.w8:
        def q(r, c):
            return torch.randint(-127, 128, (r, c), generator=g, device=device, dtype=torch.int8)

        def s(n):
            return (torch.rand(n, generator=g, device=device) * 3e-3 + 1e-3).to(torch.bfloat16)

        return ExpertWeight(up_w=q(I, H), gate_w=q(I, H), down_w=q(H, I), up_scale=s(I), gate_scale=s(I),
                            down_scale=s(H))

    def n(r, c):
        return (torch.randn(r, c, generator=g, device=device) * std).to(w.act_dtype)

    return ExpertWeight(up_w=n(I, H), gate_w=n(I, H), down_w=n(H, I))


def algorithmic_bytes(w: Workload, counts: torch.Tensor) -> int:
    """Weights of every active expert once + x in + ids/gate weights in + y out."""
    active = int((counts > 0).sum())
    a = 2
    return (active * w.expert_weight_bytes() + w.tokens * w.hidden * a + w.tokens * w.top_k * (4 + a)
            + w.tokens * w.hidden * a)


def expected_active(w: Workload) -> float:
    return w.n_experts * (1.0 - math.pow(1.0 - w.top_k / w.n_experts, w.tokens))
