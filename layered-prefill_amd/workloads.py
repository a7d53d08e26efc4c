"""Synthetic inputs of the benchmark configurations, generated on the CPU from
a seeded ``torch.Generator`` so that they are identical on every machine.

Layer shape of configs 2-5: Qwen3-30B-A3B's MoE block (hidden 2048, 128
experts, expert intermediate 768, top-8 with renormalised softmax; the
reference builds it at nanovllm/models/qwen3_moe.py:66-98).  Router logits are
N(0,1) plus a per-expert bias ln q_e - mean(ln q) with q_e proportional to
rank_e^(-1.1) over a seeded permutation of the experts ("Zipf s=1.1" load
skew).  Weights are N(0, 0.02), activations N(0, 1).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass(frozen=True)
class LayerShape:
    hidden: int
    experts: int
    intermediate: int
    top_k: int


QWEN3_30B_A3B = LayerShape(hidden=2048, experts=128, intermediate=768, top_k=8)
TINY = LayerShape(hidden=256, experts=8, intermediate=128, top_k=2)

# name -> (shape, tokens, seed, dtype)
CONFIGS = {
    "tiny_fp32": (TINY, 64, 0, torch.float32),
    "decode_256": (QWEN3_30B_A3B, 256, 1, torch.bfloat16),
    "layered_8192p_256d": (QWEN3_30B_A3B, 8448, 2, torch.bfloat16),
}


def zipf_bias(experts: int, gen: torch.Generator, s: float = 1.1) -> torch.Tensor:
    rank = torch.randperm(experts, generator=gen).double() + 1.0
    logq = -s * torch.log(rank)
    logq = logq - torch.logsumexp(logq, 0)
    return (logq - logq.mean()).float()


def make_weights(shape: LayerShape, seed: int, dtype: torch.dtype):
    gen = torch.Generator().manual_seed(1000 + seed)
    E, H, I = shape.experts, shape.hidden, shape.intermediate
    w13 = torch.empty(E, 2 * I, H, dtype=torch.float32).normal_(0.0, 0.02, generator=gen).to(dtype)
    w2 = torch.empty(E, H, I, dtype=torch.float32).normal_(0.0, 0.02, generator=gen).to(dtype)
    return w13, w2


def make_inputs(shape: LayerShape, tokens: int, seed: int, dtype: torch.dtype,
                skew: Optional[bool] = None):
    """Returns (x [T,H] dtype, router_logits [T,E] fp32)."""
    gen = torch.Generator().manual_seed(seed)
    if skew is None:
        skew = shape.experts > 8
    x = torch.randn(tokens, shape.hidden, generator=gen, dtype=torch.float32).to(dtype)
    logits = torch.randn(tokens, shape.experts, generator=gen, dtype=torch.float32)
    if skew:
        logits = logits + zipf_bias(shape.experts, gen)
    return x, logits


def make_config(name: str):
    """(shape, x, router_logits, w13, w2) for a named configuration."""
    shape, tokens, seed, dtype = CONFIGS[name]
    x, logits = make_inputs(shape, tokens, seed, dtype)
    w13, w2 = make_weights(shape, seed, dtype)
    return shape, x, logits, w13, w2


def layer_flops(tokens: int, shape: LayerShape) -> int:
    """2*T*K*H*2I for the gate-up GEMM plus 2*T*K*I*H for the down GEMM."""
    return 6 * tokens * shape.top_k * shape.hidden * shape.intermediate


def layer_bytes(tokens: int, shape: LayerShape, n_active: int, weight_bytes: int = 2,
                act_bytes: int = 2) -> int:
    """Algorithmic HBM bytes of one layer call: every active expert's weights
    once, activations in, result out, router logits in (+ fp8 scales)."""
    H, I, E = shape.hidden, shape.intermediate, shape.experts
    b = n_active * 3 * H * I * weight_bytes + tokens * H * act_bytes * 2 + tokens * E * 4
    if weight_bytes == 1:
        b += n_active * (2 * I + H) * 4
    return b
