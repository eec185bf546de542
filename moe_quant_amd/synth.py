"""Seeded synthetic inputs for the five benchmark configurations.

Tensors are drawn on the CPU with a torch.Generator in fp32 and cast to bf16, so the same
seed gives the same bits on every machine.  `scale` < 1 shrinks every dimension (kept a
multiple of 128) for CPU-sized parity twins of the full shapes.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _dim(full: int, scale: float, mult: int = 128) -> int:
    return max(mult, int(round(full * scale / mult)) * mult)


def outlier_channels(C: int, seed: int, frac: float = 0.01) -> torch.Tensor:
    k = math.ceil(frac * C)
    return torch.randperm(C, generator=_gen(seed))[:k]


def weight(R: int, C: int, seed: int, std: float = 0.02, dtype=torch.bfloat16) -> torch.Tensor:
    return (torch.randn(R, C, generator=_gen(seed)) * std).to(dtype)


def activations_outlier(n: int, C: int, seed: int, dtype=torch.bfloat16) -> torch.Tensor:
    """N(0,1) tokens with a seeded 1% of channels scaled x20."""
    x = torch.randn(n, C, generator=_gen(seed))
    x[:, outlier_channels(C, seed + 1)] *= 20.0
    return x.to(dtype)


def activations_swiglu(n: int, C: int, seed: int, dtype=torch.bfloat16) -> torch.Tensor:
    """SiLU(a)*b with a, b ~ N(0,1): the heavy-tailed input of a down projection."""
    g = _gen(seed)
    a = torch.randn(n, C, generator=g)
    b = torch.randn(n, C, generator=g)
    return (torch.nn.functional.silu(a) * b).to(dtype)


@dataclass
class LinearCase:
    name: str
    W: torch.Tensor  # (R, C) bf16
    X: torch.Tensor  # (n, C) bf16
    group_size: int = 128
    block_size: int = 128
    rel_damp: float = 0.01
    act_order: bool = False


def config1(scale: float = 1.0) -> LinearCase:
    """Single expert gate_proj: W 2048x7168, X 8192x7168 with outlier channels."""
    R, C, n = _dim(2048, scale), _dim(7168, scale), _dim(8192, scale)
    return LinearCase("cfg1_gate_proj", weight(R, C, 101), activations_outlier(n, C, 102))


def config2(scale: float = 1.0) -> LinearCase:
    """Expert down_proj + packing: W 7168x2048, X 65536x2048 SwiGLU product."""
    R, C, n = _dim(7168, scale), _dim(2048, scale), _dim(65536, scale)
    return LinearCase("cfg2_down_proj", weight(R, C, 201), activations_swiglu(n, C, 202))


MLA_SHAPES = {  # name: (R, C)
    "q_a_proj": (1536, 7168),
    "q_b_proj": (24576, 1536),
    "kv_a_proj_with_mqa": (576, 7168),
    "kv_b_proj": (32768, 512),
    "o_proj": (7168, 16384),
}


def config4(name: str, scale: float = 1.0) -> LinearCase:
    R, C = MLA_SHAPES[name]
    R, C, n = _dim(R, scale, 64), _dim(C, scale), _dim(16384, scale)
    seed = 400 + 10 * list(MLA_SHAPES).index(name)
    return LinearCase(f"cfg4_{name}", weight(R, C, seed), activations_outlier(n, C, seed + 1))


def config5(which: str, group_size: int, scale: float = 1.0) -> LinearCase:
    """Dense MLP with act-order: which in {'gate_up', 'down'}."""
    R, C = (18432, 7168) if which == "gate_up" else (7168, 18432)
    R, C, n = _dim(R, scale), _dim(C, scale), _dim(65536, scale)
    seed = 500 if which == "gate_up" else 510
    return LinearCase(
        f"cfg5_{which}_g{group_size}",
        weight(R, C, seed),
        activations_outlier(n, C, seed + 1),
        group_size=group_size,
        act_order=True,
    )


def moe_routing(n_tokens: int, n_experts: int = 256, top_k: int = 8, seed: int = 300, zipf_s: float = 1.1):
    """Top-k routing with softmax over N(0,1) logits plus a per-expert Zipf(s) log-bias.

    Returns (expert_ids (n_tokens, top_k) int64, counts (n_experts,) int64).
    Drawn in chunks so 2M tokens never materialise a 2M x 256 fp32 matrix more than once."""
    g = _gen(seed)
    ranks = torch.randperm(n_experts, generator=g).float() + 1.0
    bias = -zipf_s * torch.log(ranks)
    bias = bias - bias.mean()
    ids = torch.empty(n_tokens, top_k, dtype=torch.int64)
    step = 1 << 18
    for s in range(0, n_tokens, step):
        e = min(n_tokens, s + step)
        logits = torch.randn(e - s, n_experts, generator=g) + bias
        ids[s:e] = torch.topk(torch.softmax(logits, -1), top_k, dim=-1).indices
    counts = torch.bincount(ids.flatten(), minlength=n_experts)
    return ids, counts


def moe_layer_on_device(device, n_experts: int = 256, tokens: int = 2_097_152, hidden: int = 7168,
                        inter: int = 2048, top_k: int = 8, seed: int = 300, zipf_s: float = 1.1):
    """Config 3 generated directly in HBM (30 GB of tokens would take minutes over PCIe): returns
    (x (T, hidden) bf16, expert_ids (T, top_k) int64, [(gate, up, down) bf16]).  Same distributions as
    the CPU generators; seeded with a device generator, so bits are reproducible per device type."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    x = torch.empty(tokens, hidden, dtype=torch.bfloat16, device=device)
    outl = outlier_channels(hidden, seed + 1).to(device)
    step = 1 << 16
    for s in range(0, tokens, step):
        e = min(tokens, s + step)
        blk = torch.randn(e - s, hidden, generator=g, device=device)
        blk[:, outl] *= 20.0
        x[s:e] = blk.to(torch.bfloat16)
    ranks = torch.randperm(n_experts, generator=_gen(seed + 2)).float() + 1.0
    bias = -zipf_s * torch.log(ranks)
    bias = (bias - bias.mean()).to(device)
    ids = torch.empty(tokens, top_k, dtype=torch.int64, device=device)
    step = 1 << 18
    for s in range(0, tokens, step):
        e = min(tokens, s + step)
        logits = torch.randn(e - s, n_experts, generator=g, device=device) + bias
        ids[s:e] = torch.topk(torch.softmax(logits, -1), top_k, dim=-1).indices
    experts = []
    for _ in range(n_experts):
        gate = (torch.randn(inter, hidden, generator=g, device=device) * 0.02).to(torch.bfloat16)
        up = (torch.randn(inter, hidden, generator=g, device=device) * 0.02).to(torch.bfloat16)
        down = (torch.randn(hidden, inter, generator=g, device=device) * 0.02).to(torch.bfloat16)
        experts.append((gate, up, down))
    return x, ids, experts
