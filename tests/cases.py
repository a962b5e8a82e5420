"""Seeded synthetic routing / payload generators shared by the CPU and GPU tests.

Kinds follow the reference's make_case vocabulary (nano_ep/testing/cases.py:29-55: random, masked,
skew, mixed) plus the benchmark workloads' routing (dropout mask, Zipf popularity, biased logits)."""

from __future__ import annotations

import torch


def routing(kind: str, tokens: int, experts: int, topk: int, seed: int = 0) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    if tokens == 0:
        return torch.empty((0, topk), dtype=torch.int64)
    if kind == "masked":
        return torch.full((tokens, topk), -1, dtype=torch.int64)
    if kind == "skew":
        # every token picks the same experts, in a non-sorted order
        base = torch.arange(topk, dtype=torch.int64).roll(1) % experts
        return base.repeat(tokens, 1).contiguous()
    scores = torch.rand(tokens, experts, generator=g)
    if kind == "zipf":
        popularity = 1.0 / torch.arange(1, experts + 1, dtype=torch.float64) ** 1.2
        idx = torch.multinomial(popularity.repeat(tokens, 1), topk, replacement=False, generator=g)
        return idx.to(torch.int64).contiguous()
    if kind == "biased":
        scores = torch.randn(tokens, experts, generator=g) + torch.randn(experts, generator=g) * 2.0
    idx = scores.topk(topk, dim=1).indices.to(torch.int64)
    if kind == "mixed":
        # even tokens use a fixed non-sorted pattern, token 0 of every 5 loses its middle choice
        pattern = (torch.arange(topk, dtype=torch.int64).flip(0) + 1) % experts
        idx[::2] = pattern
        idx[::5, topk // 2] = -1
    elif kind == "dropout":
        idx = torch.where(torch.rand(tokens, topk, generator=g) < 0.1, torch.full_like(idx, -1), idx)
    elif kind == "sparse":
        idx = torch.where(torch.rand(tokens, topk, generator=g) < 0.7, torch.full_like(idx, -1), idx)
    elif kind not in ("random", "biased"):
        raise ValueError(f"unknown routing kind {kind}")
    return idx.contiguous()


def payload(tokens: int, hidden: int, seed: int = 123, dtype=torch.bfloat16) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randn(tokens, hidden, generator=g, dtype=torch.float32).to(dtype)


def gate_weights(tokens: int, topk: int, seed: int = 7) -> torch.Tensor:
    """fp32 weights, intentionally nonzero at masked slots as in the reference's cases."""
    g = torch.Generator().manual_seed(seed)
    return torch.randn(tokens, topk, generator=g, dtype=torch.float32) + 0.3
