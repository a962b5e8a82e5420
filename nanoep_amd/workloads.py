"""Seeded synthetic workloads of the benchmark configurations and their algorithmic byte counts.

Shapes: T source tokens, H hidden (bf16), E experts (all local at world_size == 1), K top-k.
After routing: N received rows, A valid (token, k) assignments, C padded expanded capacity.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    tokens: int
    hidden: int
    experts: int
    topk: int
    routing: str  # "all", "uniform", "softmax-topk-dropout", "zipf", "biased-topk"
    expand: bool
    alignment: int
    zero_padding: bool
    description: str
    async_op: bool = False          # calls return a completion event that the consumer stream waits on
    combine_weights: bool = False   # combine is given the dispatched weights and returns them as [T, K]


WORKLOADS = {
    "readme-toy": Workload("readme-toy", 16, 256, 2, 2, "all", True, 1, True,
                           "16 x 256, 2 experts top-2, every token to experts [0,1], weights 0.5"),
    "mixtral": Workload("mixtral", 4096, 4096, 8, 2, "uniform", True, 1, False,
                        "4096 x 4096, 8 experts top-2 uniform distinct ids, expanded"),
    "deepseek-v3": Workload("deepseek-v3", 4096, 7168, 256, 8, "softmax-topk-dropout", True, 1, True,
                            "4096 x 7168, 256 experts top-8 of softmax(N(0,1)), 10% of choices masked, expanded + zero_padding"),
    "deepseek-v3-a128": Workload("deepseek-v3-a128", 4096, 7168, 256, 8, "softmax-topk-dropout", True, 128, True,
                                 "the deepseek-v3 batch with expert segments padded to multiples of 128 rows"),
    "ep8-share": Workload("ep8-share", 32768, 7168, 32, 8, "zipf", False, 1, False,
                          "32768 x 7168 (8 source segments x 4096), 32 local experts top-8 Zipf(1.2), compact, cached handle"),
    "qwen3-moe": Workload("qwen3-moe", 8192, 2048, 128, 8, "biased-topk", True, 128, True,
                          "8192 x 2048, 128 experts top-8 with per-expert bias, expanded, alignment 128, zero_padding, "
                          "async_op with the consumer waiting on the completion event, combine returning the weights",
                          async_op=True, combine_weights=True),
    # short payload rows: one and two 1 KiB chunks a row
    "short-rows-512": Workload("short-rows-512", 32768, 512, 64, 8, "softmax-topk-dropout", True, 1, True,
                               "32768 x 512, 64 experts top-8, 10% of choices masked, expanded + zero_padding"),
    "short-rows-1024": Workload("short-rows-1024", 32768, 1024, 64, 8, "softmax-topk-dropout", True, 1, True,
                                "32768 x 1024, 64 experts top-8, 10% of choices masked, expanded + zero_padding"),
    # the one shape the reference publishes latencies for (its chart: 256 tokens, hidden 4096, top-8, expanded, 2 GPUs)
    "latency-256": Workload("latency-256", 256, 4096, 64, 8, "softmax-topk-dropout", True, 1, False,
                            "256 x 4096, 64 experts top-8, 10% of choices masked, expanded: a latency point, not a bandwidth one"),
}


def make_inputs(workload: Workload, seed: int = 0):
    """CPU tensors (x bf16 [T,H], topk_idx int64 [T,K], weights f32 [T,K]) of one batch."""
    g = torch.Generator().manual_seed(seed)
    tokens, hidden, experts, topk = workload.tokens, workload.hidden, workload.experts, workload.topk
    x = torch.randn(tokens, hidden, generator=g, dtype=torch.float32).to(torch.bfloat16)
    if workload.routing == "all":
        idx = torch.arange(topk, dtype=torch.int64).repeat(tokens, 1)
        weights = torch.full((tokens, topk), 0.5, dtype=torch.float32)
        return x, idx.contiguous(), weights
    logits = torch.randn(tokens, experts, generator=g, dtype=torch.float32)
    if workload.routing == "uniform":
        idx = torch.rand(tokens, experts, generator=g).topk(topk, dim=1).indices
    elif workload.routing == "zipf":
        popularity = 1.0 / torch.arange(1, experts + 1, dtype=torch.float64) ** 1.2
        idx = torch.multinomial(popularity.repeat(tokens, 1), topk, replacement=False, generator=g)
    elif workload.routing == "biased-topk":
        logits = logits + torch.randn(experts, generator=g) * 2.0
        idx = torch.softmax(logits, dim=1).topk(topk, dim=1).indices
    elif workload.routing == "softmax-topk-dropout":
        idx = torch.softmax(logits, dim=1).topk(topk, dim=1).indices
    else:
        raise ValueError(f"unknown routing {workload.routing}")
    idx = idx.to(torch.int64)
    gates = torch.softmax(logits, dim=1).gather(1, idx)
    weights = (gates / gates.sum(dim=1, keepdim=True)).to(torch.float32)
    if workload.routing == "softmax-topk-dropout":
        # masked choices keep their (nonzero) weights, as in the reference's cases
        idx = torch.where(torch.rand(tokens, topk, generator=g) < 0.1, torch.full_like(idx, -1), idx)
    return x, idx.contiguous(), weights.contiguous()


def dispatch_bytes(w: Workload, received: int, assignments: int, capacity: int, *, weighted: bool = True, fresh: bool = False) -> int:
    """Bytes a dispatch must move: source rows read once, every destination row written once,
    routing ids, weights in and out, and (fresh only) the receive metadata."""
    row = 2 * w.hidden
    if w.expand:
        written = capacity if w.zero_padding else assignments
        total = row * (received + written) + 8 * w.tokens * w.topk
        if weighted:
            total += 4 * w.tokens * w.topk + 4 * capacity
    else:
        total = row * 2 * received + 8 * received * w.topk
        if weighted:
            total += 4 * w.tokens * w.topk + 4 * received * w.topk
    if fresh:
        total += 4 * received * (w.topk + 2)
    return total


def combine_bytes(w: Workload, received: int, assignments: int, *, weighted: bool = False, bias: bool = False) -> int:
    """Bytes a combine must move: every valid expert row read once, every source row written once."""
    row = 2 * w.hidden
    read_rows = assignments if w.expand else received
    total = row * (read_rows + w.tokens) + 4 * received * (w.topk + 2) + 8 * w.tokens * w.topk
    if bias:
        total += row * w.tokens
    if weighted:
        total += 4 * read_rows * (1 if w.expand else w.topk) + 4 * w.tokens * w.topk
    return total
