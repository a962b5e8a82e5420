"""Geometry of one expert-parallel buffer (mirrors the reference's nano_ep/config.py:4-35)."""

from dataclasses import dataclass


@dataclass(frozen=True)
class EPConfig:
    """
    num_experts: experts in the whole group (all local at world_size == 1).
    num_topk: routing choices per token, at most min(32, num_experts).
    hidden: bf16 elements per token row.
    num_max_tokens_per_rank: upper bound on the source tokens of one dispatch.
    """

    num_experts: int
    num_topk: int
    hidden: int
    num_max_tokens_per_rank: int

    def __post_init__(self):
        if min(self.num_experts, self.num_topk, self.hidden, self.num_max_tokens_per_rank) <= 0:
            raise ValueError("EP dimensions and token capacity must be positive")
        if self.num_topk > min(32, self.num_experts):
            raise ValueError("num_topk must be <= min(32, num_experts)")
