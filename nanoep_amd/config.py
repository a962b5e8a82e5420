"""Geometry of one expert-parallel buffer.

The four numbers and their constraints are the reference's (nano_ep/config.py:4-35): a caller's
`EPConfig(num_experts, num_topk, hidden, num_max_tokens_per_rank)` means the same thing here.
"""

from __future__ import annotations

import dataclasses

# The kernels gather up to 32 expert rows per token (two passes of 16).
MAX_TOPK = 32

_FIELDS = ("num_experts", "num_topk", "hidden", "num_max_tokens_per_rank")


@dataclasses.dataclass(frozen=True)
class EPConfig:
    """What a buffer is sized for.

    num_experts               experts of the whole group; with one rank all of them are local
    num_topk                  routing choices per token, 1 .. min(32, num_experts)
    hidden                    bf16 elements of one token row
    num_max_tokens_per_rank   most source tokens a single dispatch may carry
    """

    num_experts: int
    num_topk: int
    hidden: int
    num_max_tokens_per_rank: int

    def __post_init__(self) -> None:
        values = [getattr(self, name) for name in _FIELDS]
        if any(value <= 0 for value in values):
            raise ValueError("EP dimensions and token capacity must be positive")
        most = min(MAX_TOPK, self.num_experts)
        if self.num_topk > most:
            raise ValueError(f"num_topk must be <= min({MAX_TOPK}, num_experts)")

    @property
    def row_bytes(self) -> int:
        """Bytes of one bf16 token row."""
        return 2 * self.hidden
