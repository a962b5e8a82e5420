"""What `dispatch` and `combine` hand back: the receive layout, the cached-routing handle, the two
result records and the completion event.

Class and field names are the reference's (nano_ep/backends/cuda.py:23-72), because callers read
them (`received.handle.layout.expert_offsets`, `result.topk_weights`, ...).  Letters used below:
T source tokens, K top-k, L local experts, R ranks (1 here), N received rows, C padded capacity of
the expanded layout.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Optional

import torch

from .config import EPConfig


@dataclasses.dataclass
class NativeLayout:
    """Where the received rows live.

    recv_metadata     int32 [N, K+2]: source rank, source token, then per choice the local expert
                      id (compact) or the expanded slot, -1 for a masked choice
    expert_counts     int64 [L] assignments per expert
    expert_offsets    int64 [L+1] first slot of each expert, counts rounded up to the alignment;
                      the last entry is C
    recv_rank_prefix  int64 [R] inclusive prefix of rows received per source rank
    recv_count        N as a Python int
    expanded_capacity C as a Python int
    """

    recv_metadata: torch.Tensor
    expert_counts: torch.Tensor
    expert_offsets: torch.Tensor
    recv_rank_prefix: torch.Tensor
    recv_count: int
    expanded_capacity: int


@dataclasses.dataclass
class NativeHandle:
    """Routing of one fresh dispatch, enough to replay it with other payloads and to combine.

    The first twelve fields are the reference's.  `token_slots` (int32 [T, K]: the slot of every
    (token, choice), -1 when masked) and `slot_order` (int64: every valid assignment as
    `(slot << 32) | (t * K + k)`, block of consecutive tokens by block and in ascending slot inside
    a block) exist on expanded handles made by this package only; the kernels run faster with them
    and give the same bytes without.
    """

    config: EPConfig
    rank: int
    world_size: int
    do_expand: bool
    alignment: int
    topk_idx: torch.Tensor  # int64 [T, K], the handle's own snapshot of the routing
    layout: NativeLayout
    dst_slots: torch.Tensor  # int64 [T, R], receive row of each token or -1
    send_counts: torch.Tensor  # int64 [R]
    owner: Any  # the buffer that made the handle
    x_dtype: torch.dtype
    num_sms: Optional[int] = None
    token_slots: Optional[torch.Tensor] = None
    slot_order: Optional[torch.Tensor] = None

    def tensors(self) -> list[torch.Tensor]:
        """The handle as the backend module takes it: the reference's seven tensors in the
        reference's order, then the private ones when the handle has them."""
        listed = [
            self.layout.recv_metadata,
            self.layout.expert_counts,
            self.layout.expert_offsets,
            self.dst_slots,
            self.send_counts,
            self.topk_idx,
            self.layout.recv_rank_prefix,
        ]
        table = getattr(self, "token_slots", None)
        order = getattr(self, "slot_order", None)
        if table is not None:
            listed.append(table)
            if order is not None:
                listed.append(order)
        return listed


class CudaEvent:
    """Completion of an `async_op=True` call.  `keepalive` pins what the queued work still reads."""

    def __init__(self, event, keepalive: tuple = ()):
        self.event = event
        self.keepalive = keepalive

    def current_stream_wait(self):
        """Order the caller's current stream after the call and tell the allocator that the
        results are used there."""
        self.event.current_stream_wait()


@dataclasses.dataclass
class NativeDispatchResult:
    """x [N, H] (compact) or [C, H] (expanded); topk_idx int64 [N, K] local ids, None when expanded;
    topk_weights [N, K] or [C], None when no weights were given."""

    x: torch.Tensor
    topk_idx: Optional[torch.Tensor]
    topk_weights: Optional[torch.Tensor]
    handle: NativeHandle
    event: Optional[CudaEvent]


@dataclasses.dataclass
class NativeCombineResult:
    """x [T, H]; topk_weights [T, K] with zeros at masked choices, None when no weights were given."""

    x: torch.Tensor
    topk_weights: Optional[torch.Tensor]
    event: Optional[CudaEvent]
