"""CPU oracle for one rank's dispatch / combine.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module, and
only as the checker: the product path (nanoep_amd) never calls it and has no CPU fallback.

It restates, for world_size == 1, the reference's scalar-loop specification:

  layout_scalar   <- reference_layout      nano_ep/testing/oracle.py:70-104
  plan fields     <- reference_plan        nano_ep/testing/oracle.py:45-67   (send_counts)
  dispatch_scalar <- reference_dispatch    nano_ep/testing/oracle.py:107-147
  combine_scalar  <- reference_combine     nano_ep/testing/oracle.py:150-186 and
                     reference_combined    nano_ep/testing/native_combine.py:168-195
                     (allow_multiple_reduction, bias, returned weights)
  handle tensors  <- csrc/include/nano_ep/pipeline.hpp:13-21, nano_ep/testing/native_dispatch.py:79-133
  window_layout   <- csrc/layout.hpp:59-98 (known answer tests/unit/test_cuda_bootstrap.py:102-106)

Each *_scalar function is a plain Python loop used on small inputs; the function without the
suffix is the vectorised torch-CPU form of the same arithmetic (stable sort by expert,
index_select / index_copy_, K-step float32 accumulation in ascending k then one bf16 cast) and is
what the full-size parity tests and the CPU baseline time.

Pinning (see tests/test_oracle.py): closed-form layouts of the reference's
test_padding_gaps_across_expert_waves inputs, the finaliser closed form of
tests/native/test_receive_counts.py, the README identity round trip, the multiplicity round trip of
tests/distributed/worker.py:292-322, the 256+1-256 rounding probe, an independent integer
round-to-nearest-even, brute force scalar-vs-vectorised on random small cases, and the
window_layout known answer.  NaN bit patterns are not pinned: the reference compares with
equal_nan=True and so do we.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class Layout:
    """Everything reference_layout returns for rank 0 plus the seven handle tensors."""

    src_tokens: torch.Tensor  # int64 [N]
    local_topk_idx: torch.Tensor  # int64 [N,K]
    expanded_slots: torch.Tensor  # int64 [N,K]
    expert_counts: torch.Tensor  # int64 [L]
    expert_offsets: torch.Tensor  # int64 [L+1]
    dst_slots: torch.Tensor  # int64 [T,1]
    send_counts: torch.Tensor  # int64 [1]
    recv_rank_prefix: torch.Tensor  # int64 [1]
    topk_idx: torch.Tensor  # int64 [T,K] snapshot
    recv_count: int
    expanded_capacity: int

    def recv_metadata(self, expand: bool) -> torch.Tensor:
        """int32 [N,K+2] = [src_rank, src_token, slots | local ids]."""
        body = self.expanded_slots if expand else self.local_topk_idx
        head = torch.stack((torch.zeros_like(self.src_tokens), self.src_tokens), dim=1)
        return torch.cat((head, body), dim=1).to(torch.int32)

    def metadata(self, expand: bool) -> list[torch.Tensor]:
        """The seven handle tensors in the reference's order."""
        return [
            self.recv_metadata(expand),
            self.expert_counts,
            self.expert_offsets,
            self.dst_slots,
            self.send_counts,
            self.topk_idx,
            self.recv_rank_prefix,
        ]


# ---------------------------------------------------------------------------------------------
# layout
# ---------------------------------------------------------------------------------------------


def layout_scalar(topk_idx: torch.Tensor, num_local_experts: int, alignment: int = 1) -> Layout:
    tokens, topk = topk_idx.shape
    src_tokens, local_rows = [], []
    counts = [0] * num_local_experts
    dst = [-1] * tokens
    for token, row in enumerate(topk_idx.tolist()):
        localized = [e if 0 <= e < num_local_experts else -1 for e in row]
        if any(e >= 0 for e in localized):
            dst[token] = len(src_tokens)
            src_tokens.append(token)
            local_rows.append(localized)
            for expert in localized:
                if expert >= 0:
                    counts[expert] += 1
    offsets = [0]
    for count in counts:
        offsets.append(offsets[-1] + ((count + alignment - 1) // alignment) * alignment)
    slots = [[-1] * topk for _ in local_rows]
    next_slot = offsets[:-1].copy()
    for row_index, row in enumerate(local_rows):
        for k, expert in enumerate(row):
            if expert >= 0:
                slots[row_index][k] = next_slot[expert]
                next_slot[expert] += 1
    received = len(local_rows)
    return Layout(
        src_tokens=torch.tensor(src_tokens, dtype=torch.int64),
        local_topk_idx=torch.tensor(local_rows, dtype=torch.int64).reshape(-1, topk),
        expanded_slots=torch.tensor(slots, dtype=torch.int64).reshape(-1, topk),
        expert_counts=torch.tensor(counts, dtype=torch.int64),
        expert_offsets=torch.tensor(offsets, dtype=torch.int64),
        dst_slots=torch.tensor(dst, dtype=torch.int64).reshape(tokens, 1),
        send_counts=torch.tensor([received], dtype=torch.int64),
        recv_rank_prefix=torch.tensor([received], dtype=torch.int64),
        topk_idx=topk_idx.clone(),
        recv_count=received,
        expanded_capacity=offsets[-1],
    )


def layout(topk_idx: torch.Tensor, num_local_experts: int, alignment: int = 1) -> Layout:
    tokens, topk = topk_idx.shape
    valid = (topk_idx >= 0) & (topk_idx < num_local_experts)
    local = torch.where(valid, topk_idx, torch.full_like(topk_idx, -1))
    received = valid.any(dim=1)
    src_tokens = torch.nonzero(received).flatten()
    count = int(src_tokens.numel())
    dst = torch.where(received, torch.cumsum(received.to(torch.int64), 0) - 1, torch.full((tokens,), -1, dtype=torch.int64))
    flat_experts = local[valid]  # row-major: token order, then k
    counts = torch.bincount(flat_experts, minlength=num_local_experts).to(torch.int64)
    padded = (counts + alignment - 1) // alignment * alignment
    offsets = torch.cat((torch.zeros(1, dtype=torch.int64), torch.cumsum(padded, 0)))
    starts = torch.cumsum(counts, 0) - counts
    order = torch.argsort(flat_experts, stable=True)
    rank_in_expert = torch.empty_like(flat_experts)
    rank_in_expert[order] = torch.arange(flat_experts.numel(), dtype=torch.int64) - starts[flat_experts[order]]
    slots_all = torch.full_like(topk_idx, -1)
    slots_all[valid] = offsets[flat_experts] + rank_in_expert
    return Layout(
        src_tokens=src_tokens,
        local_topk_idx=local[src_tokens].reshape(-1, topk),
        expanded_slots=slots_all[src_tokens].reshape(-1, topk),
        expert_counts=counts,
        expert_offsets=offsets,
        dst_slots=dst.reshape(tokens, 1),
        send_counts=torch.tensor([count], dtype=torch.int64),
        recv_rank_prefix=torch.tensor([count], dtype=torch.int64),
        topk_idx=topk_idx.clone(),
        recv_count=count,
        expanded_capacity=int(offsets[-1]),
    )


# ---------------------------------------------------------------------------------------------
# dispatch
# ---------------------------------------------------------------------------------------------


def dispatch_scalar(x, topk_idx, num_local_experts, weights=None, *, do_expand=False, alignment=1):
    """Returns (x_out, topk_idx_out | None, weights_out | None, Layout); oracle padding is zero."""
    lay = layout_scalar(topk_idx, num_local_experts, alignment)
    rows = lay.expanded_capacity if do_expand else lay.recv_count
    data = x.new_zeros((rows, x.shape[1]))
    out_weights = None
    if weights is not None:
        out_weights = weights.new_zeros((rows,) if do_expand else (rows, topk_idx.shape[1]))
    for recv, token in enumerate(lay.src_tokens.tolist()):
        if do_expand:
            for k, slot in enumerate(lay.expanded_slots[recv].tolist()):
                if slot >= 0:
                    data[slot] = x[token]
                    if weights is not None:
                        out_weights[slot] = weights[token, k]
        else:
            data[recv] = x[token]
            if weights is not None:
                out_weights[recv] = weights[token]
    return data, (None if do_expand else lay.local_topk_idx.clone()), out_weights, lay


def dispatch(x, topk_idx, num_local_experts, weights=None, *, do_expand=False, alignment=1, lay: Layout | None = None):
    if lay is None:
        lay = layout(topk_idx, num_local_experts, alignment)
    if not do_expand:
        data = x.index_select(0, lay.src_tokens)
        out_weights = None if weights is None else weights.index_select(0, lay.src_tokens)
        return data, lay.local_topk_idx.clone(), out_weights, lay
    valid = lay.expanded_slots >= 0
    slots = lay.expanded_slots[valid]
    tokens = lay.src_tokens[:, None].expand_as(lay.expanded_slots)[valid]
    data = x.new_zeros((lay.expanded_capacity, x.shape[1]))
    data.index_copy_(0, slots, x.index_select(0, tokens))
    out_weights = None
    if weights is not None:
        out_weights = weights.new_zeros((lay.expanded_capacity,))
        out_weights[slots] = weights[lay.src_tokens][valid]
    return data, None, out_weights, lay


# ---------------------------------------------------------------------------------------------
# combine
# ---------------------------------------------------------------------------------------------


def combine_scalar(y, recv_metadata, dst_slots, *, do_expand, weights=None, bias=None, multiple_reduction=False):
    """y: bf16 [C,H] (expanded) or [N,H] (compact).  Returns (out bf16 [T,H], weights f32 [T,K] | None)."""
    tokens = dst_slots.shape[0]
    topk = recv_metadata.shape[1] - 2
    hidden = y.shape[1]
    result = torch.zeros((tokens, hidden), dtype=torch.float32)
    returned = None if weights is None else torch.zeros((tokens, topk), dtype=weights.dtype)
    meta = recv_metadata.tolist()
    for token in range(tokens):
        row = int(dst_slots[token, 0])
        if row < 0:
            continue
        fields = meta[row][2:]
        choices = [k for k, value in enumerate(fields) if value >= 0]
        if do_expand and not multiple_reduction:
            for k in choices:
                result[token] += y[fields[k]].to(torch.float32)
        elif do_expand:
            partial = torch.zeros(hidden, dtype=torch.float32)
            for k in choices:
                partial += y[fields[k]].to(torch.float32)
            if len(choices) >= 2:
                partial = partial.to(y.dtype).to(torch.float32)
            result[token] += partial
        else:
            result[token] += y[row].to(torch.float32)
        if weights is not None:
            for k in choices:
                returned[token, k] = weights[fields[k]] if do_expand else weights[row, k]
    if bias is not None:
        result += bias.to(torch.float32)
    return result.to(y.dtype), returned


def combine(y, recv_metadata, dst_slots, *, do_expand, weights=None, bias=None, multiple_reduction=False):
    tokens = dst_slots.shape[0]
    topk = recv_metadata.shape[1] - 2
    hidden = y.shape[1]
    rows = dst_slots[:, 0]
    received = rows >= 0
    safe_rows = torch.where(received, rows, torch.zeros_like(rows))
    if recv_metadata.shape[0] == 0:
        fields = torch.full((tokens, topk), -1, dtype=torch.int64)
    else:
        fields = recv_metadata[:, 2:].to(torch.int64)[safe_rows]
        fields = torch.where(received[:, None], fields, torch.full_like(fields, -1))
    valid = fields >= 0
    acc = torch.zeros((tokens, hidden), dtype=torch.float32)
    if do_expand:
        for k in range(topk):
            picked = torch.nonzero(valid[:, k]).flatten()
            if picked.numel():
                acc.index_add_(0, picked, y.index_select(0, fields[picked, k]).to(torch.float32))
        if multiple_reduction:
            several = valid.sum(dim=1) >= 2
            acc = torch.where(several[:, None], acc.to(y.dtype).to(torch.float32), acc)
    else:
        picked = torch.nonzero(received).flatten()
        if picked.numel():
            acc.index_add_(0, picked, y.index_select(0, rows[picked]).to(torch.float32))
    if bias is not None:
        acc += bias.to(torch.float32)
    returned = None
    if weights is not None:
        returned = torch.zeros((tokens, topk), dtype=weights.dtype)
        if do_expand:
            returned[valid] = weights[fields[valid]]
        else:
            gathered = weights[safe_rows] if weights.shape[0] else torch.zeros((tokens, topk), dtype=weights.dtype)
            returned = torch.where(valid, gathered, returned)
    return acc.to(y.dtype), returned


# ---------------------------------------------------------------------------------------------
# helpers
# ---------------------------------------------------------------------------------------------


def bf16_round_bits(values: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns by integer round-to-nearest-even (NaN -> 0x7FC0).

    Independent of torch's cast; used to pin the cast the combine oracle relies on.
    """
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    is_nan = (bits & 0x7FFFFFFF) > 0x7F800000
    return np.where(is_nan, 0x7FC0, rounded).astype(np.uint16)


def window_layout(ranks, tokens, hidden, topk, num_experts, allow_multiple_reduction=False):
    """[signal_offset, count_offset, payload_offset, return_offset, num_bytes] of the peer window."""

    def up32(value):
        return (value + 31) // 32 * 32

    notify = (ranks + num_experts) * 8
    reduction_offset = up32(ranks * 8)
    count_offset = up32(reduction_offset + notify)
    payload_offset = up32(count_offset + notify + ranks * 8)
    wire_row = up32(up32(up32(32 + topk * 8) + topk * 4) + hidden * 2)
    return_row = up32(up32(hidden * 2) + topk * 4)
    partitions = min(ranks, topk) if allow_multiple_reduction else topk
    arena = max(ranks * tokens * wire_row, partitions * tokens * return_row)
    return [0, count_offset, payload_offset, payload_offset, up32(payload_offset + arena)]
