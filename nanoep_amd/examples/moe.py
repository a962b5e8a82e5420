"""A forward mixture-of-experts layer driven through the buffer, on one GPU:

    python -m nanoep_amd.examples.moe --layout expanded --cached --async-op

What it shows, and what the reference's example shows for several ranks
(nano_ep/examples/moe.py:96-160): activations are produced on one stream while dispatch, experts
and combine run on another and are tied to it only by events (`previous_event`, the results'
`current_stream_wait`); a handle may be kept and replayed (`--cached`); the expanded receive layout
is consumed segment by segment through `expert_offsets` / `expert_counts`, the way a grouped GEMM
would consume it; nothing is copied to the host between the steps of an iteration.  Every
iteration's output is kept and compared, after a single synchronisation at the end, with a dense
per-token evaluation that knows nothing about receive layouts.

Each expert is a gated affine map with its own seeded parameters (one scale and one shift per
channel), cheap enough that the run is about data movement.
"""

from __future__ import annotations

import argparse
import dataclasses
import json

import torch

from nanoep_amd import Buffer, EPConfig

PATTERNS = ("mixed", "skew", "masked", "uneven")
TOLERANCE = 0.03  # bf16 payloads: the reference's bound (nano_ep/examples/moe.py:150-153)


@dataclasses.dataclass
class Experts:
    """Per-expert channel parameters, fp32 [E, H]."""

    scale: torch.Tensor
    shift: torch.Tensor

    @classmethod
    def seeded(cls, count: int, hidden: int, device, seed: int = 2024) -> "Experts":
        generator = torch.Generator(device="cpu").manual_seed(seed)
        scale = 0.5 + torch.rand(count, hidden, generator=generator)
        shift = 0.25 * torch.randn(count, hidden, generator=generator)
        return cls(scale.to(device), shift.to(device))

    def forward_rows(self, rows: torch.Tensor, expert: int | torch.Tensor) -> torch.Tensor:
        """fp32 output of the given expert (one id, or one id per row) for bf16 rows."""
        return torch.sigmoid(rows.float() * self.scale[expert] + self.shift[expert]) * rows.float()


def grouped_forward(experts: Experts, received) -> torch.Tensor:
    """Expert outputs, already gate-weighted, in the receive layout of `received`."""
    handle = received.handle
    if not handle.do_expand:
        # compact: a received row carries all of its token's local choices
        total = torch.zeros(received.x.shape, dtype=torch.float32, device=received.x.device)
        for choice in range(handle.config.num_topk):
            ids = received.topk_idx[:, choice]
            chosen = ids >= 0
            term = experts.forward_rows(received.x, ids.clamp(min=0)) * received.topk_weights[:, choice, None]
            total += term * chosen[:, None]
        return total.to(received.x.dtype)
    # expanded: one segment of consecutive rows per expert, padded to the alignment; the segment
    # bounds stay on the device (a grouped GEMM would take the same two tensors)
    layout = handle.layout
    slot = torch.arange(received.x.shape[0], device=received.x.device)
    segment = torch.searchsorted(layout.expert_offsets[1:].contiguous(), slot, right=True)
    segment = segment.clamp(max=layout.expert_counts.numel() - 1)
    occupied = slot - layout.expert_offsets[segment] < layout.expert_counts[segment]
    out = experts.forward_rows(received.x, segment) * received.topk_weights[:, None]
    return (out * occupied[:, None]).to(received.x.dtype)


def dense_forward(experts: Experts, x, indices, weights) -> torch.Tensor:
    """The layer evaluated token by token at the source."""
    total = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    for choice in range(indices.shape[1]):
        ids = indices[:, choice]
        term = experts.forward_rows(x, ids.clamp(min=0)) * weights[:, choice, None]
        total += term * (ids >= 0)[:, None]
    return total.to(x.dtype)


def make_batch(options, step: int, device):
    """Seeded activations, routing and gate weights of one step.

    mixed: every token picks top-k of random scores, one choice in nine is masked;
    skew: all tokens pick the same experts; masked: no token picks anything;
    uneven: as mixed, with a few tokens fewer (the batch need not fill the buffer).
    """
    tokens = max(0, options.tokens - 3) if options.pattern == "uneven" else options.tokens
    # the routing is the same at every step (so that a kept handle stays valid); payload and gates change
    routing = torch.Generator(device="cpu").manual_seed(tokens)
    scores = torch.rand(tokens, options.experts, generator=routing)
    if options.pattern == "skew" and tokens:
        scores = scores[:1].expand(tokens, -1)
    indices = scores.topk(options.topk, dim=1).indices.to(torch.int64)
    if options.pattern == "masked":
        indices = torch.full_like(indices, -1)
    else:
        dropped = torch.rand(tokens, options.topk, generator=routing) < 1 / 9
        indices = indices.masked_fill(dropped, -1)
    payload = torch.Generator(device="cpu").manual_seed(1000 * step + 17)
    x = torch.randn(tokens, options.hidden, generator=payload).to(torch.bfloat16)
    gates = torch.rand(tokens, options.topk, generator=payload) + 0.1
    weights = gates / gates.sum(dim=1, keepdim=True)
    return x.to(device), indices.contiguous().to(device), weights.contiguous().to(device)


def parse_args(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--layout", choices=("compact", "expanded"), default="expanded")
    parser.add_argument("--pattern", choices=PATTERNS, default="mixed")
    parser.add_argument("--tokens", type=int, default=129)
    parser.add_argument("--hidden", type=int, default=1024)
    parser.add_argument("--experts", type=int, default=8)
    parser.add_argument("--topk", type=int, default=3)
    parser.add_argument("--alignment", type=int, default=16)
    parser.add_argument("--iterations", type=int, default=4)
    parser.add_argument("--cached", action="store_true", help="replay the first handle while the batch size allows")
    parser.add_argument("--async-op", action="store_true", help="run dispatch / combine on the buffer's stream, wait on their events")
    options = parser.parse_args(argv)
    if options.tokens < 0:
        parser.error("tokens must not be negative")
    for name in ("hidden", "experts", "topk", "alignment", "iterations"):
        if getattr(options, name) <= 0:
            parser.error(f"{name} must be positive")
    if options.hidden % 256:
        parser.error("hidden must be a multiple of 256")
    if options.topk > options.experts:
        parser.error("topk must not exceed experts")
    return options


@torch.no_grad()
def run(options) -> dict:
    device = torch.device("cuda", torch.cuda.current_device())
    expanded = options.layout == "expanded"
    experts = Experts.seeded(options.experts, options.hidden, device)
    produce, consume = torch.cuda.Stream(), torch.cuda.Stream()
    kept = []  # (output, expected output, returned weights, expected weights) of every step
    handle = None
    with Buffer(None, EPConfig(options.experts, options.topk, options.hidden, max(1, options.tokens))) as buffer:
        for step in range(options.iterations):
            with torch.cuda.stream(produce):
                x, indices, weights = make_batch(options, step, device)
                want = dense_forward(experts, x, indices, weights)
                want_weights = torch.where(indices >= 0, weights, torch.zeros_like(weights))
                produced = torch.cuda.Event()
                produced.record()
            with torch.cuda.stream(consume):
                reuse = handle if handle is not None and handle.topk_idx.shape == indices.shape else None
                received = buffer.dispatch(
                    x, weights=weights, topk_idx=None if reuse else indices, handle=reuse, do_expand=expanded,
                    alignment=options.alignment, zero_padding=expanded, previous_event=produced, async_op=options.async_op,
                )
                assert reuse is None or received.handle is reuse, "a replay returns the handle it was given"
                if received.event is not None:
                    received.event.current_stream_wait()
                result = buffer.combine(grouped_forward(experts, received), received.handle, weights=received.topk_weights,
                                        async_op=options.async_op)
                if result.event is not None:
                    result.event.current_stream_wait()
                kept.append((result.x, want, result.topk_weights, want_weights))
                if options.cached and handle is None:
                    handle = received.handle
                for tensor in (x, indices, weights):  # made on `produce`, read on `consume`
                    tensor.record_stream(consume)
            del x, indices, weights, received, result
            with torch.cuda.stream(produce):
                # hand the producer's memory out again while consumer work may still be queued
                torch.empty((max(1, options.tokens), options.hidden), device=device, dtype=torch.bfloat16).fill_(-77)
        torch.cuda.synchronize()
        for got, want, got_weights, want_weights in kept:
            torch.testing.assert_close(got, want, rtol=TOLERANCE, atol=TOLERANCE)
            torch.testing.assert_close(got_weights, want_weights, rtol=0, atol=0)
    return {"world_size": 1, **vars(options)}


if __name__ == "__main__":
    print("NANO_EP_MOE_OK=" + json.dumps(run(parse_args())), flush=True)
