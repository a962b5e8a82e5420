"""Forward mixture-of-experts loop on one GPU: `python -m nanoep_amd.examples.moe [--cached --async-op]`.

Follows the reference's example (nano_ep/examples/moe.py:96-160): inputs are produced on one stream,
dispatch / experts / combine run on another, cached handles and async events are optional, and the
result of every iteration is compared with a dense per-token evaluation at the end, after a single
device synchronisation.  Experts are cheap elementwise maps (tanh of an affine function of the
token, different per expert) so the example exercises the communication layouts, not GEMMs; the
expanded path walks the expert-major output with expert_offsets / expert_counts exactly as a
grouped GEMM would.
"""

from __future__ import annotations

import argparse
import json

import torch

from nanoep_amd import Buffer, EPConfig

PATTERNS = ("mixed", "skew", "masked", "uneven")


def expert_map(x: torch.Tensor, expert: torch.Tensor) -> torch.Tensor:
    """Expert `e` maps a row to tanh(x * (1 + e/32) + e/64), evaluated in fp32."""
    scale = (1 + expert.to(torch.float32) / 32).unsqueeze(-1)
    shift = (expert.to(torch.float32) / 64).unsqueeze(-1)
    return torch.tanh(x.to(torch.float32) * scale + shift)


def apply_experts(received) -> torch.Tensor:
    """Weighted expert outputs in the receive layout (padding rows become zero)."""
    handle = received.handle
    if handle.do_expand:
        layout = handle.layout
        rows = torch.arange(received.x.shape[0], device=received.x.device)
        expert = torch.bucketize(rows, layout.expert_offsets[1:], right=True).clamp(max=layout.expert_counts.numel() - 1)
        live = rows < layout.expert_offsets[expert] + layout.expert_counts[expert]
        out = expert_map(received.x, expert) * received.topk_weights.unsqueeze(-1)
        return torch.where(live.unsqueeze(-1), out, torch.zeros_like(out)).to(received.x.dtype)
    total = torch.zeros(received.x.shape, dtype=torch.float32, device=received.x.device)
    for k in range(handle.config.num_topk):
        expert = received.topk_idx[:, k]
        term = expert_map(received.x, expert.clamp(min=0)) * received.topk_weights[:, k].unsqueeze(-1)
        total += torch.where((expert >= 0).unsqueeze(-1), term, torch.zeros_like(term))
    return total.to(received.x.dtype)


def dense_answer(x, indices, weights) -> torch.Tensor:
    """Per-token evaluation that never looks at receive metadata."""
    total = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    for k in range(indices.shape[1]):
        expert = indices[:, k]
        term = expert_map(x, expert.clamp(min=0)) * weights[:, k].unsqueeze(-1)
        total += torch.where((expert >= 0).unsqueeze(-1), term, torch.zeros_like(term))
    return total.to(x.dtype)


def synthetic_batch(args, iteration, device):
    tokens = args.tokens
    if args.pattern == "uneven":
        tokens = max(0, tokens - 3)
    row = torch.arange(tokens, device=device)
    col = torch.arange(args.hidden, device=device)
    x = (((row[:, None] * 7 + col + iteration * 3) % 127 - 63) / 64).to(torch.bfloat16)
    experts = args.experts
    first = torch.zeros_like(row) if args.pattern == "skew" else row
    indices = ((first[:, None] + torch.arange(args.topk, device=device)) % experts).contiguous()
    if args.pattern == "masked":
        indices.fill_(-1)
    else:
        indices[:, -1].masked_fill_(row % 7 == 0, -1)
    weights = ((row[:, None] + torch.arange(args.topk, device=device) + iteration) % 5 + 1).float() / (5 * args.topk)
    return x.contiguous(), indices, weights.contiguous()


def parse_args(argv=None):
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--layout", choices=("compact", "expanded"), default="expanded")
    parser.add_argument("--tokens", type=int, default=129)
    parser.add_argument("--hidden", type=int, default=1024)
    parser.add_argument("--topk", type=int, default=3)
    parser.add_argument("--experts", type=int, default=8)
    parser.add_argument("--alignment", type=int, default=16)
    parser.add_argument("--iterations", type=int, default=4)
    parser.add_argument("--pattern", choices=PATTERNS, default="mixed")
    parser.add_argument("--async-op", action="store_true")
    parser.add_argument("--cached", action="store_true")
    args = parser.parse_args(argv)
    if args.tokens < 0 or min(args.hidden, args.topk, args.experts, args.alignment, args.iterations) <= 0:
        parser.error("tokens must be nonnegative; other dimensions/iterations must be positive")
    if args.hidden % 256 != 0:
        parser.error("hidden must be a multiple of 256")
    if args.topk > args.experts:
        parser.error("topk must not exceed experts")
    return args


@torch.no_grad()
def run(args) -> dict:
    device = torch.device("cuda", torch.cuda.current_device())
    config = EPConfig(args.experts, args.topk, args.hidden, max(1, args.tokens))
    producer, consumer = torch.cuda.Stream(), torch.cuda.Stream()
    expand = args.layout == "expanded"
    checks, handle = [], None
    with Buffer(None, config) as buffer:
        for iteration in range(args.iterations):
            with torch.cuda.stream(producer):
                x, indices, weights = synthetic_batch(args, iteration, device)
                expected = dense_answer(x, indices, weights)
                expected_weights = weights.masked_fill(indices < 0, 0)
                ready = torch.cuda.Event()
                ready.record()
            with torch.cuda.stream(consumer):
                if handle is not None and handle.topk_idx.shape[0] != x.shape[0]:
                    handle = None
                received = buffer.dispatch(
                    x, topk_idx=indices if handle is None else None, weights=weights, handle=handle,
                    do_expand=expand, alignment=args.alignment, zero_padding=expand, previous_event=ready, async_op=args.async_op,
                )
                if handle is not None and received.handle is not handle:
                    raise AssertionError("cached dispatch must preserve handle identity")
                if received.event is not None:
                    received.event.current_stream_wait()
                y = apply_experts(received)
                result = buffer.combine(y, received.handle, weights=received.topk_weights, async_op=args.async_op)
                if result.event is not None:
                    result.event.current_stream_wait()
                checks.append((result.x, expected, result.topk_weights, expected_weights))
                if args.cached:
                    handle = received.handle
                # x / weights were produced on another stream and are consumed here
                for tensor in (x, indices, weights):
                    tensor.record_stream(consumer)
            del x, indices, weights, y, received, result
            with torch.cuda.stream(producer):
                churn = torch.empty((max(1, args.tokens), args.hidden), device=device, dtype=torch.bfloat16)
                churn.fill_(-77)  # reuse producer memory while consumer work may still be pending
                del churn
        torch.cuda.synchronize()
        for actual, expected, actual_weights, expected_weights in checks:
            torch.testing.assert_close(actual, expected, rtol=0.03, atol=0.03)
            torch.testing.assert_close(actual_weights, expected_weights, rtol=0, atol=0)
    return {"world_size": 1, **vars(args)}


if __name__ == "__main__":
    print("NANO_EP_MOE_OK=" + json.dumps(run(parse_args())), flush=True)
