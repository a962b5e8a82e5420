"""GPU tests of the public API (EPConfig / Buffer.dispatch / Buffer.combine) against the CPU oracle.

The cases restate what the reference checks at world_size == 1: the README round trip
(README.md:44-70), fresh + cached replay with pointer-stable metadata and untouched earlier results
(tests/native/test_native_dispatch.py:93-208), async_op / previous_event stream handling and the
exact multiplicity round trip (tests/distributed/worker.py:180-343), plus the five benchmark shapes of nanoep_amd/workloads.py.
"""

import dataclasses

import pytest
import torch
from torch.utils import deterministic

import cases
from nanoep_amd import Buffer, CudaBuffer, EPConfig
from nanoep_amd._native import load_extension
from oracle import nanoep_oracle as oracle

pytestmark = pytest.mark.gpu


def bits(tensor):
    tensor = tensor.detach().cpu().contiguous()
    return tensor.view(torch.int16) if tensor.dtype == torch.bfloat16 else tensor.view(torch.int32)


def assert_same_bits(actual, expected, what=""):
    assert tuple(actual.shape) == tuple(expected.shape), what
    assert actual.dtype == expected.dtype, what
    assert torch.equal(bits(actual), bits(expected)), f"{what}: bit mismatch"


def assert_handle(handle, expected: oracle.Layout, expand, alignment, buffer):
    assert handle.owner is buffer and handle.do_expand is expand and handle.alignment == alignment
    assert (handle.rank, handle.world_size) == (0, 1)
    layout = handle.layout
    assert layout.recv_count == expected.recv_count and layout.expanded_capacity == expected.expanded_capacity
    got = [layout.recv_metadata, layout.expert_counts, layout.expert_offsets, handle.dst_slots, handle.send_counts,
           handle.topk_idx, layout.recv_rank_prefix]
    for actual, want in zip(got, expected.metadata(expand)):
        assert actual.is_cuda and actual.is_contiguous() and actual.dtype == want.dtype
        assert torch.equal(actual.cpu(), want)


def assert_dispatch_result(result, x, idx, weights, experts, expand, alignment, zero_padding):
    want_x, want_idx, want_w, lay = oracle.dispatch(x, idx, experts, weights, do_expand=expand, alignment=alignment)
    got_x = result.x.cpu()
    assert result.x.dtype == torch.bfloat16 and result.x.is_contiguous()
    if expand:
        assert result.topk_idx is None
        live = torch.zeros(lay.expanded_capacity, dtype=torch.bool)
        live[lay.expanded_slots[lay.expanded_slots >= 0]] = True
        assert got_x.shape == want_x.shape
        assert_same_bits(got_x[live], want_x[live], "expanded x")
        if weights is not None:
            assert_same_bits(result.topk_weights.cpu()[live], want_w[live], "expanded weights")
        if zero_padding:
            assert_same_bits(got_x[~live], want_x[~live], "gap rows are zero")
            if weights is not None:
                assert_same_bits(result.topk_weights.cpu()[~live], want_w[~live], "gap weights are zero")
    else:
        assert_same_bits(got_x, want_x, "compact x")
        assert torch.equal(result.topk_idx.cpu(), want_idx)
        if weights is not None:
            assert_same_bits(result.topk_weights, want_w, "compact weights")
    if weights is None:
        assert result.topk_weights is None
    return lay


def test_readme_round_trip(device):
    """The README toy shape (16 x 256, two experts, top-2): identity experts weighted once, combine reproduces x."""
    config = EPConfig(num_experts=2, num_topk=2, hidden=256, num_max_tokens_per_rank=16)
    x = cases.payload(16, 256, seed=0).to(device)
    indices = torch.tensor([[0, 1]], dtype=torch.int64).repeat(16, 1).to(device)
    weights = torch.full((16, 2), 0.5, dtype=torch.float32, device=device)
    with CudaBuffer(None, config) as buffer:
        received = buffer.dispatch(x, topk_idx=indices, weights=weights, do_expand=True, zero_padding=True)
        assert received.x.shape == (32, 256) and received.topk_weights.shape == (32,)
        expert_x = (received.x.float() * received.topk_weights[:, None]).to(received.x.dtype)
        result = buffer.combine(expert_x, received.handle)
        torch.testing.assert_close(result.x, x, rtol=0, atol=0)
        assert result.topk_weights is None and result.event is None


def test_readme_round_trip_with_a_gloo_control_group(device):
    """The reference's toy run as its README writes it: a single-member Gloo group handed to Buffer
    (README.md:44-70), identity experts, combine reproduces x.  Groups the build cannot serve (a
    second member is not available on one GPU; another backend is) are refused."""
    import torch.distributed as dist

    assert not dist.is_initialized()
    dist.init_process_group("gloo", store=dist.HashStore(), rank=0, world_size=1)
    try:
        group = dist.new_group(ranks=[0], backend="gloo")
        config = EPConfig(num_experts=2, num_topk=2, hidden=256, num_max_tokens_per_rank=16)
        x = cases.payload(16, 256, seed=0).to(device)
        indices = torch.tensor([[0, 1]], dtype=torch.int64).repeat(16, 1).to(device)
        weights = torch.full((16, 2), 0.5, dtype=torch.float32, device=device)
        for control in (group, dist.group.WORLD):
            with Buffer(control, config) as buffer:
                assert (buffer._rank, buffer._world_size) == (0, 1)
                received = buffer.dispatch(x, topk_idx=indices, weights=weights, do_expand=True, zero_padding=True)
                assert (received.handle.rank, received.handle.world_size) == (0, 1)
                expert_x = (received.x.float() * received.topk_weights[:, None]).to(received.x.dtype)
                result = buffer.combine(expert_x, received.handle)
                torch.testing.assert_close(result.x, x, rtol=0, atol=0)
        with pytest.raises(ValueError, match="divisible|hidden"):
            Buffer(group, EPConfig(num_experts=2, num_topk=2, hidden=128, num_max_tokens_per_rank=16))
    finally:
        dist.destroy_process_group()


@pytest.mark.parametrize(
    "expand,zero_padding,weighted,kind,hidden,alignment",
    [
        pytest.param(False, False, True, "mixed", 256, 1, id="compact-weighted"),
        pytest.param(False, False, False, "masked", 512, 4, id="compact-masked"),
        pytest.param(False, False, True, "skew", 768, 16, id="compact-skew"),
        pytest.param(True, False, True, "mixed", 512, 4, id="expanded-weighted"),
        pytest.param(True, False, False, "masked", 768, 16, id="expanded-masked"),
        pytest.param(True, True, True, "mixed", 768, 16, id="expanded-zero-padding"),
        pytest.param(True, True, False, "skew", 256, 4, id="expanded-skew"),
    ],
)
@pytest.mark.parametrize("walk", ["slot-order", "token-order"])
def test_fresh_and_cached_replay(device, tuning, walk, expand, zero_padding, weighted, kind, hidden, alignment):
    # the library walks the slot-order list of its own handles (fresh: device-side entry count,
    # replay: exact count); the switch covers the token-order walk with the slot table as well
    if walk == "token-order":
        tuning("DISPATCH_ORDER", "0")
    tokens, experts, topk = 19, 3, 3
    idx = cases.routing(kind, tokens, experts, topk, seed=2)
    x = cases.payload(tokens, hidden)
    w = cases.gate_weights(tokens, topk)
    buffer = Buffer(None, EPConfig(experts, topk, hidden, 32))
    try:
        idx_dev = idx.to(device)
        fresh = buffer.dispatch(
            x.to(device), topk_idx=idx_dev, weights=w.to(device) if weighted else None, do_expand=expand,
            alignment=alignment, zero_padding=zero_padding,
        )
        lay = assert_dispatch_result(fresh, x, idx, w if weighted else None, experts, expand, alignment, zero_padding)
        assert_handle(fresh.handle, lay, expand, alignment, buffer)
        handle = fresh.handle
        assert handle.num_sms == torch.cuda.get_device_properties(device).multi_processor_count
        assert handle.x_dtype == torch.bfloat16 and handle.config == buffer._config
        saved = [t.cpu().clone() for t in (fresh.x, fresh.topk_weights, fresh.topk_idx) if t is not None]
        metadata = [handle.layout.recv_metadata, handle.layout.expert_counts, handle.layout.expert_offsets, handle.dst_slots,
                    handle.send_counts, handle.topk_idx, handle.layout.recv_rank_prefix]
        pointers = [t.data_ptr() for t in metadata]
        saved_metadata = [t.cpu().clone() for t in metadata]
        idx_dev.fill_(99)  # the handle owns a snapshot: later edits of the caller's ids must not matter

        for step, replay_weighted in enumerate((not weighted, weighted), start=1):
            new_x, new_w = x + 2 * step, -w + step
            replay = buffer.dispatch(
                new_x.to(device), weights=new_w.to(device) if replay_weighted else None, handle=handle,
                zero_padding=zero_padding,
            )
            assert replay.handle is handle
            assert_dispatch_result(replay, new_x, idx, new_w if replay_weighted else None, experts, expand, alignment, zero_padding)
            assert [t.data_ptr() for t in metadata] == pointers
            for actual, expected in zip(metadata, saved_metadata):
                assert torch.equal(actual.cpu(), expected)
            # earlier results own their storage: later calls leave every byte of them alone
            for actual, expected in zip([t for t in (fresh.x, fresh.topk_weights, fresh.topk_idx) if t is not None], saved):
                assert torch.equal(actual.cpu().view(torch.uint8), expected.view(torch.uint8))

        # combine on the replayed layout, weights returned at their original k with masked slots zero
        rows = handle.layout.expanded_capacity if expand else handle.layout.recv_count
        y = cases.payload(rows, hidden, seed=77)
        yw = cases.gate_weights(rows, 1).flatten() if expand else cases.gate_weights(rows, topk)
        bias = cases.payload(tokens, hidden, seed=78)
        result = buffer.combine(y.to(device), handle, weights=yw.to(device), bias=bias.to(device))
        want, want_w = oracle.combine(y, lay.recv_metadata(expand), lay.dst_slots, do_expand=expand, weights=yw, bias=bias)
        assert_same_bits(result.x, want, "combined x")
        assert_same_bits(result.topk_weights, want_w, "combined weights")
    finally:
        buffer.close()


def held_rows(tensor, hidden):
    return tensor.untyped_storage().nbytes() // (2 * hidden)


@pytest.mark.parametrize("alignment,at_bound", [(1, True), (3, True), (4, False), (64, False)])
def test_fresh_dispatch_allocation_orders(device, alignment, at_bound):
    """A fresh dispatch allocates its outputs at their upper bound and narrows them while the
    alignment gaps add at most an eighth to that bound (the permute then runs right behind the
    layout), and exactly, after the host has the counts, beyond: same results, and never more than
    1.25 times the rows in use are held."""
    tokens, experts, topk, hidden = 40, 8, 4, 512
    assert (experts * (alignment - 1) * 8 <= tokens * topk) == at_bound
    idx = cases.routing("random", tokens, experts, topk, seed=alignment)
    idx[0, 0] = -1
    x = cases.payload(tokens, hidden)
    w = cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        fresh = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                                alignment=alignment, zero_padding=True)
        lay = assert_dispatch_result(fresh, x, idx, w, experts, True, alignment, True)
        assert_handle(fresh.handle, lay, True, alignment, buffer)
        bound = tokens * topk + experts * (alignment - 1)
        if at_bound:
            assert held_rows(fresh.x, hidden) >= bound > fresh.x.shape[0]
        else:
            assert held_rows(fresh.x, hidden) < bound
        assert fresh.x.untyped_storage().nbytes() <= 1.25 * fresh.x.nbytes + 512
        assert not buffer._runtime.prefers_exact_outputs()
        replay = buffer.dispatch(x.to(device), weights=w.to(device), handle=fresh.handle, zero_padding=True)
        assert torch.equal(replay.x.view(torch.int16), fresh.x.view(torch.int16))
        assert torch.equal(replay.topk_weights, fresh.topk_weights)


def test_fresh_dispatch_with_large_alignment_gaps_allocates_by_what_the_last_call_used(device):
    """Alignment 64 on 8 experts: the upper bound of the shapes is far from what routing fills, so the
    first call of a geometry allocates after the counts are known.  The next one allocates for what
    that call used plus an eighth, ahead of the counts, and keeps the result when the rows in use fit
    and fill four fifths of it; a batch that uses far fewer rows, or more than were allocated, is
    permuted again into exact outputs.  Every result is the oracle's and holds at most 1.25 times its rows."""
    tokens, experts, topk, hidden, alignment = 300, 8, 4, 512, 64
    x, w = cases.payload(tokens, hidden, seed=2), cases.gate_weights(tokens, topk)
    dense = cases.routing("random", tokens, experts, topk, seed=1)
    similar = cases.routing("random", tokens, experts, topk, seed=2)
    sparse = dense.clone()
    sparse[tokens // 3:] = -1
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        held = []
        for idx in (dense, similar, sparse, sparse, dense, dense):
            result = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                                     alignment=alignment, zero_padding=True)
            assert_dispatch_result(result, x, idx, w, experts, True, alignment, True)
            assert result.x.untyped_storage().nbytes() <= 1.25 * result.x.nbytes + 512
            held.append(held_rows(result.x, hidden) - result.x.shape[0])
            replay = buffer.dispatch(x.to(device), weights=w.to(device), handle=result.handle, zero_padding=True)
            assert torch.equal(replay.x.view(torch.int16), result.x.view(torch.int16))
        # first of a geometry: exact; same fill: early outputs kept; far fewer rows: exact; same again: early;
        # far more rows than allocated: exact; same again: early
        assert [extra > 0 for extra in held] == [False, True, False, True, False, True]
        # another geometry (other alignment) starts over
        other = buffer.dispatch(x.to(device), topk_idx=dense.to(device), do_expand=True, alignment=32)
        assert held_rows(other.x, hidden) == other.x.shape[0]


@pytest.mark.parametrize("switch,at_bound", [("0", False), ("1", True)], ids=["always-exact", "at-the-bound"])
def test_fresh_output_order_can_be_forced(device, tuning, switch, at_bound):
    """The FRESH_OUTPUTS switch at 0 allocates a fresh dispatch's outputs after the counts are known whatever
    the shapes, =1 at the bound whenever the alignment rule allows (a runtime that has turned to the
    exact order included): same results."""
    tuning("FRESH_OUTPUTS", switch)
    tokens, experts, topk, hidden = 200, 8, 4, 512
    idx = cases.routing("dropout", tokens, experts, topk, seed=6)
    x, w = cases.payload(tokens, hidden, seed=7), cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        for expand in (True, False):
            result = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=expand, zero_padding=True)
            assert_dispatch_result(result, x, idx, w, experts, expand, 1, True)
            if expand:  # some choices are masked: the rows in use are fewer than the bound
                assert result.x.shape[0] < tokens * topk
                assert (held_rows(result.x, hidden) >= tokens * topk) == at_bound


@pytest.mark.parametrize("expand", [False, True], ids=["compact", "expanded"])
def test_fresh_dispatch_never_holds_much_more_than_it_uses(device, expand):
    """With many masked choices the upper bound is far above what routing fills.  The call that finds
    that out permutes again into exact outputs, later calls allocate after the counts are known, and
    a batch that fills the bound again turns the runtime back: every result is the oracle's and
    holds at most 1.25 times its rows."""
    tokens, experts, topk, hidden = 96, 8, 4, 512
    sparse = cases.routing("random", tokens, experts, topk, seed=1)
    sparse[torch.rand(tokens, topk, generator=torch.Generator().manual_seed(5)) < 0.6] = -1
    sparse[::2] = -1  # half the tokens are not sent at all
    dense = cases.routing("random", tokens, experts, topk, seed=2)
    x, w = cases.payload(tokens, hidden, seed=3), cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        runtime = buffer._runtime
        for idx, exact_before, exact_after in ((sparse, False, True), (sparse, True, True), (dense, True, False), (dense, False, False)):
            assert runtime.prefers_exact_outputs() is exact_before
            result = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=expand, zero_padding=True)
            assert_dispatch_result(result, x, idx, w, experts, expand, 1, True)
            assert result.x.untyped_storage().nbytes() <= 1.25 * result.x.nbytes + 512
            assert result.topk_weights.untyped_storage().nbytes() <= 1.25 * result.topk_weights.nbytes + 512
            assert runtime.prefers_exact_outputs() is exact_after
            combined = buffer.combine(result.x, result.handle)
            lay = oracle.layout(idx, experts, 1)
            want, _ = oracle.combine(result.x.cpu(), lay.recv_metadata(expand), lay.dst_slots, do_expand=expand)
            assert_same_bits(combined.x, want, "combine after the allocation order changed")


def test_fresh_dispatch_launch_follows_the_share_of_valid_choices(device):
    """The permute of a fresh dispatch is enqueued before the host knows how many choices are valid;
    its launch is sized by the share the runtime saw last.  Batches whose share falls and rises
    again (so that the launch is too large, then too small) all give the oracle's result."""
    tokens, experts, topk, hidden = 600, 32, 8, 1024
    full = cases.routing("random", tokens, experts, topk, seed=3)
    x, w = cases.payload(tokens, hidden, seed=3), cases.gate_weights(tokens, topk)
    generator = torch.Generator().manual_seed(11)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        assert buffer._runtime.valid_share_65536() == 65536
        for masked in (0.0, 0.15, 0.15, 0.05, 0.0, 0.1):
            idx = torch.where(torch.rand(tokens, topk, generator=generator) < masked, torch.full_like(full, -1), full)
            result = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True, zero_padding=True)
            lay = assert_dispatch_result(result, x, idx, w, experts, True, 1, True)
            assert not buffer._runtime.prefers_exact_outputs()
            valid = int(lay.expert_counts.sum())
            assert buffer._runtime.valid_share_65536() == -(-valid * 65536 // (tokens * topk))


def test_headline_shapes_hold_at_most_a_quarter_more_than_they_use(device):
    """The DeepSeek-V3 batch with alignment 1 (at the bound) and 128 (exact order)."""
    from nanoep_amd import workloads

    for name in ("deepseek-v3", "deepseek-v3-a128"):
        work = workloads.WORKLOADS[name]
        x, idx, w = workloads.make_inputs(work)
        with Buffer(None, EPConfig(work.experts, work.topk, work.hidden, work.tokens)) as buffer:
            result = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                                     alignment=work.alignment, zero_padding=True)
            lay = oracle.layout(idx, work.experts, work.alignment)
            assert result.x.shape[0] == lay.expanded_capacity
            assert result.x.untyped_storage().nbytes() <= 1.25 * result.x.nbytes
            del result


@pytest.mark.parametrize("recall", [False, True], ids=["no-recall", "recall"])
@pytest.mark.parametrize("tokens,hidden", [(2048, 4096), (37, 512)], ids=["16MiB", "small"])
def test_replay_with_only_the_reference_handle_tensors(device, tuning, tokens, hidden, recall):
    """A handle that carries just the reference's seven tensors (as one that went through the
    reference's own Python class would) replays to the same bytes.  While it is one of the buffer's
    latest fresh dispatches the runtime hands its private tensors back (recall); otherwise the
    payload follows the handle's own dst_slots and recv_metadata in token order."""
    if not recall:
        tuning("RECALL_ORDER", "0")
    experts, topk, alignment = 16, 4, 8
    idx = cases.routing("dropout", tokens, experts, topk, seed=9)
    x, w = cases.payload(tokens, hidden, seed=4), cases.gate_weights(tokens, topk)
    buffer = Buffer(None, EPConfig(experts, topk, hidden, tokens))
    try:
        fresh = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                                alignment=alignment, zero_padding=True)
        bare = dataclasses.replace(fresh.handle, token_slots=None, slot_order=None)
        for step in (1, 2):
            new_x, new_w = x * step + 1, w - step
            replay = buffer.dispatch(new_x.to(device), weights=new_w.to(device), handle=bare, zero_padding=True)
            assert replay.handle is bare
            assert_dispatch_result(replay, new_x, idx, new_w, experts, True, alignment, True)
            full = buffer.dispatch(new_x.to(device), weights=new_w.to(device), handle=fresh.handle, zero_padding=True)
            assert torch.equal(replay.x.view(torch.int16), full.x.view(torch.int16))
            assert torch.equal(replay.topk_weights.view(torch.int32), full.topk_weights.view(torch.int32))
            assert buffer._runtime.private_recalls() == (step if recall else 0)
        # a fresh dispatch after such replays still reads its own counts
        again = buffer.dispatch(x.to(device), topk_idx=idx.flip(0).contiguous().to(device), do_expand=True, alignment=alignment)
        lay = oracle.layout(idx.flip(0).contiguous(), experts, alignment)
        assert again.handle.layout.recv_count == lay.recv_count and again.handle.layout.expanded_capacity == lay.expanded_capacity
        # ... the runtime remembers its latest few dispatches: the older handle is still recalled
        recalls = buffer._runtime.private_recalls()
        combined = buffer.combine(full.x, bare)
        want, _ = oracle.combine(full.x.cpu(), oracle.layout(idx, experts, alignment).recv_metadata(True),
                                 oracle.layout(idx, experts, alignment).dst_slots, do_expand=True)
        assert_same_bits(combined.x, want, "combine through the bare handle")
        late = buffer.dispatch(x.to(device), weights=w.to(device), handle=bare, zero_padding=True)
        assert_dispatch_result(late, x, idx, w, experts, True, alignment, True)
        assert buffer._runtime.private_recalls() == recalls + (2 if recall else 0)
        # and so is the latest one, by dispatch and by combine
        recalls = buffer._runtime.private_recalls()
        newest = dataclasses.replace(again.handle, token_slots=None, slot_order=None)
        newest_replay = buffer.dispatch(x.to(device), handle=newest)
        assert_dispatch_result(newest_replay, x, idx.flip(0).contiguous(), None, experts, True, alignment, False)
        rows = again.handle.layout.expanded_capacity
        y = cases.payload(rows, hidden, seed=12)
        flipped = oracle.layout(idx.flip(0).contiguous(), experts, alignment)
        want_newest, _ = oracle.combine(y, flipped.recv_metadata(True), flipped.dst_slots, do_expand=True)
        assert_same_bits(buffer.combine(y.to(device), newest).x, want_newest, "combine through the newest bare handle")
        assert buffer._runtime.private_recalls() == recalls + (2 if recall else 0)
        # after four more fresh dispatches whose handles are still alive the first handle has dropped
        # out of the runtime's memory (handles that died are forgotten first)
        alive = []
        for seed in range(4):
            other = cases.routing("dropout", tokens, experts, topk, seed=20 + seed)
            alive.append(buffer.dispatch(x.to(device), topk_idx=other.to(device), do_expand=True, alignment=alignment).handle)
        recalls = buffer._runtime.private_recalls()
        forgotten = buffer.dispatch(x.to(device), weights=w.to(device), handle=bare, zero_padding=True)
        assert_dispatch_result(forgotten, x, idx, w, experts, True, alignment, True)
        assert buffer._runtime.private_recalls() == recalls
    finally:
        buffer.close()


def test_a_foreign_seven_tensor_handle_is_followed_as_written(device):
    """A valid handle in another row and slot order than this library's own (here: receive rows and
    slots in reverse token order, as a caller may build them) is honoured by the host extension
    whatever the payload size: every row lands where the handle's recv_metadata says, and combine
    brings it back.  (A 16 MiB payload: nothing about the size of the batch changes that.)"""
    tokens, experts, topk, hidden, alignment = 2048, 16, 4, 4096, 4
    idx = cases.routing("dropout", tokens, experts, topk, seed=3)
    x, w = cases.payload(tokens, hidden, seed=6), cases.gate_weights(tokens, topk)
    lay = oracle.layout(idx, experts, alignment)
    # reversed rows: receive row r holds the (N-1-r)-th sending token; reversed slots inside every expert segment
    meta = lay.recv_metadata(True).flip(0).contiguous()
    counts, offsets = lay.expert_counts, lay.expert_offsets
    slots = meta[:, 2:].clone().to(torch.int64)
    expert_of = torch.bucketize(slots.clamp(min=0), offsets[1:], right=True)
    mirrored = offsets[expert_of] + counts[expert_of] - 1 - (slots - offsets[expert_of])
    meta[:, 2:] = torch.where(slots >= 0, mirrored, slots).to(torch.int32)
    dst = torch.where(lay.dst_slots >= 0, lay.recv_count - 1 - lay.dst_slots, lay.dst_slots)
    public = [meta, counts, offsets, dst, lay.send_counts, idx.clone(), lay.recv_rank_prefix]
    native = load_extension()
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        handle = [t.to(device) for t in public]
        stream = buffer.comm_stream.cuda_stream
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        outputs, returned, (received, capacity), event = native.dispatch(
            buffer._runtime, x.to(device), handle[5], w.to(device), experts, tokens, alignment, handle, lay.expanded_capacity,
            False, True, True, cus, stream, -1, False)
        assert event is None and (received, capacity) == (lay.recv_count, lay.expanded_capacity)
        got_x, got_w = outputs[0].cpu(), outputs[2].cpu()
        want_x = torch.zeros_like(got_x)
        want_w = torch.zeros_like(got_w)
        for row in range(meta.shape[0]):
            token = int(meta[row, 1])
            for k in range(topk):
                slot = int(meta[row, 2 + k])
                if slot >= 0:
                    want_x[slot] = x[token]
                    want_w[slot] = w[token, k]
        assert_same_bits(got_x, want_x, "rows follow the handle's recv_metadata")
        assert_same_bits(got_w, want_w, "weights follow the handle's recv_metadata")
        (combined, restored), _ = native.combine(buffer._runtime, outputs[0], handle, outputs[2], None, tokens, True, False, cus,
                                                 stream, -1, False)
        want, want_cw = oracle.combine(want_x, meta, dst, do_expand=True, weights=want_w)
        assert_same_bits(combined, want, "combine through the foreign handle")
        assert_same_bits(restored, want_cw, "weights restored through the foreign handle")


def reversed_handle(lay, idx):
    """The handle of `lay` with reversed receive rows and reversed slots inside every expert segment:
    coherent, and in another order than this library's own (the reference's expert_inputs builds its
    handles this way, nano_ep/testing/native_combine.py:62-74)."""
    meta = lay.recv_metadata(True).flip(0).contiguous()
    slots = meta[:, 2:].clone().to(torch.int64)
    expert_of = torch.bucketize(slots.clamp(min=0), lay.expert_offsets[1:], right=True)
    mirrored = lay.expert_offsets[expert_of] + lay.expert_counts[expert_of] - 1 - (slots - lay.expert_offsets[expert_of])
    meta[:, 2:] = torch.where(slots >= 0, mirrored, slots).to(torch.int32)
    dst = torch.where(lay.dst_slots >= 0, lay.recv_count - 1 - lay.dst_slots, lay.dst_slots)
    return [meta, lay.expert_counts, lay.expert_offsets, dst, lay.send_counts, idx.clone(), lay.recv_rank_prefix]


def test_a_reversed_handle_at_the_headline_shape_is_rebuilt_once_and_followed(device, tuning):
    """4096 x 7168, 256 experts, top-8 with masked choices, and a seven-tensor handle in reversed order:
    the runtime rebuilds the private tensors from the handle itself at the first replay and keeps
    them, every replay lands its rows where the handle says (vectorised closed form of the handle,
    which for the reversed handle is the oracle's dispatch with every expert segment mirrored), the
    walk that never rebuilds writes the same bytes, and combine brings the rows back."""
    tokens, experts, topk, hidden, alignment = 4096, 256, 8, 7168, 1
    idx = cases.routing("dropout", tokens, experts, topk, seed=31)
    lay = oracle.layout(idx, experts, alignment)
    public = reversed_handle(lay, idx)
    meta, dst = public[0], public[3]
    native = load_extension()
    cus = torch.cuda.get_device_properties(device).multi_processor_count

    def expected(x, w):
        rows = meta[:, 1].to(torch.int64)[:, None].expand(-1, topk)
        slots = meta[:, 2:].to(torch.int64)
        live = slots >= 0
        want_x = torch.zeros((lay.expanded_capacity, hidden), dtype=torch.bfloat16)
        want_w = torch.zeros(lay.expanded_capacity, dtype=torch.float32)
        want_x[slots[live]] = x[rows[live]]
        ks = torch.arange(topk)[None, :].expand_as(slots)
        want_w[slots[live]] = w[rows[live], ks[live]]
        return want_x, want_w

    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        handle = [t.to(device) for t in public]
        stream = buffer.comm_stream.cuda_stream
        first = None
        for step in (1, 2, 3):
            x = cases.payload(tokens, hidden, seed=40 + step)
            w = cases.gate_weights(tokens, topk, seed=step)
            if step == 3:
                tuning("REBUILD_ORDER", 0)  # the token-order walk through the handle's own tensors
            outputs, returned, (received, capacity), event = native.dispatch(
                buffer._runtime, x.to(device), handle[5], w.to(device), experts, tokens, alignment, handle, lay.expanded_capacity,
                False, True, True, cus, stream, -1, False)
            assert all(a is b for a, b in zip(returned, handle)) and len(returned) == 7
            want_x, want_w = expected(x, w)
            assert_same_bits(outputs[0], want_x, f"replay {step} rows follow the handle")
            assert_same_bits(outputs[2], want_w, f"replay {step} weights follow the handle")
            assert buffer._runtime.rebuilds() == 1
            first = first or (outputs, want_x, want_w)
        tuning("REBUILD_ORDER", -1)
        outputs, want_x, want_w = first
        (combined, restored), _ = native.combine(buffer._runtime, outputs[0], handle, outputs[2], None, tokens, True, False, cus,
                                                 stream, -1, False)
        want, want_cw = oracle.combine(want_x, meta, dst, do_expand=True, weights=want_w)
        assert_same_bits(combined, want, "combine through the reversed handle")
        assert_same_bits(restored, want_cw, "weights restored through the reversed handle")
        assert buffer._runtime.rebuilds() == 1
        # editing the handle through torch makes it another handle: it is rebuilt
        handle[3].copy_(handle[3])
        native.dispatch(buffer._runtime, x.to(device), handle[5], None, experts, tokens, alignment, handle, lay.expanded_capacity,
                        False, True, False, cus, stream, -1, False)
        assert buffer._runtime.rebuilds() == 2


def test_the_fifth_oldest_handle_of_a_buffer_still_takes_the_slot_order_walk(device):
    """A caller that keeps five seven-tensor handles alive (one per layer, say): the runtime
    remembers the private tensors of its latest four, the oldest one has them rebuilt from the
    handle itself, once, and every replay equals the oracle."""
    tokens, experts, topk, hidden, alignment = 2048, 32, 4, 4096, 16
    x, w = cases.payload(tokens, hidden, seed=8), cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        routings = [cases.routing("dropout", tokens, experts, topk, seed=50 + layer) for layer in range(5)]
        bare = []
        for idx in routings:
            fresh = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True, alignment=alignment)
            bare.append(dataclasses.replace(fresh.handle, token_slots=None, slot_order=None))
        for _ in range(2):
            for layer in (4, 3, 2, 1, 0):
                replay = buffer.dispatch(x.to(device), weights=w.to(device), handle=bare[layer], zero_padding=True)
                assert_dispatch_result(replay, x, routings[layer], w, experts, True, alignment, True)
        assert buffer._runtime.rebuilds() == 1 and buffer._runtime.private_recalls() == 8


def test_a_compute_unit_budget_confines_the_kernels_and_changes_no_result(device):
    """num_sms below the device's compute units: the call runs on a stream created with a CU mask of
    about that many units (the same number on every XCD).  Results are the oracle's whatever the
    budget, synchronous or not, calls with different budgets stay ordered one behind the other, and
    the kernel time grows as the budget shrinks (a 16 MiB payload on a quarter of the device takes
    about twice as long as on all of it: 1.9 to 2.2 times in practice, half again as long is asked for)."""
    tokens, experts, topk, hidden, alignment = 2048, 16, 4, 4096, 8
    idx = cases.routing("dropout", tokens, experts, topk, seed=4)
    x, w = cases.payload(tokens, hidden, seed=5), cases.gate_weights(tokens, topk)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        quarter = cus // 4
        assert buffer._runtime.budget_stream_cus(quarter) == quarter and buffer._runtime.budget_stream(cus) == 0
        assert buffer.budget_stream(quarter) is not buffer.comm_stream and buffer.budget_stream(cus) is buffer.comm_stream
        fresh = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True, alignment=alignment,
                                zero_padding=True, num_sms=quarter)
        lay = assert_dispatch_result(fresh, x, idx, w, experts, True, alignment, True)
        assert fresh.handle.num_sms == quarter
        for budget, asynchronous in ((quarter, True), (cus, True), (cus // 2, False), (None, False), (cus, False), (quarter, True)):
            replay = buffer.dispatch((x * 2).to(device), weights=w.to(device), handle=fresh.handle, zero_padding=True,
                                     num_sms=budget, async_op=asynchronous)
            if asynchronous:
                replay.event.current_stream_wait()
            assert_dispatch_result(replay, x * 2, idx, w, experts, True, alignment, True)
            combined = buffer.combine(replay.x, fresh.handle, weights=replay.topk_weights, num_sms=budget, async_op=asynchronous)
            if asynchronous:
                combined.event.current_stream_wait()
            want, want_w = oracle.combine(replay.x.cpu(), lay.recv_metadata(True), lay.dst_slots, do_expand=True, weights=replay.topk_weights.cpu())
            assert_same_bits(combined.x, want, f"combine with budget {budget}")
            assert_same_bits(combined.topk_weights, want_w, f"combine weights with budget {budget}")

        def kernel_us(budget):
            stream = buffer.budget_stream(budget)
            payload = x.to(device)
            with torch.cuda.stream(stream):
                for _ in range(5):
                    buffer.dispatch(payload, handle=fresh.handle, num_sms=budget)
                begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                begin.record(stream)
                for _ in range(20):
                    buffer.dispatch(payload, handle=fresh.handle, num_sms=budget)
                end.record(stream)
                torch.cuda.synchronize()
            return begin.elapsed_time(end) * 1e3 / 20

        whole, confined = kernel_us(cus), kernel_us(quarter)
        assert confined > 1.5 * whole, (whole, confined)


@pytest.mark.parametrize("expand", [False, True], ids=["compact", "expanded"])
def test_async_streams_and_previous_event(device, expand):
    tokens, experts, topk, hidden = 301, 16, 4, 1024
    idx = cases.routing("dropout", tokens, experts, topk, seed=5)
    x_cpu = cases.payload(tokens, hidden)
    w_cpu = cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, 512)) as buffer:
        producer, consumer = torch.cuda.Stream(), torch.cuda.Stream()
        with torch.cuda.stream(producer):
            x, w, idx_dev = x_cpu.to(device, non_blocking=True), w_cpu.to(device), idx.to(device)
            torch.cuda._sleep(2_000_000)  # make a missing dependency on the producer visible
            x = x * 1
            ready = torch.cuda.Event()
            ready.record()
        with torch.cuda.stream(consumer):
            received = buffer.dispatch(
                x, topk_idx=idx_dev, weights=w, do_expand=expand, alignment=8, zero_padding=expand,
                previous_event=ready, async_op=True,
            )
            assert received.event is not None
            assert any(item is received.handle for item in received.event.keepalive)
            received.event.current_stream_wait()
            lay = assert_dispatch_result(received, x_cpu, idx, w_cpu, experts, expand, 8, expand)
            y = received.x * 1
            combined = buffer.combine(y, received.handle, weights=received.topk_weights, async_op=True)
            combined.event.current_stream_wait()
            want, want_w = oracle.combine(
                oracle.dispatch(x_cpu, idx, experts, w_cpu, do_expand=expand, alignment=8)[0],
                lay.recv_metadata(expand), lay.dst_slots, do_expand=expand,
                weights=oracle.dispatch(x_cpu, idx, experts, w_cpu, do_expand=expand, alignment=8)[2],
            )
            assert_same_bits(combined.x, want, "async combine")
            assert_same_bits(combined.topk_weights, want_w, "async combine weights")
            expected_weights = w_cpu.masked_fill(idx < 0, 0)
            assert_same_bits(combined.topk_weights, expected_weights, "weights return to their source slot")
        torch.cuda.synchronize()


def test_exact_multiplicity_round_trip(device):
    """combine(dispatch(x)) == x * multiplicity + bias exactly in bf16 for small-integer x."""
    tokens, experts, topk, hidden = 64, 6, 3, 256
    idx = cases.routing("mixed", tokens, experts, topk, seed=31)
    x_cpu = torch.full((tokens, hidden), 3, dtype=torch.bfloat16)
    with Buffer(None, EPConfig(experts, topk, hidden, 64)) as buffer:
        for expand in (False, True):
            received = buffer.dispatch(x_cpu.to(device) + 0, topk_idx=idx.to(device), do_expand=expand, alignment=4,
                                       zero_padding=expand, async_op=True)
            scratch = torch.empty_like(x_cpu, device=device)
            scratch.fill_(-77)  # allocator churn while the communication stream may still be busy
            received.event.current_stream_wait()
            assert received.topk_weights is None
            combined = buffer.combine(received.x, received.handle, bias=torch.ones_like(x_cpu, device=device), async_op=expand)
            if expand:
                combined.event.current_stream_wait()
            valid = (idx >= 0).sum(dim=1)
            multiplicity = valid if expand else (valid > 0).to(torch.int64)
            expected = x_cpu * multiplicity.to(torch.bfloat16).unsqueeze(1) + 1
            torch.testing.assert_close(combined.x.cpu(), expected, rtol=0, atol=0)
            assert combined.topk_weights is None


def test_rounding_probe_and_multiple_reduction(device):
    """256 + 1 - 256: fp32 accumulation keeps the 1 that a bf16 partial sum would lose; the
    allow_multiple_reduction mode rounds the partial sum to bf16 before the bias and may lose it."""
    hidden = 256
    idx = torch.tensor([[0, 1, 2]], dtype=torch.int64)
    for multi, expected in ((False, 1.0 + 0.5), (True, 1.0 + 0.5)):
        with Buffer(None, EPConfig(3, 3, hidden, 4), allow_multiple_reduction=multi) as buffer:
            x = torch.zeros((1, hidden), dtype=torch.bfloat16, device=device)
            received = buffer.dispatch(x, topk_idx=idx.to(device), do_expand=True)
            y = torch.empty((3, hidden), dtype=torch.bfloat16, device=device)
            slots = received.handle.layout.recv_metadata[0, 2:].tolist()
            y[slots[0]] = 256.0
            y[slots[1]] = 1.0
            y[slots[2]] = -256.0
            bias = torch.full((1, hidden), 0.5, dtype=torch.bfloat16, device=device)
            out = buffer.combine(y, received.handle, bias=bias).x
            assert torch.all(out.float() == expected), (multi, out[0, :4])
    # a partial sum that is not representable in bf16: 256 + 1 = 257 rounds to 256 before the bias
    with Buffer(None, EPConfig(3, 3, hidden, 4), allow_multiple_reduction=True) as buffer:
        idx2 = torch.tensor([[0, 1, -1]], dtype=torch.int64)
        received = buffer.dispatch(torch.zeros((1, hidden), dtype=torch.bfloat16, device=device), topk_idx=idx2.to(device), do_expand=True)
        slots = received.handle.layout.recv_metadata[0, 2:].tolist()
        y = torch.zeros((2, hidden), dtype=torch.bfloat16, device=device)
        y[slots[0]] = 256.0
        y[slots[1]] = 1.0
        bias = torch.full((1, hidden), 1.0, dtype=torch.bfloat16, device=device)
        out = buffer.combine(y, received.handle, bias=bias).x
        assert torch.all(out.float() == 256.0)  # bf16(256 + 1) = 256, then bf16(256 + 1) = 256
    with Buffer(None, EPConfig(3, 3, hidden, 4)) as buffer:
        received = buffer.dispatch(torch.zeros((1, hidden), dtype=torch.bfloat16, device=device), topk_idx=idx2.to(device), do_expand=True)
        out = buffer.combine(y, received.handle, bias=bias).x
        assert torch.all(out.float() == 258.0)  # bf16(256 + 1 + 1) = 258


def test_argument_errors(device):
    config = EPConfig(4, 2, 256, 8)
    buffer, other = Buffer(None, config), Buffer(None, config)
    x = cases.payload(8, 256).to(device)
    idx = cases.routing("random", 8, 4, 2).to(device)
    try:
        with pytest.raises(ValueError, match="requires topk_idx"):
            buffer.dispatch(x)
        with pytest.raises(ValueError, match="alignment"):
            buffer.dispatch(x, topk_idx=idx, alignment=0)
        with pytest.raises(ValueError, match="do_expand"):
            buffer.dispatch(x, topk_idx=idx, do_expand=1)
        with pytest.raises(ValueError, match="hidden"):
            buffer.dispatch(x[:, :128].contiguous(), topk_idx=idx)
        with pytest.raises(ValueError, match="shape"):
            buffer.dispatch(x, topk_idx=idx[:, :1].contiguous())
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        for bad in (-1, cus + 1, True, 1.5):
            with pytest.raises(ValueError, match="num_sms"):
                buffer.dispatch(x, topk_idx=idx, num_sms=bad)
        received = buffer.dispatch(x, topk_idx=idx, do_expand=True, alignment=4, num_sms=7)
        assert received.handle.num_sms == 7
        assert buffer.dispatch(x, topk_idx=idx, num_sms=0).handle.num_sms == cus
        with pytest.raises(ValueError, match="another CudaBuffer"):
            other.dispatch(x, handle=received.handle)
        with pytest.raises(ValueError, match="omit topk_idx"):
            buffer.dispatch(x, topk_idx=idx, handle=received.handle)
        with pytest.raises(ValueError, match="alignment"):
            buffer.dispatch(x, handle=received.handle, alignment=8)
        with pytest.raises(ValueError, match="layout"):
            buffer.dispatch(x, handle=received.handle, do_expand=False)
        with pytest.raises(ValueError, match="bfloat16"):
            buffer.combine(received.x.float(), received.handle)
        with pytest.raises(ValueError, match="another CudaBuffer"):
            other.combine(received.x, received.handle)
        with pytest.raises(ValueError, match="weights"):
            buffer.combine(received.x, received.handle, weights=torch.zeros(3, device=device))
        with pytest.raises(ValueError, match="bias"):
            buffer.combine(received.x, received.handle, bias=torch.zeros((8, 256), device=device))
        # data-dependent routing errors come back as RuntimeError instead of a device trap
        bad_idx = idx.clone()
        bad_idx[0, 0] = 4
        with pytest.raises(RuntimeError, match="out of range"):
            buffer.dispatch(x, topk_idx=bad_idx)
        bad_idx[0] = 1
        with pytest.raises(RuntimeError, match="duplicate"):
            buffer.dispatch(x, topk_idx=bad_idx)
        # the buffer stays usable after a rejected routing
        again = buffer.dispatch(x, topk_idx=idx, do_expand=True, alignment=4)
        assert again.handle.layout.recv_count == received.handle.layout.recv_count
        buffer.close()
        buffer.close()
        with pytest.raises(RuntimeError, match="closed"):
            buffer.dispatch(x, topk_idx=idx)
        with pytest.raises(RuntimeError, match="closed"):
            buffer.combine(received.x, received.handle)
    finally:
        buffer.close()
        other.close()
    with pytest.raises(TypeError):
        Buffer(None, config, allow_multiple_reduction=1)
    with pytest.raises(ValueError, match="256"):
        Buffer(None, EPConfig(4, 2, 128, 8))


@pytest.mark.parametrize("seed", range(12))
def test_randomized_shapes_through_the_api(device, seed):
    """Odd token counts, expert counts, top-k and alignments through fresh dispatch, replay and
    combine: the handle's tensors are carved out of one allocation whose sections move with every
    one of these numbers."""
    generator = torch.Generator().manual_seed(1000 + seed)

    def pick(options):
        return options[int(torch.randint(len(options), (1,), generator=generator))]

    topk = pick([1, 2, 3, 4, 5, 7, 8])
    experts = max(topk, pick([3, 8, 17, 64, 129]))
    tokens = pick([1, 5, 33, 255, 256, 257, 777, 1500])
    hidden = pick([256, 512, 1280])
    alignment = pick([1, 1, 3, 8, 16])
    kind = pick(["random", "dropout", "sparse", "mixed"])
    expand = pick([True, True, False])
    idx = cases.routing(kind, tokens, experts, topk, seed=seed)
    x, w = cases.payload(tokens, hidden, seed=seed), cases.gate_weights(tokens, topk, seed=seed)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens + 3)) as buffer:
        for weighted in (True, False):
            gate = w if weighted else None
            fresh = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=None if gate is None else gate.to(device),
                                    do_expand=expand, alignment=alignment, zero_padding=expand)
            lay = assert_dispatch_result(fresh, x, idx, gate, experts, expand, alignment, expand)
            assert_handle(fresh.handle, lay, expand, alignment, buffer)
            replay = buffer.dispatch((x * 2).to(device), weights=None if gate is None else gate.to(device), handle=fresh.handle,
                                     zero_padding=expand)
            assert_dispatch_result(replay, x * 2, idx, gate, experts, expand, alignment, expand)
            combined = buffer.combine(fresh.x, fresh.handle, weights=fresh.topk_weights)
            want, want_w = oracle.combine(fresh.x.cpu(), lay.recv_metadata(expand), lay.dst_slots, do_expand=expand,
                                          weights=None if gate is None else fresh.topk_weights.cpu())
            assert_same_bits(combined.x, want, "combined x")
            if weighted:
                assert_same_bits(combined.topk_weights, want_w, "combined weights")


def test_fresh_dispatches_of_two_threads_on_one_buffer(device):
    """dispatch runs without the interpreter lock, and a buffer has one mailbox for N and C: fresh
    dispatches of two Python threads take turns at it, and each gets the counts and the layout of
    its own routing."""
    import threading

    tokens, experts, topk, hidden = 700, 32, 4, 512
    routings = [cases.routing("dropout", tokens - 100 * i, experts, topk, seed=40 + i) for i in range(2)]
    for i, idx in enumerate(routings):
        idx[: 50 * (i + 1)] = -1  # different N and C per thread
    xs = [cases.payload(idx.shape[0], hidden, seed=i) for i, idx in enumerate(routings)]
    expected = [oracle.layout(idx, experts, 4) for idx in routings]
    assert expected[0].recv_count != expected[1].recv_count
    failures = []
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        start = threading.Barrier(2)

        def worker(which):
            try:
                torch.cuda.set_device(device)
                stream = torch.cuda.Stream(device=device)
                idx_gpu, x_gpu = routings[which].to(device), xs[which].to(device)
                torch.cuda.synchronize()
                start.wait()
                with torch.cuda.stream(stream):
                    for _ in range(60):
                        result = buffer.dispatch(x_gpu, topk_idx=idx_gpu, do_expand=True, alignment=4, zero_padding=True)
                        layout = result.handle.layout
                        if (layout.recv_count, layout.expanded_capacity) != (expected[which].recv_count, expected[which].expanded_capacity):
                            failures.append((which, layout.recv_count, layout.expanded_capacity))
                            return
                    stream.synchronize()
                    assert_dispatch_result(result, xs[which], routings[which], None, experts, True, 4, True)
                    assert_handle(result.handle, expected[which], True, 4, buffer)
            except Exception as error:  # noqa: BLE001 - reported by the main thread
                failures.append((which, repr(error)))

        threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
        for thread in threads:
            thread.start()
        for thread in threads:
            thread.join(timeout=100)
        assert not any(thread.is_alive() for thread in threads)
        assert failures == []
        assert not buffer._runtime.counts_failed()


def test_a_fresh_dispatch_that_lost_its_counts_leaves_the_runtime_failed(device):
    """The reference latches a failure when the host wait for N and C does not end well
    (csrc/peer.cu:229-232) and serves nothing afterwards: a count stored late must not answer a
    later call.  Here the loss is staged on the host (a turn at the mailbox that ends without a
    verdict); no kernel misbehaves."""
    tokens, experts, topk, hidden = 8, 4, 2, 256
    idx = cases.routing("random", tokens, experts, topk).to(device)
    x = cases.payload(tokens, hidden).to(device)
    buffer = Buffer(None, EPConfig(experts, topk, hidden, tokens))
    received = buffer.dispatch(x, topk_idx=idx, do_expand=True)
    assert not buffer._runtime.counts_failed()
    buffer._runtime.lose_counts_for_test()
    assert buffer._runtime.counts_failed()
    for call in (
        lambda: buffer.dispatch(x, topk_idx=idx, do_expand=True),
        lambda: buffer.dispatch(x, handle=received.handle),
        lambda: buffer.combine(received.x, received.handle),
        lambda: buffer._runtime.lose_counts_for_test(),
    ):
        with pytest.raises(RuntimeError, match="failed while waiting for its counts"):
            call()
    buffer.close()  # closing still works
    with pytest.raises(RuntimeError, match="closed"):
        buffer.dispatch(x, topk_idx=idx)


@pytest.mark.parametrize("alignment", [1, 16], ids=["outputs-at-the-bound", "outputs-exact"])
def test_rejected_routing_with_padding_and_weights_then_a_good_dispatch(device, alignment):
    """A routing error is only known once the host has the status word; where the outputs are
    allocated at their bound the permute has by then run on the rejected layout.  It must not harm
    anything: earlier results and their neighbours in memory keep their bytes, the error is the
    routing error, and the next dispatch is the oracle's."""
    tokens, experts, topk, hidden = 300, 16, 4, 512
    idx = cases.routing("dropout", tokens, experts, topk, seed=8)
    x, w = cases.payload(tokens, hidden, seed=2), cases.gate_weights(tokens, topk)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        before = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                                 alignment=alignment, zero_padding=True)
        kept_x, kept_w = before.x.clone(), before.topk_weights.clone()
        # freed blocks around the next allocations carry a known pattern
        guards = [torch.full((rows, hidden), -3.0, dtype=torch.bfloat16, device=device) for rows in (64, 2048, 64)]
        pattern = [guard.clone() for guard in guards]
        for bad_value, message in ((experts, "out of range"), (-2, "out of range"), (None, "duplicate")):
            bad = idx.clone()
            if bad_value is None:
                bad[7] = 3
            else:
                bad[5, 1] = bad_value
            with pytest.raises(RuntimeError, match=message):
                buffer.dispatch(x.to(device), topk_idx=bad.to(device), weights=w.to(device), do_expand=True,
                                alignment=alignment, zero_padding=True)
            assert not buffer._runtime.counts_failed()
        torch.cuda.synchronize()
        for guard, want in zip(guards, pattern):
            assert torch.equal(guard.view(torch.int16), want.view(torch.int16))
        assert torch.equal(before.x.view(torch.int16), kept_x.view(torch.int16))
        assert torch.equal(before.topk_weights.view(torch.int32), kept_w.view(torch.int32))
        good = buffer.dispatch(x.to(device), topk_idx=idx.to(device), weights=w.to(device), do_expand=True,
                               alignment=alignment, zero_padding=True)
        lay = assert_dispatch_result(good, x, idx, w, experts, True, alignment, True)
        assert_handle(good.handle, lay, True, alignment, buffer)


def test_deterministic_fill_is_rejected_by_the_api_but_not_the_backend(device):
    """The API refuses deterministic algorithms + fill_uninitialized_memory (as the reference does);
    the native module accepts them, and the poison torch then writes into every torch.empty output
    proves that dispatch and combine write every byte they own."""
    native = load_extension()
    enabled = torch.are_deterministic_algorithms_enabled()
    warn_only = torch.is_deterministic_algorithms_warn_only_enabled()
    fill = deterministic.fill_uninitialized_memory
    tokens, experts, topk, hidden = 37, 5, 3, 512
    idx = cases.routing("mixed", tokens, experts, topk, seed=8)
    x, w = cases.payload(tokens, hidden), cases.gate_weights(tokens, topk)
    config = EPConfig(experts, topk, hidden, 64)
    buffer = Buffer(None, config)
    torch.use_deterministic_algorithms(True)
    deterministic.fill_uninitialized_memory = True
    try:
        with pytest.raises(RuntimeError, match="fill_uninitialized_memory"):
            buffer.dispatch(x.to(device), topk_idx=idx.to(device))
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            for expand, zero_padding in ((False, False), (True, True)):
                outputs, metadata, counts, event = native.dispatch(
                    buffer._runtime, x.to(device), idx.to(device), w.to(device), experts, 64, 4, [], 0, False,
                    expand=expand, zero_padding=zero_padding, num_sms=0, comm_stream=stream.cuda_stream,
                )
                assert event is not None  # async_op defaults to True at the native boundary
                event.current_stream_wait()
                want_x, want_idx, want_w, lay = oracle.dispatch(x, idx, experts, w, do_expand=expand, alignment=4)
                assert list(counts) == [lay.recv_count, lay.expanded_capacity]
                assert_same_bits(outputs[0], want_x, "every output row is written")
                assert_same_bits(outputs[2], want_w, "every output weight is written")
                assert (outputs[1].shape == (0,)) if expand else torch.equal(outputs[1].cpu(), want_idx)
                y = outputs[0]
                results, event = native.combine(buffer._runtime, y, metadata, outputs[2], None, 64, expand, False, 0, stream.cuda_stream)
                event.current_stream_wait()
                want, want_ow = oracle.combine(want_x, lay.recv_metadata(expand), lay.dst_slots, do_expand=expand, weights=want_w)
                assert_same_bits(results[0], want, "every combined row is written")
                assert_same_bits(results[1], want_ow, "every combined weight is written")
        stream.synchronize()
    finally:
        deterministic.fill_uninitialized_memory = fill
        torch.use_deterministic_algorithms(enabled, warn_only=warn_only)
        buffer.close()


@pytest.mark.parametrize(
    "tokens,hidden,experts,topk,kind,expand,alignment,zero_padding,cached_iterations",
    [
        pytest.param(4096, 4096, 8, 2, "random", True, 1, False, 1, id="mixtral"),
        pytest.param(4096, 7168, 256, 8, "dropout", True, 1, True, 1, id="deepseek-v3"),
        pytest.param(32768, 7168, 32, 8, "zipf", False, 1, False, 3, id="ep8-share-cached"),
        pytest.param(8192, 2048, 128, 8, "biased", True, 128, True, 1, id="qwen3-async"),
    ],
)
def test_baseline_configs_through_the_api(device, tokens, hidden, experts, topk, kind, expand, alignment, zero_padding,
                                          cached_iterations):
    idx = cases.routing(kind, tokens, experts, topk, seed=11)
    x = cases.payload(tokens, hidden)
    logits = cases.gate_weights(tokens, topk, seed=3)
    w = torch.softmax(logits, dim=1)
    asynchronous = kind == "biased"
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        side = torch.cuda.Stream() if asynchronous else torch.cuda.current_stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            x_dev, w_dev = x.to(device), w.to(device)
            received = buffer.dispatch(x_dev, topk_idx=idx.to(device), weights=w_dev, do_expand=expand, alignment=alignment,
                                       zero_padding=zero_padding, async_op=asynchronous)
            if asynchronous:
                received.event.current_stream_wait()
            lay = assert_dispatch_result(received, x, idx, w, experts, expand, alignment, zero_padding)
            assert_handle(received.handle, lay, expand, alignment, buffer)
            for _ in range(cached_iterations):
                replay = buffer.dispatch(x_dev, weights=w_dev, handle=received.handle, zero_padding=zero_padding,
                                         async_op=asynchronous)
                if asynchronous:
                    replay.event.current_stream_wait()
                assert replay.handle is received.handle
                # identity experts apply each gate weight once (expanded) or sum the weighted copies (compact)
                if expand:
                    y = (replay.x.float() * replay.topk_weights[:, None]).to(torch.bfloat16)
                else:
                    gate = torch.where(replay.topk_idx >= 0, replay.topk_weights, torch.zeros_like(replay.topk_weights)).sum(1)
                    y = (replay.x.float() * gate[:, None]).to(torch.bfloat16)
                combined = buffer.combine(y, replay.handle, weights=replay.topk_weights, async_op=asynchronous)
                if asynchronous:
                    combined.event.current_stream_wait()
            want, want_w = oracle.combine(y.cpu(), lay.recv_metadata(expand), lay.dst_slots, do_expand=expand,
                                          weights=replay.topk_weights.cpu())
            assert_same_bits(combined.x, want, "combined x")
            assert_same_bits(combined.topk_weights, want_w, "combined weights")
            assert_same_bits(combined.topk_weights, w.masked_fill(idx < 0, 0), "weights return to their k")
            # size-independent property: the weighted identity round trip stays close to x
            scale = torch.where(idx >= 0, w, torch.zeros_like(w)).sum(1, keepdim=True)
            torch.testing.assert_close(combined.x.cpu().float(), x.float() * scale, rtol=0.03, atol=0.03)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()


def test_cached_dispatch_and_combine_replay_in_a_hip_graph(device):
    """Cached dispatch and combine launch one kernel each and wait on nothing, so they can be
    captured; every replay (with eager work and synchronisations in between) matches eager results.
    Fresh dispatch polls the host for N/C and must refuse capture."""
    tokens, experts, topk, hidden = 512, 32, 4, 2048
    idx = cases.routing("dropout", tokens, experts, topk, seed=21)
    w = cases.gate_weights(tokens, topk).to(device)
    with Buffer(None, EPConfig(experts, topk, hidden, tokens)) as buffer:
        static_x = cases.payload(tokens, hidden, seed=1).to(device)
        fresh = buffer.dispatch(static_x, topk_idx=idx.to(device), weights=w, do_expand=True, alignment=16, zero_padding=True)
        handle = fresh.handle
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            replay = buffer.dispatch(static_x, weights=w, handle=handle, zero_padding=True)
            expert_x = (replay.x.float() * replay.topk_weights[:, None]).to(torch.bfloat16)
            combined = buffer.combine(expert_x, handle, weights=replay.topk_weights)
        for step in range(4):
            new_x = cases.payload(tokens, hidden, seed=100 + step).to(device)
            static_x.copy_(new_x)
            graph.replay()
            torch.cuda.synchronize()
            eager = buffer.dispatch(new_x, weights=w, handle=handle, zero_padding=True)
            eager_y = (eager.x.float() * eager.topk_weights[:, None]).to(torch.bfloat16)
            eager_combined = buffer.combine(eager_y, handle, weights=eager.topk_weights)
            torch.cuda.synchronize()
            assert_same_bits(replay.x, eager.x.cpu(), f"graph replay {step}: dispatched rows")
            assert_same_bits(combined.x, eager_combined.x.cpu(), f"graph replay {step}: combined rows")
            assert_same_bits(combined.topk_weights, eager_combined.topk_weights.cpu(), f"graph replay {step}: weights")
        idx_dev = idx.to(device)
        torch.cuda.synchronize()
        probe = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="captured"):
            with torch.cuda.graph(probe):
                buffer.dispatch(static_x, topk_idx=idx_dev, weights=w, do_expand=True)
        torch.cuda.synchronize()
        # the buffer still works after the refused capture
        again = buffer.dispatch(static_x, topk_idx=idx_dev, weights=w, do_expand=True, alignment=16, zero_padding=True)
        assert again.handle.layout.expanded_capacity == handle.layout.expanded_capacity
