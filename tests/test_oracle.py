"""Pins of the CPU oracle (no GPU).  Each check is chosen so that a plausible mistake -- a dropped
term, a wrong index, a transposed operand, a wrong rounding -- fails at least one of them; none of
them re-types the oracle's own formula."""

import numpy as np
import pytest
import torch

import cases
from oracle import nanoep_oracle as oracle


def closed_form_gap_case(experts, tokens, alignment):
    """Inputs of the reference's test_padding_gaps_across_expert_waves
    (tests/native/test_native_dispatch.py:289-310) and their layout written out by hand."""
    selected = [2, 33, experts - 1] if experts > 32 else [0, 1, 2]
    idx = torch.tensor([selected] * tokens, dtype=torch.int64)
    if tokens > 1:
        idx[::2, 1] = -1
        idx[::3, 2] = -1
    # every token keeps choice 0; choice 1 survives on odd tokens; choice 2 on tokens not divisible by 3
    counts = torch.zeros(experts, dtype=torch.int64)
    counts[selected[0]] = tokens
    counts[selected[1]] = tokens // 2 if tokens > 1 else 1
    counts[selected[2]] = tokens - (tokens + 2) // 3 if tokens > 1 else 1
    padded = -(-counts // alignment) * alignment
    offsets = torch.zeros(experts + 1, dtype=torch.int64)
    for e in range(experts):
        offsets[e + 1] = offsets[e] + padded[e]
    slots = torch.full((tokens, 3), -1, dtype=torch.int64)
    for t in range(tokens):
        slots[t, 0] = offsets[selected[0]] + t
        if tokens == 1 or t % 2 == 1:
            slots[t, 1] = offsets[selected[1]] + (t // 2 if tokens > 1 else 0)
        if tokens == 1 or t % 3 != 0:
            slots[t, 2] = offsets[selected[2]] + (t - (t + 2) // 3 if tokens > 1 else 0)
    return idx, counts, offsets, slots


@pytest.mark.parametrize("experts,tokens,alignment", [(3, 1, 128), (40, 9, 1), (65, 9, 4), (65, 64, 16)])
@pytest.mark.parametrize("impl", [oracle.layout_scalar, oracle.layout], ids=["scalar", "vectorised"])
def test_layout_closed_form(impl, experts, tokens, alignment):
    idx, counts, offsets, slots = closed_form_gap_case(experts, tokens, alignment)
    lay = impl(idx, experts, alignment)
    assert lay.recv_count == tokens and torch.equal(lay.src_tokens, torch.arange(tokens))
    assert torch.equal(lay.expert_counts, counts)
    assert torch.equal(lay.expert_offsets, offsets)
    assert lay.expanded_capacity == int(offsets[-1])
    assert torch.equal(lay.expanded_slots, slots)
    assert torch.equal(lay.dst_slots.flatten(), torch.arange(tokens))
    assert lay.send_counts.tolist() == [tokens] and lay.recv_rank_prefix.tolist() == [tokens]


@pytest.mark.parametrize("experts,alignment,kind", [(31, 1, "random"), (31, 4, "random"), (32, 16, "random"), (33, 4, "zero")])
def test_count_finaliser_closed_form(experts, alignment, kind):
    """The closed form of the reference's tests/native/test_receive_counts.py:29-45 for one rank."""
    g = torch.Generator().manual_seed(71)
    counts = torch.randint(0, 19, (experts,), generator=g, dtype=torch.int64)
    counts[::3] = 0
    if kind == "zero":
        counts.zero_()
    # build a routing with exactly those counts: expert e is chosen by tokens 0..counts[e]-1, one expert per column
    tokens = int(counts.max()) if counts.numel() and counts.max() > 0 else 3
    idx = torch.full((tokens, experts), -1, dtype=torch.int64)
    for e in range(experts):
        idx[: counts[e], e] = e
    idx = idx[:, :32] if experts > 32 else idx
    counts = counts[:32] if experts > 32 else counts
    local_experts = experts
    for impl in (oracle.layout_scalar, oracle.layout):
        lay = impl(idx, local_experts, alignment)
        want = torch.zeros(local_experts, dtype=torch.int64)
        want[: counts.numel()] = counts
        padded = (want + alignment - 1) // alignment * alignment
        assert torch.equal(lay.expert_counts, want)
        assert torch.equal(lay.expert_offsets, torch.cat((torch.zeros(1, dtype=torch.int64), padded.cumsum(0))))
        assert lay.recv_count == int((idx >= 0).any(dim=1).sum())


@pytest.mark.parametrize("kind", ["random", "masked", "skew", "mixed", "dropout", "sparse", "zipf", "biased"])
@pytest.mark.parametrize("tokens,experts,topk,alignment", [(5, 3, 3, 1), (19, 3, 3, 16), (64, 40, 3, 4), (300, 65, 8, 128), (257, 8, 2, 1)])
def test_layout_invariants_and_scalar_agreement(kind, tokens, experts, topk, alignment):
    idx = cases.routing(kind, tokens, experts, topk, seed=tokens)
    scalar, vector = oracle.layout_scalar(idx, experts, alignment), oracle.layout(idx, experts, alignment)
    for name in ("src_tokens", "local_topk_idx", "expanded_slots", "expert_counts", "expert_offsets", "dst_slots", "send_counts",
                 "recv_rank_prefix", "topk_idx"):
        assert torch.equal(getattr(scalar, name), getattr(vector, name)), name
    lay = vector
    # the reference's own assertions (nano_ep/testing/native_dispatch.py:54-57): invalid <-> -1 and
    # every expert's slot set is exactly arange(start, start + count); plus token order inside it
    valid = lay.local_topk_idx >= 0
    assert torch.equal(lay.expanded_slots >= 0, valid)
    for expert, count in enumerate(lay.expert_counts.tolist()):
        start = int(lay.expert_offsets[expert])
        chosen = lay.expanded_slots[lay.local_topk_idx == expert]
        assert torch.equal(chosen, torch.arange(start, start + count))  # ascending with the receive row
        assert int(lay.expert_offsets[expert + 1]) - start == -(-count // alignment) * alignment
    assert torch.equal(lay.expert_counts, torch.bincount(idx[idx >= 0], minlength=experts))
    received = (idx >= 0).any(dim=1)
    assert torch.equal(lay.src_tokens, torch.nonzero(received).flatten())
    assert torch.equal(lay.dst_slots.flatten()[received], torch.arange(lay.recv_count))
    assert (lay.dst_slots.flatten()[~received] == -1).all()
    assert torch.equal(lay.local_topk_idx, idx[received])
    meta = lay.recv_metadata(True)
    assert meta.dtype == torch.int32 and meta.shape == (lay.recv_count, topk + 2)
    assert (meta[:, 0] == 0).all() and torch.equal(meta[:, 1].long(), lay.src_tokens)
    assert torch.equal(lay.recv_metadata(False)[:, 2:].long(), lay.local_topk_idx)


@pytest.mark.parametrize("expand", [False, True])
def test_dispatch_is_a_byte_gather(expand):
    """recv_x[slot(t,k)] == x[t] bit for bit, NaN payloads and -0 included; padding is zero."""
    tokens, experts, topk, hidden = 23, 7, 3, 16
    idx = cases.routing("dropout", tokens, experts, topk, seed=4)
    patterns = torch.tensor([0x7FC1, 0xFFC0, 0x7F81, 0x8000, 0x0001, 0x3F80, 0xC2F7], dtype=torch.int32)
    raw = patterns.repeat(tokens * hidden // len(patterns) + 1)[: tokens * hidden]
    x = raw.to(torch.int16).view(torch.bfloat16).reshape(tokens, hidden)
    w = cases.gate_weights(tokens, topk)
    for impl in (oracle.dispatch_scalar, oracle.dispatch):
        out, out_idx, out_w, lay = impl(x, idx, experts, w, do_expand=expand, alignment=4)
        touched = torch.zeros(out.shape[0], dtype=torch.bool)
        for row, token in enumerate(lay.src_tokens.tolist()):
            if expand:
                for k in range(topk):
                    slot = int(lay.expanded_slots[row, k])
                    if slot >= 0:
                        assert torch.equal(out[slot].view(torch.int16), x[token].view(torch.int16))
                        assert out_w[slot] == w[token, k]
                        touched[slot] = True
            else:
                assert torch.equal(out[row].view(torch.int16), x[token].view(torch.int16))
                assert torch.equal(out_w[row], w[token])  # the complete source row, masked slots included
                assert torch.equal(out_idx[row], idx[token])
                touched[row] = True
        assert (out[~touched].view(torch.int16) == 0).all()
        if expand:
            assert out_idx is None and (out_w[~touched] == 0).all()
            assert out.shape[0] == lay.expanded_capacity
        else:
            assert touched.all()


def test_readme_identity_round_trip():
    """README.md:56-67 of the reference: identity experts weighted once, combine reproduces x."""
    x = cases.payload(16, 256, seed=0)
    idx = torch.tensor([[0, 1]], dtype=torch.int64).repeat(16, 1)
    w = torch.full((16, 2), 0.5)
    for d, c in ((oracle.dispatch_scalar, oracle.combine_scalar), (oracle.dispatch, oracle.combine)):
        out, _, out_w, lay = d(x, idx, 2, w, do_expand=True, alignment=1)
        expert_x = (out.float() * out_w[:, None]).to(torch.bfloat16)
        combined, returned = c(expert_x, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
        assert returned is None and torch.equal(combined.view(torch.int16), x.view(torch.int16))


@pytest.mark.parametrize("expand", [False, True])
def test_multiplicity_round_trip_is_exact(expand):
    """combine(dispatch(x)) == x * multiplicity + bias exactly for small integers
    (tests/distributed/worker.py:292-322 of the reference)."""
    tokens, experts, topk, hidden = 40, 6, 3, 32
    idx = cases.routing("mixed", tokens, experts, topk, seed=31)
    x = torch.full((tokens, hidden), 3, dtype=torch.bfloat16)
    bias = torch.ones_like(x)
    for d, c in ((oracle.dispatch_scalar, oracle.combine_scalar), (oracle.dispatch, oracle.combine)):
        out, _, _, lay = d(x, idx, experts, None, do_expand=expand, alignment=4)
        combined, _ = c(out, lay.recv_metadata(expand), lay.dst_slots, do_expand=expand, bias=bias)
        valid = (idx >= 0).sum(dim=1)
        multiplicity = valid if expand else (valid > 0).long()
        assert torch.equal(combined.float(), x.float() * multiplicity[:, None] + 1)


def test_combine_accumulates_in_fp32_in_ascending_k():
    """256 + 1 - 256 keeps the 1 only with an fp32 accumulator; 2^30 - 2^30 + 64 depends on the order."""
    idx = torch.tensor([[0, 1, 2]], dtype=torch.int64)
    lay = oracle.layout(idx, 3, 1)
    y = torch.tensor([[256.0], [1.0], [-256.0]], dtype=torch.bfloat16).repeat(1, 8)
    for c in (oracle.combine_scalar, oracle.combine):
        out, _ = c(y, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
        assert (out.float() == 1.0).all()
        # order matters in fp32: ((0 + 2^30) - 2^30) + 64 = 64, but any order that adds 64 to +-2^30
        # first loses it (64 is half an ulp of 2^30 and the tie rounds to even)
        ascending = torch.tensor([[2.0**30], [-(2.0**30)], [64.0]], dtype=torch.bfloat16).repeat(1, 8)
        out, _ = c(ascending, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
        assert (out.float() == 64.0).all()
        rotated = torch.tensor([[64.0], [2.0**30], [-(2.0**30)]], dtype=torch.bfloat16).repeat(1, 8)
        out, _ = c(rotated, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
        assert (out.float() == 0.0).all()
        # allow_multiple_reduction: bf16(256 + 1) = 256 before the bias; single reduction keeps 257 -> 258 with +1
        two = torch.tensor([[0, 1, -1]], dtype=torch.int64)
        lay2 = oracle.layout(two, 3, 1)
        y2 = torch.tensor([[256.0], [1.0]], dtype=torch.bfloat16).repeat(1, 8)
        bias = torch.ones((1, 8), dtype=torch.bfloat16)
        multi, _ = c(y2, lay2.recv_metadata(True), lay2.dst_slots, do_expand=True, bias=bias, multiple_reduction=True)
        single, _ = c(y2, lay2.recv_metadata(True), lay2.dst_slots, do_expand=True, bias=bias)
        assert (multi.float() == 256.0).all() and (single.float() == 258.0).all()


def test_combine_special_values():
    """0 + (-0) = +0, masked tokens give 0 (+bias), weights come back at their k with masked slots 0."""
    idx = torch.tensor([[0, -1], [-1, -1], [1, 0]], dtype=torch.int64)
    lay = oracle.layout(idx, 2, 1)
    y = torch.zeros((lay.expanded_capacity, 4), dtype=torch.bfloat16)
    y[:] = -0.0
    w = torch.arange(1, lay.expanded_capacity + 1, dtype=torch.float32)
    bias = torch.full((3, 4), 0.25, dtype=torch.bfloat16)
    for c in (oracle.combine_scalar, oracle.combine):
        out, _ = c(y, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
        assert (out.view(torch.int16) == 0).all()  # +0, never -0
        out, returned = c(y, lay.recv_metadata(True), lay.dst_slots, do_expand=True, weights=w, bias=bias)
        assert (out.float() == 0.25).all()
        slots = torch.full((3, 2), -1, dtype=torch.int64)
        slots[lay.src_tokens] = lay.expanded_slots
        want = torch.where(slots >= 0, w[slots.clamp(min=0)], torch.zeros(()))
        assert torch.equal(returned, want) and returned[1].tolist() == [0.0, 0.0]


def test_bf16_cast_is_round_to_nearest_even():
    """The torch cast the combine oracle relies on agrees with an integer RNE on every finite
    pattern class: ties to even both ways, overflow to inf, subnormals, negative zero."""
    probes = np.array(
        [0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F7F8000, 0x00000001, 0x00008000, 0x00018000,
         0x80000000, 0x80008000, 0xC2F7A3D7, 0x7F800000, 0xFF800000, 0x33800000, 0x477FE000],
        dtype=np.uint32,
    )
    rng = np.random.default_rng(5)
    bits = np.concatenate([probes, rng.integers(0, 2**32, size=200_000, dtype=np.uint64).astype(np.uint32)])
    values = bits.view(np.float32)
    finite = ~np.isnan(values)
    mine = oracle.bf16_round_bits(values)
    theirs = torch.from_numpy(values.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(mine[finite], theirs[finite])
    assert mine[0] == 0x3F80 and mine[1] == 0x3F82  # the two ties: down to even, up to even
    nan_out = torch.from_numpy(values[~finite].copy()).to(torch.bfloat16)
    assert torch.isnan(nan_out).all()  # NaN stays NaN; its bit pattern is not pinned


def test_combine_matches_integer_rounding_independently():
    """Vectorised combine against a numpy restatement: float32 adds in ascending k, integer RNE."""
    tokens, experts, topk, hidden = 50, 9, 4, 24
    idx = cases.routing("dropout", tokens, experts, topk, seed=12)
    lay = oracle.layout(idx, experts, 2)
    y = (cases.payload(lay.expanded_capacity, hidden, seed=3).float() * 37.5).to(torch.bfloat16)
    bias = cases.payload(tokens, hidden, seed=4)
    out, _ = oracle.combine(y, lay.recv_metadata(True), lay.dst_slots, do_expand=True, bias=bias)
    y32 = y.float().numpy()
    acc = np.zeros((tokens, hidden), dtype=np.float32)
    slots = np.full((tokens, topk), -1, dtype=np.int64)
    slots[lay.src_tokens.numpy()] = lay.expanded_slots.numpy()
    for k in range(topk):
        live = slots[:, k] >= 0
        acc[live] = acc[live] + y32[slots[live, k]]
    acc = acc + bias.float().numpy()
    assert np.array_equal(oracle.bf16_round_bits(acc), out.view(torch.int16).numpy().view(np.uint16))


def test_window_layout_known_answer():
    """tests/unit/test_cuda_bootstrap.py:102-106 of the reference."""
    assert oracle.window_layout(2, 8, 256, 2, 4) == [0, 96, 160, 160, 9888]
    one = oracle.window_layout(1, 16, 256, 2, 2)
    assert one[0] == 0 and one[2] == one[3] and all(v % 32 == 0 for v in one)
