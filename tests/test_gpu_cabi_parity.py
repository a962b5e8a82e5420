"""GPU parity of the HIP kernels against the CPU oracle, called through the C ABI.

Bar: bit-exact for the layout, the indices and the dispatched payload (a byte copy, NaN payloads
included); bit-exact for combine on every non-NaN output (fixed ascending-k fp32 accumulation,
one round-to-nearest-even cast), NaN <-> NaN otherwise.  Cases mirror the reference's
tests/native/test_native_dispatch.py:211-310 and tests/native/test_native_combine.py:30-77.
"""

import pytest
import torch

import cabi
import cases
from oracle import nanoep_oracle as oracle

pytestmark = pytest.mark.gpu

POISON = 0xA5


def bits(tensor):
    return tensor.contiguous().view(torch.int16) if tensor.dtype == torch.bfloat16 else tensor.contiguous().view(torch.int32)


def assert_bits_equal(actual, expected, what):
    assert actual.shape == expected.shape, f"{what}: shape {tuple(actual.shape)} != {tuple(expected.shape)}"
    assert actual.dtype == expected.dtype, what
    assert torch.equal(bits(actual.cpu()), bits(expected)), f"{what}: bit mismatch"


def assert_layout(metadata, counts, expected: oracle.Layout, expand, hidden=0):
    assert counts[0] == expected.recv_count and counts[1] == expected.expanded_capacity
    assert counts[2] == int(expected.expert_counts.sum()) and counts[3] == 0
    for actual, want, name in zip(
        metadata,
        expected.metadata(expand),
        ["recv_metadata", "expert_counts", "expert_offsets", "dst_slots", "send_counts", "topk_snapshot", "recv_rank_prefix"],
    ):
        assert actual.dtype == want.dtype and actual.is_contiguous(), name
        assert tuple(actual.shape) == tuple(want.shape), name
        assert torch.equal(actual.cpu(), want), name
    if expand:
        # private slot table: slot[t,k] for every source token, -1 when masked
        table = torch.full(expected.topk_idx.shape, -1, dtype=torch.int32)
        table[expected.src_tokens] = expected.expanded_slots.to(torch.int32)
        assert torch.equal(metadata[7].cpu(), table), "token_slots"
        # private slot-order list: block of consecutive tokens by block, the valid assignments as
        # (slot << 32) | (t * K + k) in ascending slot order, without gaps; -1 from entry A on
        tokens, topk = expected.topk_idx.shape
        block_tokens = cabi.lib().nanoep_layout_block_tokens(tokens, expected.expert_counts.numel(), hidden)
        flat = table.flatten().to(torch.int64)
        packed = (flat << 32) | torch.arange(flat.numel(), dtype=torch.int64)
        want = []
        for first in range(0, tokens, block_tokens):
            part = packed[first * topk : (first + block_tokens) * topk]
            want.append(part[flat[first * topk : (first + block_tokens) * topk] >= 0].sort().values)
        entries = cabi.lib().nanoep_slot_order_entries(tokens, topk, expected.expert_counts.numel())
        got = metadata[8].cpu()
        assert got.numel() == entries == ((tokens + 255) // 256 * 256 * topk + 1 if tokens else 0)
        if entries:
            want.append(torch.full((entries - 1 - counts[2],), -1, dtype=torch.int64))
            want.append(torch.tensor([counts[2]], dtype=torch.int64))  # count word at the end of the buffer
            assert torch.equal(got, torch.cat(want)), "slot_order"


def run_dispatch_combine(device, idx, hidden, experts, alignment, expand, zero_padding, weighted, *, seed=0, num_cus=0):
    tokens, topk = idx.shape
    x = cases.payload(tokens, hidden, seed=123 + seed)
    w = cases.gate_weights(tokens, topk, seed=7 + seed) if weighted else None
    expected_layout = oracle.layout(idx, experts, alignment)
    metadata, counts = cabi.layout(idx.to(device), experts, alignment, expand, hidden=hidden)
    assert_layout(metadata, counts, expected_layout, expand, hidden)
    want_x, want_idx, want_w, _ = oracle.dispatch(x, idx, experts, w, do_expand=expand, alignment=alignment, lay=expected_layout)
    got_x, got_idx, got_w = cabi.dispatch(
        x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
        num_cus=num_cus, poison=POISON,
    )
    torch.cuda.synchronize()
    if expand:
        # the same handle without the private slot table must give the same bytes
        plain_x, _, plain_w = cabi.dispatch(
            x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
            num_cus=num_cus, poison=POISON, use_table=False, use_order=False,
        )
        assert torch.equal(plain_x.view(torch.int16), got_x.view(torch.int16))
        assert plain_w is None or torch.equal(plain_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must the slot-order walk that reads its entry count on the device
        device_x, _, device_w = cabi.dispatch(
            x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
            num_cus=num_cus, poison=POISON, order_count="device",
        )
        assert torch.equal(device_x.view(torch.int16), got_x.view(torch.int16))
        assert device_w is None or torch.equal(device_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must the walk that moves two chunks a wavefront (the library's choice for sources
        # beyond the last-level cache), with either entry count
        for order_count in ("exact", "device"):
            wide_x, _, wide_w = cabi.dispatch(
                x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
                num_cus=num_cus, poison=POISON, order_count=order_count, span=2,
            )
            assert torch.equal(wide_x.view(torch.int16), got_x.view(torch.int16))
            assert wide_w is None or torch.equal(wide_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must that walk with other numbers of list entries a workgroup and of chunks a wavefront
        # (rows of up to four pieces share workgroups, longer ones take one each), with either entry count
        for rows in (1, 2, 4, 16):
            for order_count, span in (("exact", 1), ("device", 1), ("exact", 2), ("device", 4)):
                rows_x, _, rows_w = cabi.dispatch(
                    x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
                    num_cus=num_cus, poison=POISON, order_count=order_count, span=span, rows=rows,
                )
                assert torch.equal(rows_x.view(torch.int16), got_x.view(torch.int16))
                assert rows_w is None or torch.equal(rows_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must the walk with and without its window-wise source prefetch
        for prefetch in (0, 1):
            for rows in (None, 3):
                for order_count in ("exact", "device"):
                    fetched_x, _, fetched_w = cabi.dispatch(
                        x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
                        num_cus=num_cus, poison=POISON, prefetch=prefetch, rows=rows, order_count=order_count,
                    )
                    assert torch.equal(fetched_x.view(torch.int16), got_x.view(torch.int16))
                    assert fetched_w is None or torch.equal(fetched_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must rows of at most 512 bytes with one list entry a wavefront instead of four or eight
        if hidden <= 256:
            for order_count in ("exact", "device"):
                for rows in (None, 3):
                    single_x, _, single_w = cabi.dispatch(
                        x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
                        num_cus=num_cus, poison=POISON, pack=1, rows=rows, order_count=order_count,
                    )
                    assert torch.equal(single_x.view(torch.int16), got_x.view(torch.int16))
                    assert single_w is None or torch.equal(single_w.view(torch.int32), got_w.view(torch.int32))
        # ... so must the same call with the library's switches left alone
        auto_x, _, auto_w = cabi.dispatch(
            x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
            num_cus=num_cus, poison=POISON, walk="auto",
        )
        assert torch.equal(auto_x.view(torch.int16), got_x.view(torch.int16))
        assert auto_w is None or torch.equal(auto_w.view(torch.int32), got_w.view(torch.int32))
        # ... and so must the token-order walk with the slot table
        table_x, _, table_w = cabi.dispatch(
            x.to(device), None if w is None else w.to(device), metadata, counts, experts, alignment, expand, zero_padding,
            num_cus=num_cus, poison=POISON, use_order=False,
        )
        assert torch.equal(table_x.view(torch.int16), got_x.view(torch.int16))
        assert table_w is None or torch.equal(table_w.view(torch.int32), got_w.view(torch.int32))
        assert got_idx is None
        live = torch.zeros(counts[1], dtype=torch.bool)
        live[expected_layout.expanded_slots[expected_layout.expanded_slots >= 0]] = True
        assert_bits_equal(got_x.cpu()[live], want_x[live], "expanded x")
        if weighted:
            assert_bits_equal(got_w.cpu()[live], want_w[live], "expanded weights")
        gaps = ~live
        if zero_padding:
            assert_bits_equal(got_x.cpu()[gaps], torch.zeros_like(want_x[gaps]), "gap rows")
            if weighted:
                assert_bits_equal(got_w.cpu()[gaps], torch.zeros_like(want_w[gaps]), "gap weights")
        else:
            # untouched rows keep the poison: the kernel writes nothing it does not own
            assert (got_x.cpu()[gaps].view(torch.uint8) == POISON).all()
    else:
        assert_bits_equal(got_x, want_x, "compact x")
        assert torch.equal(got_idx.cpu(), want_idx)
        if weighted:
            assert_bits_equal(got_w, want_w, "compact weights")

    # identity-free combine: feed arbitrary expert outputs, compare with the oracle's accumulation
    rows = counts[1] if expand else counts[0]
    y = cases.payload(rows, hidden, seed=999 + seed)
    yw = None
    if weighted:
        yw = cases.gate_weights(rows, 1, seed=5).flatten() if expand else cases.gate_weights(rows, topk, seed=5)
    bias = cases.payload(tokens, hidden, seed=31 + seed) if seed % 2 else None
    for multi in (False, True):
        want_out, want_ow = oracle.combine(
            y, expected_layout.recv_metadata(expand), expected_layout.dst_slots, do_expand=expand, weights=yw, bias=bias,
            multiple_reduction=multi,
        )
        got_out, got_ow = cabi.combine(
            y.to(device), None if yw is None else yw.to(device), None if bias is None else bias.to(device), metadata,
            counts, expand, multiple_reduction=multi, num_cus=num_cus, poison=POISON,
        )
        torch.cuda.synchronize()
        assert_bits_equal(got_out, want_out, f"combine x multi={multi}")
        if weighted:
            assert_bits_equal(got_ow, want_ow, "combine weights")
        # either kind of store for the output rows
        for stores in (0, 1):
            stored_out, stored_ow = cabi.combine(
                y.to(device), None if yw is None else yw.to(device), None if bias is None else bias.to(device), metadata,
                counts, expand, multiple_reduction=multi, num_cus=num_cus, poison=POISON, stores=stores,
            )
            torch.cuda.synchronize()
            assert_bits_equal(stored_out, want_out, f"combine x multi={multi} stores={stores}")
            if weighted:
                assert_bits_equal(stored_ow, want_ow, f"combine weights stores={stores}")
        # one to sixteen tokens a wavefront (a choice only with five or more rows a token; the library
        # picks by batch size, and small test batches would all take two)
        if expand and topk > 4:
            for units in (1, 2, 3, 4, 7, 8, 9, 13, 16):
                held_out, held_ow = cabi.combine(
                    y.to(device), None if yw is None else yw.to(device), None if bias is None else bias.to(device), metadata,
                    counts, expand, multiple_reduction=multi, num_cus=num_cus, poison=POISON, units=units,
                )
                torch.cuda.synchronize()
                assert_bits_equal(held_out, want_out, f"combine x multi={multi} units={units}")
                if weighted:
                    assert_bits_equal(held_ow, want_ow, f"combine weights units={units}")
        if expand:
            plain_out, plain_ow = cabi.combine(
                y.to(device), None if yw is None else yw.to(device), None if bias is None else bias.to(device), metadata,
                counts, expand, multiple_reduction=multi, num_cus=num_cus, poison=POISON, use_table=False,
            )
            assert_bits_equal(plain_out, want_out, f"combine x without slot table multi={multi}")
            if weighted:
                assert_bits_equal(plain_ow, want_ow, "combine weights without slot table")
    return metadata, counts


LAYOUTS = [(False, False), (True, False), (True, True)]
LAYOUT_IDS = ["compact", "expanded", "expanded-zero-padding"]


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
def test_small_cases(device, expand, zero_padding, weighted, kind, hidden, alignment):
    idx = cases.routing(kind, 5, 3, 3, seed=0)
    run_dispatch_combine(device, idx, hidden, 3, alignment, expand, zero_padding, weighted, seed=1)


@pytest.mark.parametrize("expand,zero_padding", LAYOUTS, ids=LAYOUT_IDS)
def test_multiple_blocks(device, expand, zero_padding):
    idx = cases.routing("mixed", 19, 3, 3, seed=3)
    run_dispatch_combine(device, idx, 512, 3, 16, expand, zero_padding, True, seed=2)


@pytest.mark.parametrize(
    "expand,zero_padding,weighted,hidden",
    [
        pytest.param(False, False, True, 512, id="compact"),
        pytest.param(True, False, False, 768, id="expanded"),
        pytest.param(True, True, True, 512, id="expanded-zero-padding"),
    ],
)
def test_more_tokens_than_resident_waves(device, expand, zero_padding, weighted, hidden):
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    tokens = cus * 32 + 3
    idx = cases.routing("skew", tokens, 3, 3)
    idx[:3] = -1
    idx[::2, 1:] = -1
    run_dispatch_combine(device, idx, hidden, 3, 128, expand, zero_padding, weighted, seed=3)


@pytest.mark.parametrize(
    "experts,tokens,alignment,weighted,zero_padding",
    [
        pytest.param(3, 1, 128, True, True, id="single-wave-zero-padding"),
        pytest.param(40, 9, 1, False, False, id="multiple-waves-unaligned"),
        pytest.param(65, 9, 4, True, True, id="multiple-waves-zero-padding"),
    ],
)
def test_padding_gaps_across_expert_waves(device, experts, tokens, alignment, weighted, zero_padding):
    selected = [2, 33, experts - 1] if experts > 32 else [0, 1, 2]
    idx = torch.tensor([selected] * tokens, dtype=torch.int64)
    if tokens > 1:
        idx[::2, 1] = -1
        idx[::3, 2] = -1
    run_dispatch_combine(device, idx, 256, experts, alignment, True, zero_padding, weighted, seed=5)


@pytest.mark.parametrize(
    "name,tokens,hidden,experts,topk,kind,expand,alignment,zero_padding",
    [
        pytest.param("mixtral", 4096, 4096, 8, 2, "random", True, 1, False, id="mixtral-4096x4096-e8-k2"),
        pytest.param("dsv3", 4096, 7168, 256, 8, "dropout", True, 1, True, id="dsv3-4096x7168-e256-k8"),
        pytest.param("dsv3-a128", 4096, 7168, 256, 8, "dropout", True, 128, True, id="dsv3-align128"),
        pytest.param("qwen3", 8192, 2048, 128, 8, "biased", True, 128, True, id="qwen3-8192x2048-e128-k8"),
        pytest.param("ep8", 32768, 7168, 32, 8, "zipf", False, 1, False, id="ep8-share-32768x7168-l32-k8"),
    ],
)
def test_baseline_shapes(device, name, tokens, hidden, experts, topk, kind, expand, alignment, zero_padding):
    idx = cases.routing(kind, tokens, experts, topk, seed=11)
    run_dispatch_combine(device, idx, hidden, experts, alignment, expand, zero_padding, True, seed=6)


@pytest.mark.parametrize(
    "tokens,hidden,experts,topk",
    [
        pytest.param(5000, 7168, 64, 6, id="two-rounds-of-wavefronts"),
        pytest.param(9001, 2048, 128, 8, id="one-round-every-gth-token-with-a-remainder"),
        pytest.param(3000, 7168, 64, 12, id="one-round-two-passes-of-rows"),
    ],
)
def test_combine_launches_of_one_round_and_of_several(device, tokens, hidden, experts, topk):
    """The held sums of the combine at the sizes that decide their launch: one round of resident
    wavefronts (a wavefront then takes every G-th token, here with groups that the last tokens do not
    fill), several rounds (consecutive tokens), and more than eight rows a token (two passes)."""
    idx = cases.routing("dropout", tokens, experts, topk, seed=21)
    run_dispatch_combine(device, idx, hidden, experts, 1, True, False, True, seed=3)


def closed_form_slots(idx, experts, alignment):
    """slot[t,k] from the definition, evaluated with torch on the device of idx: experts ascending,
    inside an expert the tokens ascending, every expert's range padded to the alignment."""
    flat = idx.flatten()
    valid = flat >= 0
    counts = torch.bincount(flat[valid], minlength=experts)
    padded = (counts + alignment - 1) // alignment * alignment
    offsets = torch.cumsum(padded, 0) - padded
    keys = torch.where(valid, flat, torch.full_like(flat, experts))
    order = torch.sort(keys, stable=True).indices  # (t, k) pairs expert by expert, tokens ascending
    sorted_keys = keys[order]
    first_of_expert = torch.cumsum(counts, 0) - counts
    live = sorted_keys < experts
    position = torch.arange(flat.numel(), device=idx.device)
    slot_sorted = torch.where(
        live, offsets[sorted_keys.clamp(max=experts - 1)] + position - first_of_expert[sorted_keys.clamp(max=experts - 1)],
        torch.full_like(position, -1),
    )
    slots = torch.empty_like(flat)
    slots[order] = slot_sorted
    return slots.view_as(idx), counts, int(padded.sum())


@pytest.mark.parametrize(
    "tokens,hidden,experts,topk,expand,alignment",
    [
        pytest.param(40960, 7168, 256, 8, True, 1, id="expanded-4.7GB"),
        pytest.param(40960, 7168, 64, 8, True, 128, id="expanded-align128-4.5GB"),
        pytest.param(303104, 7168, 8, 2, False, 1, id="compact-4.3GB"),
    ],
)
def test_rows_beyond_four_gib(device, tokens, hidden, experts, topk, expand, alignment):
    """Receive buffers larger than 2^32 bytes: row addresses must be formed in 64 bits.  At this size
    the check is by properties that fix the result without the CPU oracle: the slots against their
    closed form, every received row against its source row bit for bit, padding rows zero, and
    combine over identity experts equal to multiplicity * x, exact for small-integer payloads."""
    small = cases.routing("dropout", 700, 40, 6, seed=3)  # the closed form itself, against the oracle
    want = oracle.layout(small, 40, 8)
    small_slots, small_counts, small_capacity = closed_form_slots(small, 40, 8)
    assert torch.equal(small_slots[want.src_tokens], want.expanded_slots) and small_capacity == want.expanded_capacity
    assert torch.equal(small_counts, want.expert_counts)

    g = torch.Generator(device=device).manual_seed(99)
    idx = torch.rand(tokens, experts, device=device, generator=g).topk(topk, dim=1).indices.to(torch.int64)
    idx = torch.where(torch.rand(tokens, topk, device=device, generator=g) < 0.05, torch.full_like(idx, -1), idx)
    idx = idx.contiguous()
    x = torch.randint(-4, 5, (tokens, hidden), device=device, generator=g).to(torch.bfloat16)
    w = torch.rand(tokens, topk, device=device, generator=g)

    metadata, counts = cabi.layout(idx, experts, alignment, expand, hidden=hidden)
    slots, expert_counts, capacity = closed_form_slots(idx, experts, alignment)
    sent = (idx >= 0).any(dim=1)
    assert counts[0] == int(sent.sum()) and counts[1] == capacity and counts[2] == int((idx >= 0).sum()) and counts[3] == 0
    assert torch.equal(metadata[1], expert_counts)
    rows = capacity if expand else counts[0]
    assert rows * hidden * 2 > 2**32
    row_of_token = torch.where(sent, torch.cumsum(sent, 0) - 1, torch.full((tokens,), -1, device=device))
    assert torch.equal(metadata[3].flatten(), row_of_token)
    if expand:
        assert torch.equal(metadata[0][:, 2:].to(torch.int64), slots[sent])
        assert torch.equal(metadata[7].to(torch.int64), slots)

    recv_x, recv_idx, recv_w = cabi.dispatch(x, w, metadata, counts, experts, alignment, expand, expand, poison=POISON)
    torch.cuda.synchronize()
    assert recv_x.shape == (rows, hidden)
    if expand:
        written = torch.zeros(rows, dtype=torch.bool, device=device)
        for k in range(topk):
            live = slots[:, k] >= 0
            assert torch.equal(bits(recv_x[slots[live, k]]), bits(x[live])), f"payload of choice {k}"
            assert torch.equal(recv_w[slots[live, k]], w[live, k])
            written[slots[live, k]] = True
        assert int(written.sum()) == counts[2]
        assert not recv_x[~written].view(torch.int16).any() and not recv_w[~written].view(torch.int32).any()
    else:
        assert torch.equal(bits(recv_x), bits(x[sent]))
        assert torch.equal(recv_w, w[sent])
        assert torch.equal(recv_idx, idx[sent])

    out, out_w = cabi.combine(recv_x, recv_w, None, metadata, counts, expand, poison=POISON)
    torch.cuda.synchronize()
    multiplicity = (idx >= 0).sum(dim=1, keepdim=True) if expand else sent[:, None].to(torch.int64)
    assert torch.equal(out.float(), x.float() * multiplicity)  # |sum| <= 32: exact in bf16
    assert torch.equal(out_w, torch.where(idx >= 0, w, torch.zeros_like(w)))


@pytest.mark.parametrize("topk,experts,hidden", [(1, 4, 256), (5, 16, 1024), (12, 40, 512), (32, 64, 256), (32, 32, 2048)])
@pytest.mark.parametrize("expand", [False, True], ids=["compact", "expanded"])
def test_topk_range(device, topk, experts, hidden, expand):
    """Every top-k the API admits (1..32), including the ones that need two gather groups."""
    idx = cases.routing("dropout", 77, experts, topk, seed=topk)
    run_dispatch_combine(device, idx, hidden, experts, 8, expand, expand, True, seed=topk)


@pytest.mark.parametrize("launches", ["2", "3"], ids=["scan-in-assign", "separate-scan"])
@pytest.mark.parametrize(
    "tokens,experts,topk,kind,alignment",
    [(1000, 16, 4, "mixed", 8), (4096, 256, 8, "dropout", 1), (700, 1500, 9, "sparse", 3), (2049, 8, 2, "skew", 128), (5000, 40, 17, "random", 1)],
)
@pytest.mark.parametrize("expand", [False, True], ids=["compact", "expanded"])
@pytest.mark.parametrize("hidden", [0, 2048, 16384, 40000], ids=["windows-256", "windows-512", "windows-128", "windows-64"])
def test_both_layout_launch_plans(device, tuning, hidden, launches, tokens, experts, topk, kind, alignment, expand):
    """The layout runs as two launches (every block scans the block histograms itself) or three
    (single-workgroup scan), chosen by size; both plans must give the oracle's handle."""
    tuning("LAYOUT_LAUNCHES", launches)
    idx = cases.routing(kind, tokens, experts, topk, seed=5)
    metadata, counts = cabi.layout(idx.to(device), experts, alignment, expand, hidden=hidden)
    assert_layout(metadata, counts, oracle.layout(idx, experts, alignment), expand, hidden)


@pytest.mark.parametrize("tokens,experts,topk,hidden", [(16400, 64, 4, 1024), (15500, 1400, 3, 256), (20001, 8, 2, 512)])
def test_windows_of_1024_tokens(device, tokens, experts, topk, hidden):
    """Rows of up to 1024 elements in batches of more than 15 360 tokens: the slot-order list is
    ordered by windows of 1024 tokens, four layout blocks each (eight when 1400 experts shrink the
    blocks); ragged last window."""
    assert cabi.lib().nanoep_layout_block_tokens(tokens, experts, hidden) == 1024
    idx = cases.routing("dropout", tokens, experts, topk, seed=tokens)
    run_dispatch_combine(device, idx, hidden, experts, 8, True, True, True, seed=3)


@pytest.mark.parametrize(
    "window,tokens,experts",
    [(96, 1000, 24), (160, 4096, 24), (192, 4096, 24), (224, 2000, 24), (512, 1500, 24),
     # windows that are not whole wavefronts, with experts that fall to the threads of the last, partial one
     (96, 1000, 72), (96, 1000, 96), (96, 1000, 256), (160, 4096, 160), (160, 4096, 256), (224, 2000, 200), (224, 2000, 256)],
)
def test_forced_window_sizes(device, tuning, window, tokens, experts):
    """The WINDOW_TOKENS switch orders the slot-order list by windows of any multiple of 32 tokens up to
    256 (one layout workgroup each; the last one ragged, and more workgroups' worth of tokens than
    the list buffer, which is sized by blocks of 256, has room for beyond the batch)."""
    tuning("WINDOW_TOKENS", str(window))
    assert cabi.lib().nanoep_layout_block_tokens(tokens, experts, 512) == window
    idx = cases.routing("dropout", tokens, experts, 4, seed=window)
    run_dispatch_combine(device, idx, 512, experts, 8, True, True, True, seed=5)


@pytest.mark.parametrize("xcds", [1, 2, 3, 4, 8, 16])
@pytest.mark.parametrize("tokens,experts,topk,hidden,alignment", [(3000, 40, 8, 5120, 16), (5000, 16, 2, 1024, 1), (900, 8, 4, 256, 4)])
def test_any_xcd_count_gives_the_same_bytes(device, tuning, xcds, tokens, experts, topk, hidden, alignment):
    """The kernels take the XCD count as an argument (the device's; the XCDS switch stands in for a
    partitioned or another part).  The block remap is a bijection for any count, so every count gives
    the oracle's bytes through every walk; what the count changes is locality, which is not tested."""
    tuning("XCDS", xcds)
    assert cabi.device_topology()[1] == xcds
    idx = cases.routing("dropout", tokens, experts, topk, seed=xcds)
    run_dispatch_combine(device, idx, hidden, experts, alignment, True, True, True, seed=xcds)
    if xcds in (1, 3):
        run_dispatch_combine(device, idx, hidden, experts, alignment, False, False, True, seed=xcds)


@pytest.mark.parametrize(
    "tokens,experts,topk,hidden,alignment",
    [
        pytest.param(700, 12, 4, 512, 16, id="general-kernel-with-zero-fill"),
        pytest.param(900, 40, 8, 5120, 1, id="one-workgroup-a-row"),
        pytest.param(3000, 16, 2, 256, 4, id="weights-in-workgroups-of-their-own"),
    ],
)
def test_device_side_count_with_a_launch_sized_for_another_count(device, tokens, experts, topk, hidden, alignment):
    """A dispatch enqueued before the host knows A may size its launch for an expected count: far
    too small (workgroups take many turns), a little too small, exact, too large.  Same bytes."""
    idx = cases.routing("dropout", tokens, experts, topk, seed=77)
    x = cases.payload(tokens, hidden, seed=8).to(device)
    w = cases.gate_weights(tokens, topk).to(device)
    metadata, counts = cabi.layout(idx.to(device), experts, alignment, True, hidden=hidden)
    assignments = counts[2]
    want_x, _, want_w = cabi.dispatch(x, w, metadata, counts, experts, alignment, True, True, poison=POISON)
    for expected in (2, 9, assignments // 3, assignments - 1, assignments, assignments + 1, tokens * topk, tokens * topk + 1000):
        for span, prefetch in ((1, 0), (2, 0), (1, 1), (2, 1)):
            got_x, _, got_w = cabi.dispatch(x, w, metadata, counts, experts, alignment, True, True, poison=POISON,
                                            order_count=("device", expected), span=span, prefetch=prefetch)
            assert torch.equal(got_x.view(torch.int16), want_x.view(torch.int16)), (expected, span, prefetch)
            assert torch.equal(got_w.view(torch.int32), want_w.view(torch.int32)), (expected, span, prefetch)


@pytest.mark.parametrize("use_order", [True, False], ids=["slot-order", "token-order"])
@pytest.mark.parametrize("bad", ["out-of-range", "duplicate"])
def test_dispatch_behind_a_rejected_layout_stays_inside_its_bound(device, bad, use_order):
    """A caller that enqueues the permute before it has read the counts (outputs at their upper
    bound, entry count read on the device) finds out about a routing error afterwards.  Whatever
    the rejected layout holds, the permute, its zero fill and its weights write nothing outside
    the rows they were given: guard rows on both sides keep their pattern."""
    tokens, experts, topk, hidden, alignment, guard = 700, 12, 4, 512, 16, 8
    idx = cases.routing("dropout", tokens, experts, topk, seed=31)
    if bad == "duplicate":
        idx[5] = 3
        idx[600, 1] = idx[600, 0] = 7
    else:
        idx[5, 2], idx[300, 0], idx[699, 3] = experts, -5, 1 << 40
    x = cases.payload(tokens, hidden, seed=1).to(device)
    w = cases.gate_weights(tokens, topk).to(device)
    metadata, counts = cabi.layout(idx.to(device), experts, alignment, True, raise_on_routing=False, hidden=hidden)
    assert counts[3] & (2 if bad == "duplicate" else 1)
    bound = tokens * topk + experts * (alignment - 1)
    rows = torch.full((guard + bound + guard, hidden), -3.0, dtype=torch.bfloat16, device=device)
    row_weights = torch.full((guard + bound + guard,), -3.0, dtype=torch.float32, device=device)
    order = metadata[8] if use_order else None
    library = cabi.lib()
    cabi.check(library.nanoep_dispatch(
        cabi.ptr(x), cabi.ptr(w), cabi.ptr(metadata[0]), cabi.ptr(metadata[3]), cabi.ptr(metadata[7]), cabi.ptr(order),
        -1 if use_order else 0, cabi.ptr(metadata[1]), cabi.ptr(metadata[2]), tokens, bound, tokens, hidden, topk, experts, alignment, 1, 1,
        rows[guard:].data_ptr(), None, row_weights[guard:].data_ptr(), 0, cabi.stream_handle()))
    torch.cuda.synchronize()
    for name, tensor in (("rows", rows), ("weights", row_weights)):
        edges = torch.cat((tensor[:guard], tensor[guard + bound:])).cpu()
        assert torch.equal(edges, torch.full_like(edges, -3.0)), f"{name} outside the bound were written"
    # every row that was written holds a source row or zeros
    written = rows[guard:guard + bound].cpu()
    touched = (written.view(torch.int16) != torch.tensor(-3.0, dtype=torch.bfloat16).view(torch.int16)).any(dim=1)
    assert touched.any()


@pytest.mark.parametrize("tokens", [300, 5000])
def test_most_local_experts(device, tokens):
    """3839 local experts, the most the assignment kernel's LDS arrays take: layout workgroups of
    32 tokens, eight to a window."""
    experts = 3839
    assert cabi.lib().nanoep_layout_block_tokens(tokens, experts, 0) > 0 and cabi.lib().nanoep_layout_block_tokens(tokens, experts + 1, 0) == 0
    idx = cases.routing("dropout", tokens, experts, 5, seed=tokens)
    run_dispatch_combine(device, idx, 512, experts, 3, True, True, True, seed=tokens)


@pytest.mark.parametrize("seed", range(24))
def test_randomized_shapes(device, seed):
    """Seeded random geometries: ragged token counts, hidden sizes that are not multiples of 512 or
    even of 64 vectors, odd top-k, expert counts past one and two wavefronts of experts, odd
    alignments -- every one checked bit for bit against the oracle through all walks."""
    g = torch.Generator().manual_seed(1000 + seed)

    def pick(options):
        return options[int(torch.randint(len(options), (1,), generator=g))]

    topk = pick([1, 2, 3, 4, 6, 7, 8, 11])
    experts = max(topk, pick([1, 2, 5, 8, 31, 64, 65, 130, 300]))
    tokens = pick([1, 2, 31, 33, 63, 100, 255, 256, 257, 511, 700])
    hidden = 8 * pick([1, 3, 8, 31, 32, 33, 64, 65, 96, 128, 160, 257])
    alignment = pick([1, 1, 2, 3, 8, 128])
    kind = pick(["random", "dropout", "sparse", "biased"])
    expand = pick([False, True, True])
    zero_padding = expand and pick([False, True])
    weighted = pick([False, True])
    idx = cases.routing(kind, tokens, experts, topk, seed=seed)
    run_dispatch_combine(device, idx, hidden, experts, alignment, expand, zero_padding, weighted, seed=seed)


@pytest.mark.parametrize(
    "hidden,tokens",
    [(8200, 300), (16384, 257), (16392, 300), (32768, 260), (32776, 120), (65544, 70)],
    ids=["17-chunks", "32-chunks", "33-chunks", "64-chunks", "65-chunks-token-order", "129-chunks-token-order"],
)
def test_rows_wider_than_a_workgroup_of_single_chunks(device, hidden, tokens):
    """Rows of more than 16 KiB: the slot-order walk moves two or four chunks a wavefront so that 16
    wavefronts still cover a row; rows beyond 64 KiB take the token-order walk.  Bit for bit against
    the oracle either way, with every forced width that still fits."""
    idx = cases.routing("dropout", tokens, 9, 3, seed=hidden)
    run_dispatch_combine(device, idx, hidden, 9, 4, True, True, True, seed=tokens)


@pytest.mark.parametrize("seed", range(10))
def test_randomized_multi_block_shapes(device, seed):
    """Seeded batches of a thousand to nine thousand tokens (many layout blocks, token counts that
    are no multiple of a block, both layout plans by size, rows of 512 bytes to 18 KiB), checked bit
    for bit against the oracle through all walks."""
    g = torch.Generator().manual_seed(7000 + seed)

    def pick(options):
        return options[int(torch.randint(len(options), (1,), generator=g))]

    topk = pick([1, 2, 4, 6, 8, 9, 16])
    experts = max(topk, pick([8, 32, 64, 160, 256, 384, 1000]))
    tokens = pick([1000, 2047, 2048, 3000, 4097, 6000, 8192, 9001])
    hidden = pick([256, 512, 1024, 2048, 2816, 4096, 7168, 8192, 9216])
    alignment = pick([1, 1, 8, 128])
    kind = pick(["random", "dropout", "sparse", "biased"])
    expand = pick([True, True, False])
    zero_padding = expand and pick([False, True])
    weighted = pick([False, True])
    idx = cases.routing(kind, tokens, experts, topk, seed=100 + seed)
    run_dispatch_combine(device, idx, hidden, experts, alignment, expand, zero_padding, weighted, seed=seed)


def test_empty_inputs(device):
    for expand in (False, True):
        idx = torch.empty((0, 4), dtype=torch.int64)
        metadata, counts = cabi.layout(idx.to(device), 8, 4, expand)
        assert counts == (0, 0, 0, 0)
        assert torch.equal(metadata[1].cpu(), torch.zeros(8, dtype=torch.int64))
        assert torch.equal(metadata[2].cpu(), torch.zeros(9, dtype=torch.int64))
        x = torch.empty((0, 256), dtype=torch.bfloat16, device=device)
        got_x, _, _ = cabi.dispatch(x, None, metadata, counts, 8, 4, expand, True)
        assert got_x.shape == (0, 256)
        out, _ = cabi.combine(got_x, None, None, metadata, counts, expand)
        assert out.shape == (0, 256)
    # all tokens masked: nothing received, combine still writes zeros (+bias) for every token
    idx = cases.routing("masked", 7, 4, 2)
    run_dispatch_combine(device, idx, 256, 4, 8, True, True, True, seed=7)


def test_routing_errors_are_reported(device):
    idx = torch.tensor([[0, 1], [5, 1]], dtype=torch.int64)  # 5 is outside [0, 4)
    _, counts = cabi.layout(idx.to(device), 4, 1, True, raise_on_routing=False)
    assert counts[3] & 1
    idx = torch.tensor([[0, 1], [2, 2]], dtype=torch.int64)  # duplicate inside a token
    _, counts = cabi.layout(idx.to(device), 4, 1, True, raise_on_routing=False)
    assert counts[3] & 2
    with pytest.raises(cabi.NanoEPError):
        cabi.layout(idx.to(device), 4, 1, True)


def test_special_values_survive_dispatch_and_round_in_combine(device):
    """NaN payloads, infinities, -0 and subnormals are copied bit for bit; combine's 0 + x turns
    -0 into +0 and keeps subnormal sums exact."""
    tokens, hidden, experts, topk = 6, 256, 4, 2
    idx = torch.tensor([[0, 1], [1, 2], [3, -1], [-1, 2], [0, 3], [2, 1]], dtype=torch.int64)
    patterns = torch.tensor([0x7FC1, 0xFFC0, 0x7F81, 0x7F80, 0xFF80, 0x8000, 0x0001, 0x8001, 0x007F, 0x3F80], dtype=torch.int32)
    raw = patterns.repeat((tokens * hidden + len(patterns) - 1) // len(patterns))[: tokens * hidden]
    x = raw.to(torch.int16).view(torch.bfloat16).reshape(tokens, hidden).contiguous()
    metadata, counts = cabi.layout(idx.to(device), experts, 1, True)
    got_x, _, _ = cabi.dispatch(x.to(device), None, metadata, counts, experts, 1, True, False)
    lay = oracle.layout(idx, experts, 1)
    want_x, _, _, _ = oracle.dispatch(x, idx, experts, None, do_expand=True, lay=lay)
    assert_bits_equal(got_x, want_x, "special values")
    got, _ = cabi.combine(got_x, None, None, metadata, counts, True)
    want, _ = oracle.combine(want_x, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
    got_cpu = got.cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got_cpu), nan)
    assert torch.equal(bits(got_cpu)[~nan], bits(want)[~nan])


def test_accumulation_is_fp32_in_ascending_k(device):
    """((0 + 2^30) - 2^30) + 64 = 64 only when rows are added in ascending k in fp32; 256 + 1 - 256 = 1
    only with an fp32 accumulator."""
    idx = torch.tensor([[0, 1, 2]], dtype=torch.int64)
    metadata, counts = cabi.layout(idx.to(device), 3, 1, True)
    for rows, want in (([2.0**30, -(2.0**30), 64.0], 64.0), ([64.0, 2.0**30, -(2.0**30)], 0.0), ([256.0, 1.0, -256.0], 1.0)):
        y = torch.tensor(rows, dtype=torch.bfloat16).reshape(3, 1).repeat(1, 256).contiguous()
        for use_table in (True, False):
            got, _ = cabi.combine(y.to(device), None, None, metadata, counts, True, use_table=use_table)
            assert (got.float().cpu() == want).all(), (rows, use_table)


def test_reversed_handle_order_is_honoured(device):
    """Combine must follow the handle, not assume token-ordered slots (the reference's
    expert_inputs builds handles with reversed receive and slot order)."""
    idx = cases.routing("mixed", 11, 3, 3, seed=9)
    lay = oracle.layout(idx, 3, 4)
    order = torch.arange(lay.recv_count).flip(0)
    slots = lay.expanded_slots[order].clone()
    local = lay.local_topk_idx[order]
    for expert, count in enumerate(lay.expert_counts.tolist()):
        start = int(lay.expert_offsets[expert])
        mask = local == expert
        slots[mask] = 2 * start + count - 1 - slots[mask]
    tokens = lay.src_tokens[order]
    dst = torch.full((11, 1), -1, dtype=torch.int64)
    dst[tokens, 0] = torch.arange(lay.recv_count)
    for expand in (False, True):
        body = slots if expand else local
        meta = torch.cat((torch.zeros_like(tokens)[:, None], tokens[:, None], body), dim=1).to(torch.int32)
        rows = lay.expanded_capacity if expand else lay.recv_count
        y = cases.payload(rows, 256, seed=4)
        w = cases.gate_weights(rows, 1).flatten() if expand else cases.gate_weights(rows, 3)
        metadata = [meta.to(device), None, None, dst.to(device)]
        counts = (lay.recv_count, lay.expanded_capacity, 0, 0)
        got, got_w = cabi.combine(y.to(device), w.to(device), None, metadata, counts, expand)
        want, want_w = oracle.combine_scalar(y, meta, dst, do_expand=expand, weights=w)
        assert_bits_equal(got, want, "reversed handle x")
        assert_bits_equal(got_w, want_w, "reversed handle weights")
        # cached dispatch follows the same handle: every row lands where the metadata says
        x = cases.payload(11, 256, seed=6)
        xw = cases.gate_weights(11, 3, seed=8)
        metadata = [meta.to(device), lay.expert_counts.to(device), lay.expert_offsets.to(device), dst.to(device)]
        got_x, got_idx, got_xw = cabi.dispatch(x.to(device), xw.to(device), metadata, counts, 3, 4, expand, True)
        got_x, got_xw = got_x.cpu(), got_xw.cpu()
        for row, token in enumerate(tokens.tolist()):
            if expand:
                for k in range(3):
                    slot = int(slots[row, k])
                    if slot >= 0:
                        assert torch.equal(got_x[slot].view(torch.int16), x[token].view(torch.int16))
                        assert got_xw[slot] == xw[token, k]
            else:
                assert torch.equal(got_x[row].view(torch.int16), x[token].view(torch.int16))
                assert torch.equal(got_xw[row], xw[token]) and torch.equal(got_idx.cpu()[row], local[row])
        if expand:
            live = torch.zeros(lay.expanded_capacity, dtype=torch.bool)
            live[slots[slots >= 0]] = True
            assert (got_x[~live].view(torch.int16) == 0).all() and (got_xw[~live] == 0).all()


def expected_slot_order(table: torch.Tensor, window: int, entries: int):
    """Closed form of a slot-order buffer: window of consecutive tokens by window, the valid
    (slot << 32) | (t * K + k) ascending, -1 up to the count word, the count."""
    tokens, topk = table.shape
    flat = table.flatten().to(torch.int64)
    packed = (flat << 32) | torch.arange(flat.numel(), dtype=torch.int64)
    parts = []
    for first in range(0, tokens, window):
        span = slice(first * topk, (first + window) * topk)
        parts.append(packed[span][flat[span] >= 0].sort().values)
    assigned = int((flat >= 0).sum())
    parts.append(torch.full((entries - 1 - assigned,), -1, dtype=torch.int64))
    parts.append(torch.tensor([assigned], dtype=torch.int64))
    return torch.cat(parts)


@pytest.mark.parametrize(
    "tokens,experts,topk,kind,alignment,hidden",
    [
        pytest.param(19, 3, 3, "mixed", 4, 256, id="one-window"),
        pytest.param(1000, 16, 4, "dropout", 8, 512, id="ragged-last-window"),
        pytest.param(4096, 256, 8, "dropout", 1, 7168, id="headline-routing"),
        pytest.param(4096, 8, 2, "random", 1, 4096, id="mixtral-routing"),
        pytest.param(8192, 128, 8, "biased", 128, 2048, id="qwen3-routing"),
        pytest.param(3000, 40, 17, "sparse", 3, 1024, id="odd-topk-window-halved"),
        pytest.param(700, 64, 32, "random", 1, 256, id="top-32"),
        pytest.param(2500, 8, 1, "dropout", 16, 8192, id="top-1"),
        pytest.param(600, 8, 2, "masked", 1, 512, id="nothing-received"),
    ],
)
def test_private_tensors_rebuilt_from_the_public_ones(device, tokens, experts, topk, kind, alignment, hidden):
    """nanoep_rebuild_order reads nothing but recv_metadata and dst_slots, and gives the layout's own
    slot table back bit for bit, and a slot-order list that is the closed form for its window size
    (the layout's own list when both take the same window); the dispatch that walks the rebuilt pair
    writes the same bytes, with the count from the host and from the device."""
    idx = cases.routing(kind, tokens, experts, topk, seed=17)
    metadata, counts = cabi.layout(idx.to(device), experts, alignment, True, hidden=hidden)
    public = metadata[:7]
    tag = 5 << 32
    table, order, word = cabi.rebuild_order(public, counts, experts, hidden, host_tag=tag)
    assert torch.equal(table.cpu(), metadata[7].cpu())
    window = cabi.lib().nanoep_rebuild_window_tokens(tokens, topk, hidden)
    assert window * topk <= 4096 and window >= 32
    assert torch.equal(order.cpu(), expected_slot_order(metadata[7].cpu(), window, order.numel()))
    assert word == tag | counts[2]
    if window == cabi.lib().nanoep_layout_block_tokens(tokens, experts, hidden):
        assert torch.equal(order.cpu(), metadata[8].cpu())
    if counts[0] == 0:
        return
    x, w = cases.payload(tokens, hidden, seed=3), cases.gate_weights(tokens, topk)
    want_x, _, want_w = cabi.dispatch(x.to(device), w.to(device), public, counts, experts, alignment, True, True, poison=POISON)
    rebuilt = public + [table, order]
    for order_count in ("exact", "device"):
        got_x, _, got_w = cabi.dispatch(x.to(device), w.to(device), rebuilt, counts, experts, alignment, True, True, poison=POISON,
                                        order_count=order_count)
        assert torch.equal(got_x.view(torch.int16), want_x.view(torch.int16))
        assert torch.equal(got_w.view(torch.int32), want_w.view(torch.int32))


def test_rebuild_follows_a_handle_in_another_order(device):
    """A coherent handle with reversed receive rows and reversed slots inside every expert segment
    (as the reference's expert_inputs builds them, nano_ep/testing/native_combine.py:62-74), plus
    slots outside the capacity that must be dropped: the rebuilt pair says what the handle says."""
    tokens, experts, topk, hidden, alignment = 1500, 12, 4, 512, 4
    idx = cases.routing("dropout", tokens, experts, topk, seed=23)
    lay = oracle.layout(idx, experts, alignment)
    meta = lay.recv_metadata(True).flip(0).contiguous()
    slots = meta[:, 2:].clone().to(torch.int64)
    expert_of = torch.bucketize(slots.clamp(min=0), lay.expert_offsets[1:], right=True)
    mirrored = lay.expert_offsets[expert_of] + lay.expert_counts[expert_of] - 1 - (slots - lay.expert_offsets[expert_of])
    meta[:, 2:] = torch.where(slots >= 0, mirrored, slots).to(torch.int32)
    meta[5, 2] = lay.expanded_capacity  # one past the last row: not a slot
    meta[7, 3] = -3
    dst = torch.where(lay.dst_slots >= 0, lay.recv_count - 1 - lay.dst_slots, lay.dst_slots)
    dst[int(meta[11, 1]), 0] = lay.recv_count  # a token pointing past the receive rows is not sent
    want_table = torch.full((tokens, topk), -1, dtype=torch.int32)
    for token in range(tokens):
        row = int(dst[token, 0])
        if 0 <= row < lay.recv_count:
            values = meta[row, 2:]
            want_table[token] = torch.where((values >= 0) & (values < lay.expanded_capacity), values, torch.full_like(values, -1))
    public = [meta.to(device), lay.expert_counts.to(device), lay.expert_offsets.to(device), dst.to(device)]
    counts = (lay.recv_count, lay.expanded_capacity, 0, 0)
    table, order, _ = cabi.rebuild_order(public, counts, experts, hidden)
    assert torch.equal(table.cpu(), want_table)
    window = cabi.lib().nanoep_rebuild_window_tokens(tokens, topk, hidden)
    assert torch.equal(order.cpu(), expected_slot_order(want_table, window, order.numel()))
    x, w = cases.payload(tokens, hidden, seed=5), cases.gate_weights(tokens, topk)
    want_x, _, want_w = cabi.dispatch(x.to(device), w.to(device), public, counts, experts, alignment, True, True, poison=POISON)
    got_x, _, got_w = cabi.dispatch(x.to(device), w.to(device), public + [None, None, None, table, order], counts, experts, alignment,
                                    True, True, poison=POISON, order_count="device")
    assert torch.equal(got_x.view(torch.int16), want_x.view(torch.int16))
    assert torch.equal(got_w.view(torch.int32), want_w.view(torch.int32))
    # every row the table names holds its token; the rows of the dropped entries are nobody's and keep the poison
    live = want_table >= 0
    rows = want_table[live].to(torch.int64)
    source = torch.arange(tokens)[:, None].expand(-1, topk)[live]
    assert_bits_equal(got_x.cpu()[rows], x[source], "rows follow the rebuilt table")
    dropped = [int(mirrored[row, k]) for row, k in [(5, 0), (7, 1)] + [(11, k) for k in range(topk)] if slots[row, k] >= 0]
    assert dropped and (got_x.cpu()[torch.tensor(dropped)].view(torch.uint8) == POISON).all()


def test_window_layout_known_answer():
    assert cabi.window_layout(2, 8, 256, 2, 4) == [0, 96, 160, 160, 9888]
