"""nanoep_layout_static (the layout entry point that allocates nothing: its workspace is a device
array of the library) gives the results of nanoep_layout bit for bit, call after call."""

import pytest
import torch

import cabi
import cases

pytestmark = pytest.mark.gpu


def same_layout(got, want):
    (got_meta, got_counts), (want_meta, want_counts) = got, want
    assert got_counts == want_counts
    assert len(got_meta) == len(want_meta)
    for index, (a, b) in enumerate(zip(got_meta, want_meta)):
        assert a.dtype == b.dtype and a.shape == b.shape, index
        assert torch.equal(a.cpu(), b.cpu()), f"handle tensor {index} differs"


@pytest.mark.parametrize("expand", [True, False])
def test_static_scratch_layout_equals_the_workspace_layout_twice_in_a_row(device, expand):
    # the second call is smaller: whatever the first left in the array must not show
    for tokens, experts, topk, alignment, hidden, kind in ((4096, 256, 8, 1, 7168, "dropout"), (1000, 40, 5, 16, 2048, "mixed")):
        idx = cases.routing(kind, tokens, experts, topk, seed=tokens).to(device)
        print("nanoep_layout_static", tokens, experts, topk, alignment, hidden, kind, "expand", expand, flush=True)
        want = cabi.layout(idx, experts, alignment, expand, hidden=hidden)
        got = cabi.layout(idx, experts, alignment, expand, hidden=hidden, static_scratch=True)
        same_layout(got, want)


def test_static_scratch_layout_feeds_dispatch_and_combine(device):
    from oracle import nanoep_oracle as oracle

    tokens, experts, topk, hidden, alignment = 777, 24, 6, 512, 8
    idx_cpu = cases.routing("dropout", tokens, experts, topk, seed=3)
    x_cpu, w_cpu = cases.payload(tokens, hidden), cases.gate_weights(tokens, topk)
    metadata, counts = cabi.layout(idx_cpu.to(device), experts, alignment, True, hidden=hidden, static_scratch=True)
    recv_x, _, recv_w = cabi.dispatch(x_cpu.to(device), w_cpu.to(device), metadata, counts, experts, alignment, True, True)
    want_x, _, want_w, lay = oracle.dispatch(x_cpu, idx_cpu, experts, w_cpu, do_expand=True, alignment=alignment)
    assert counts[0] == lay.recv_count and counts[1] == lay.expanded_capacity
    assert torch.equal(recv_x.cpu().view(torch.int16), want_x.view(torch.int16))
    assert torch.equal(recv_w.cpu().view(torch.int32), want_w.view(torch.int32))
    out_x, _ = cabi.combine(recv_x, None, None, metadata, counts, True)
    want, _ = oracle.combine(want_x, lay.recv_metadata(True), lay.dst_slots, do_expand=True)
    assert torch.equal(out_x.cpu().view(torch.int16), want.view(torch.int16))


def test_static_scratch_layout_refuses_what_does_not_fit(device):
    idx = torch.zeros((131072, 8), dtype=torch.int64, device=device)
    with pytest.raises(cabi.NanoEPError) as raised:
        cabi.layout(idx, 256, 1, False, static_scratch=True)
    assert raised.value.status == 6 and "static scratch" in str(raised.value)
