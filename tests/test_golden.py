"""Hand-derived known answers (tests/golden/known_answers.json) against the oracle on the CPU and
against the HIP kernels through the C ABI on the GPU.  The fixture was written by hand from the
layout rules; nothing computed it."""

import json
from pathlib import Path

import numpy as np
import pytest
import torch

import cabi
from oracle import nanoep_oracle as oracle

GOLDEN = json.loads((Path(__file__).parent / "golden" / "known_answers.json").read_text())
CASES = {case["name"]: case for case in GOLDEN["cases"]}
HIDDEN = 256


def rows(values, dtype=torch.bfloat16):
    """[len(values), HIDDEN] with every element of row i equal to values[i]."""
    return torch.tensor(values, dtype=torch.float32).repeat_interleave(HIDDEN).reshape(len(values), HIDDEN).to(dtype)


def expected_layout_tensors(case, expand):
    metadata = case["recv_metadata_expanded" if expand else "recv_metadata_compact"]
    return (
        torch.tensor(metadata, dtype=torch.int32),
        torch.tensor(case["expert_counts"], dtype=torch.int64),
        torch.tensor(case["expert_offsets"], dtype=torch.int64),
        torch.tensor(case["dst_slots"], dtype=torch.int64).reshape(-1, 1),
    )


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("impl", [oracle.layout_scalar, oracle.layout], ids=["scalar", "vectorised"])
def test_oracle_layout_matches_the_known_answers(impl, name):
    case = CASES[name]
    idx = torch.tensor(case["topk_idx"], dtype=torch.int64)
    lay = impl(idx, case["experts"], case["alignment"])
    assert lay.recv_count == case["recv_count"] and lay.expanded_capacity == case["expanded_capacity"]
    for expand in (False, True):
        want_meta, want_counts, want_offsets, want_dst = expected_layout_tensors(case, expand)
        assert torch.equal(lay.recv_metadata(expand), want_meta)
        assert torch.equal(lay.expert_counts, want_counts) and torch.equal(lay.expert_offsets, want_offsets)
        assert torch.equal(lay.dst_slots, want_dst)


@pytest.mark.parametrize("scalar", [True, False], ids=["scalar", "vectorised"])
def test_oracle_dispatch_and_combine_match_the_known_answers(scalar):
    case = CASES["mixed_hand"]
    idx = torch.tensor(case["topk_idx"], dtype=torch.int64)
    x, w = rows(case["x_row_values"]), torch.tensor(case["weights"], dtype=torch.float32)
    dispatch = oracle.dispatch_scalar if scalar else oracle.dispatch
    combine = oracle.combine_scalar if scalar else oracle.combine
    out_x, _, out_w, _ = dispatch(x, idx, case["experts"], w, do_expand=True, alignment=case["alignment"])
    assert torch.equal(out_x, rows(case["expanded_x_row_values"]))
    assert torch.equal(out_w, torch.tensor(case["expanded_weights"], dtype=torch.float32))
    out_x, out_idx, out_w, _ = dispatch(x, idx, case["experts"], w, do_expand=False, alignment=case["alignment"])
    assert torch.equal(out_x, rows(case["compact_x_row_values"]))
    assert torch.equal(out_w, torch.tensor(case["compact_weights"], dtype=torch.float32))
    assert torch.equal(out_idx, torch.tensor(case["recv_metadata_compact"], dtype=torch.int64)[:, 2:])
    meta, _, _, dst = expected_layout_tensors(case, True)
    y, yw = rows(case["combine_y_row_values"]), torch.tensor(case["combine_y_weights"], dtype=torch.float32)
    got, got_w = combine(y, meta, dst, do_expand=True, weights=yw)
    assert torch.equal(got, rows(case["combine_expanded_out_row_values"]))
    assert torch.equal(got_w, torch.tensor(case["combine_expanded_out_weights"], dtype=torch.float32))
    got, _ = combine(y, meta, dst, do_expand=True, bias=rows(case["combine_bias_row_values"]))
    assert torch.equal(got, rows(case["combine_expanded_out_with_bias_row_values"]))


def test_bf16_rounding_known_answers():
    for probe in GOLDEN["bf16_round_to_nearest_even"]:
        bits = np.array([int(probe["f32_bits"], 16)], dtype=np.uint32)
        want = int(probe["bf16_bits"], 16)
        assert int(oracle.bf16_round_bits(bits.view(np.float32))[0]) == want, probe["note"]
        cast = torch.from_numpy(bits.view(np.float32).copy()).to(torch.bfloat16).view(torch.int16)
        assert int(cast[0]) & 0xFFFF == want, probe["note"]


def test_window_layout_known_answer():
    probe = GOLDEN["window_layout"]
    assert oracle.window_layout(*probe["args"]) == probe["expected"]
    assert cabi.window_layout(*probe["args"]) == probe["expected"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("expand", [False, True], ids=["compact", "expanded"])
def test_gpu_layout_matches_the_known_answers(device, name, expand):
    case = CASES[name]
    idx = torch.tensor(case["topk_idx"], dtype=torch.int64, device=device)
    metadata, counts = cabi.layout(idx, case["experts"], case["alignment"], expand)
    assert counts[0] == case["recv_count"] and counts[1] == case["expanded_capacity"] and counts[3] == 0
    want_meta, want_counts, want_offsets, want_dst = expected_layout_tensors(case, expand)
    assert torch.equal(metadata[0].cpu(), want_meta)
    assert torch.equal(metadata[1].cpu(), want_counts) and torch.equal(metadata[2].cpu(), want_offsets)
    assert torch.equal(metadata[3].cpu(), want_dst)
    assert torch.equal(metadata[5].cpu(), idx.cpu())
    assert metadata[4].tolist() == [case["recv_count"]] and metadata[6].tolist() == [case["recv_count"]]


@pytest.mark.gpu
def test_gpu_dispatch_and_combine_match_the_known_answers(device):
    case = CASES["mixed_hand"]
    idx = torch.tensor(case["topk_idx"], dtype=torch.int64, device=device)
    x, w = rows(case["x_row_values"]).to(device), torch.tensor(case["weights"], dtype=torch.float32, device=device)
    experts, alignment = case["experts"], case["alignment"]
    for use_order in (True, False):
        metadata, counts = cabi.layout(idx, experts, alignment, True)
        out_x, _, out_w = cabi.dispatch(x, w, metadata, counts, experts, alignment, True, True, use_order=use_order)
        assert torch.equal(out_x.cpu(), rows(case["expanded_x_row_values"]))
        assert torch.equal(out_w.cpu(), torch.tensor(case["expanded_weights"], dtype=torch.float32))
    y = rows(case["combine_y_row_values"]).to(device)
    yw = torch.tensor(case["combine_y_weights"], dtype=torch.float32, device=device)
    got, got_w = cabi.combine(y, yw, None, metadata, counts, True)
    assert torch.equal(got.cpu(), rows(case["combine_expanded_out_row_values"]))
    assert torch.equal(got_w.cpu(), torch.tensor(case["combine_expanded_out_weights"], dtype=torch.float32))
    got, _ = cabi.combine(y, None, rows(case["combine_bias_row_values"]).to(device), metadata, counts, True)
    assert torch.equal(got.cpu(), rows(case["combine_expanded_out_with_bias_row_values"]))
    metadata, counts = cabi.layout(idx, experts, alignment, False)
    out_x, out_idx, out_w = cabi.dispatch(x, w, metadata, counts, experts, alignment, False, False)
    assert torch.equal(out_x.cpu(), rows(case["compact_x_row_values"]))
    assert torch.equal(out_w.cpu(), torch.tensor(case["compact_weights"], dtype=torch.float32))
    assert torch.equal(out_idx.cpu(), torch.tensor(case["recv_metadata_compact"], dtype=torch.int64)[:, 2:])
