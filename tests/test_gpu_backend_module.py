"""The native module `_nanoep_torch` driven the way the reference's own Python class drives its
backend module, with nothing of nanoep_amd's Python layer in between.

What is replayed, call for call:
  * the bootstrap of CudaBuffer.__init__ (nano_ep/backends/cuda.py:155-193): window_layout ->
    PeerRuntime(rank, world_size, num_bytes) -> local_window()[count_offset : ...].fill_(255) ->
    export_local_handle -> import_peer_handles -> torch.cuda.Stream, and its known answers
    (tests/unit/test_cuda_bootstrap.py:102-106, 175-178);
  * close_peer_runtime (cuda.py:75-86): close_peer_mappings, then close;
  * dispatch / combine with the positional argument lists and the seven-tensor metadata lists of
    cuda.py:296-326 and :398-421, fresh, cached and asynchronous, against the CPU oracle;
  * the JIT warm-up entry points with the argument lists the reference's launch tests pass
    (tests/distributed/test_acceptance.py:46-49): accepted, nothing to compile.
"""

import pytest
import torch

import cases
from nanoep_amd._native import load_extension
from oracle import nanoep_oracle as oracle

pytestmark = pytest.mark.gpu


def same_bits(actual, expected):
    actual, expected = actual.detach().cpu().contiguous(), expected.contiguous()
    view = torch.int16 if actual.dtype == torch.bfloat16 else torch.int32
    return actual.shape == expected.shape and actual.dtype == expected.dtype and torch.equal(actual.view(view), expected.view(view))


class ReferenceShapedBuffer:
    """The reference CudaBuffer's use of its backend module at world_size == 1, restated: the same
    calls in the same order with the same arguments, no collectives (a single rank gathers its own
    handle)."""

    def __init__(self, native, device, experts, topk, hidden, max_tokens, allow_multiple_reduction=False):
        self.native, self.device = native, device
        self.experts, self.topk, self.hidden, self.max_tokens = experts, topk, hidden, max_tokens
        self.multiple = allow_multiple_reduction
        self.device_sms = torch.cuda.get_device_properties(device).multi_processor_count
        (self.signal_offset, self.count_offset, self.payload_offset, self.return_offset, self.num_bytes) = native.window_layout(
            1, max_tokens, hidden, topk, experts, allow_multiple_reduction)
        self.runtime = native.PeerRuntime(0, 1, self.num_bytes)
        window = self.runtime.local_window()
        window[self.count_offset : self.count_offset + (1 + experts) * 8].fill_(255)
        torch.cuda.current_stream(device).synchronize()
        del window
        self.handle = self.runtime.export_local_handle()
        self.runtime.import_peer_handles([self.handle])
        self.comm_stream = torch.cuda.Stream(device=device)

    def dispatch(self, x, routing, weights, *, alignment=1, cached=None, expand=False, zero_padding=False, previous_event=None,
                 async_op=False):
        cached_metadata, cached_capacity = ([], 0) if cached is None else (cached[0], cached[1])
        return self.native.dispatch(
            self.runtime, x, routing, weights, self.experts, self.max_tokens, alignment, cached_metadata, cached_capacity,
            self.multiple, expand, zero_padding, self.device_sms, self.comm_stream.cuda_stream,
            -1 if previous_event is None else previous_event.cuda_event, async_op)

    def combine(self, x, metadata, weights, bias, *, expand, previous_event=None, async_op=False):
        with torch.cuda.device(self.device):
            return self.native.combine(
                self.runtime, x, metadata, weights, bias, self.max_tokens, expand, self.multiple, self.device_sms,
                self.comm_stream.cuda_stream, -1 if previous_event is None else previous_event.cuda_event, async_op)

    def close(self):
        torch.cuda.synchronize(self.device)
        self.runtime.close_peer_mappings()
        self.runtime.close()


def test_bootstrap_sequence_and_runtime_surface(device):
    native = load_extension()
    assert native.window_layout(2, 8, 256, 2, 4, False) == [0, 96, 160, 160, 9888]
    assert native.window_layout(2, 8, 256, 2, 4) == [0, 96, 160, 160, 9888]  # allow_multiple_reduction defaults to False
    with pytest.raises(ValueError):
        native.window_layout(2, 8, 256, 2, 5, False)  # experts not divisible by ranks

    experts, topk, hidden, max_tokens = 8, 2, 256, 64
    signal, count, payload, returned, num_bytes = native.window_layout(1, max_tokens, hidden, topk, experts, False)
    assert signal == 0 and count % 32 == 0 and payload == returned and payload >= count + (1 + experts) * 8 and num_bytes > payload
    runtime = native.PeerRuntime(0, 1, num_bytes)

    window = runtime.local_window()
    assert window.dtype == torch.uint8 and window.is_cuda and tuple(window.shape) == (num_bytes,) and window.is_contiguous()
    assert int(window.count_nonzero()) == 0  # send cursors and barrier signals start at zero
    window[count : count + (1 + experts) * 8].fill_(255)
    torch.cuda.current_stream(device).synchronize()
    again = runtime.local_window()
    assert again.data_ptr() == window.data_ptr()
    counts = again[count : count + (1 + experts) * 8].view(torch.int64)
    assert torch.equal(counts.cpu(), torch.full((1 + experts,), -1, dtype=torch.int64))  # all-one bytes are int64 -1
    assert int(again[:count].count_nonzero()) == 0 and int(again[count + (1 + experts) * 8 :].count_nonzero()) == 0

    handle = runtime.export_local_handle()
    assert isinstance(handle, bytes) and len(handle) == 64
    for wrong in ([], [handle, handle]):
        with pytest.raises(ValueError, match="exactly one handle"):
            runtime.import_peer_handles(wrong)
    with pytest.raises(ValueError, match="exactly 64 bytes"):
        runtime.import_peer_handles([handle[:63]])
    with pytest.raises(ValueError, match="exactly 64 bytes"):
        runtime.import_peer_handles([handle + b"\0"])
    runtime.import_peer_handles([handle])

    addresses = runtime.peer_addresses()
    assert addresses.dtype == torch.int64 and addresses.is_cuda and tuple(addresses.shape) == (1,)
    assert int(addresses[0]) == runtime.local_window().data_ptr()

    stream = torch.cuda.Stream(device=device)
    runtime.barrier(stream.cuda_stream)  # next epoch
    runtime.barrier(stream.cuda_stream, 5)  # explicit epoch
    runtime.barrier(stream.cuda_stream)  # epoch 6
    with pytest.raises(RuntimeError, match="strictly increase"):
        runtime.barrier(stream.cuda_stream, 6)
    runtime.barrier(stream.cuda_stream, 7)
    stream.synchronize()

    # the JIT warm-ups of the reference's launch tests: (hidden, topk, world_size, experts_per_rank, max_tokens, ...)
    geometry = (hidden, topk, 1, experts, max_tokens)
    assert native.init_jit("/nonexistent/source/dir") is None
    for cached in (False, True):
        for expand in (False, True):
            assert native.prepare_dispatch(*geometry, 16, cached, expand, True, expand) is None
    assert native.prepare_combine(*geometry, True, False, True) is None

    # close order (close_peer_runtime): unmap first, then free; both may be repeated
    with pytest.raises(RuntimeError, match="close_peer_mappings"):
        runtime.close()
    runtime.close_peer_mappings()
    runtime.close_peer_mappings()
    runtime.close()
    runtime.close()
    for call in (runtime.local_window, runtime.peer_addresses, lambda: runtime.barrier(stream.cuda_stream),
                 lambda: runtime.import_peer_handles([handle])):
        with pytest.raises(RuntimeError, match="closed"):
            call()

    # a runtime that never imported handles still has to unmap before it frees
    lonely = native.PeerRuntime(0, 1, 0)
    with pytest.raises(RuntimeError, match="close_peer_mappings"):
        lonely.close()
    lonely.close_peer_mappings()
    lonely.close()
    with pytest.raises(RuntimeError):
        native.PeerRuntime(1, 2, 64)  # one rank only


@pytest.mark.parametrize(
    "expand,alignment,zero_padding,kind",
    [
        pytest.param(False, 1, False, "mixed", id="compact"),
        pytest.param(False, 4, False, "dropout", id="compact-aligned-counts"),
        pytest.param(True, 1, True, "dropout", id="expanded"),
        pytest.param(True, 16, True, "mixed", id="expanded-padded"),
    ],
)
def test_fresh_cached_and_combine_through_seven_tensor_metadata(device, expand, alignment, zero_padding, kind):
    """Fresh dispatch, cached replays (with and without weights, as tests/native/test_native_dispatch.py:163-175
    toggles them) and combine, every call with exactly the reference's seven metadata tensors."""
    native = load_extension()
    tokens, experts, topk, hidden = 333, 24, 4, 768
    idx = cases.routing(kind, tokens, experts, topk, seed=17)
    x, w = cases.payload(tokens, hidden, seed=5), cases.gate_weights(tokens, topk)
    bias = cases.payload(tokens, hidden, seed=6)
    want_x, want_idx, want_w, lay = oracle.dispatch(x, idx, experts, w, do_expand=expand, alignment=alignment)
    live = torch.ones(want_x.shape[0], dtype=torch.bool)
    if expand and not zero_padding:
        live[:] = False
        live[lay.expanded_slots[lay.expanded_slots >= 0]] = True
    buffer = ReferenceShapedBuffer(native, device, experts, topk, hidden, 512)
    try:
        idx_gpu = idx.to(device)
        outputs, metadata, counts, completed = buffer.dispatch(x.to(device), idx_gpu, w.to(device), alignment=alignment,
                                                               expand=expand, zero_padding=zero_padding)
        assert completed is None and tuple(counts) == (lay.recv_count, lay.expanded_capacity)
        assert len(outputs) == 3 and len(metadata) >= 7
        seven = list(metadata[:7])  # what cuda.py:296-304 rebuilds from the handle
        for got, want in zip(seven, lay.metadata(expand)):
            assert got.dtype == want.dtype and got.is_contiguous() and torch.equal(got.cpu(), want)
        idx_gpu.fill_(-1)  # the snapshot is the handle's own copy
        assert torch.equal(seven[5].cpu(), idx)
        assert same_bits(outputs[0][live.to(device)], want_x[live])
        if expand:
            assert outputs[1].numel() == 0 and outputs[1].dtype == torch.int64
            assert same_bits(outputs[2][live.to(device)], want_w[live])
        else:
            assert torch.equal(outputs[1].cpu(), want_idx) and same_bits(outputs[2], want_w)

        # cached replays: new payload, weights present then absent, the identical seven tensors come back
        for step, weighted in ((1, True), (2, False)):
            new_x, new_w = x * 2 + step, (w * step if weighted else None)
            cached_out, cached_meta, cached_counts, _ = buffer.dispatch(
                new_x.to(device), seven[5], None if new_w is None else new_w.to(device), alignment=alignment,
                cached=(seven, lay.expanded_capacity), expand=expand, zero_padding=zero_padding)
            assert tuple(cached_counts) == (lay.recv_count, lay.expanded_capacity)
            assert all(a.data_ptr() == b.data_ptr() for a, b in zip(cached_meta[:7], seven))
            replay_x, _, replay_w, _ = oracle.dispatch(new_x, idx, experts, new_w, do_expand=expand, alignment=alignment)
            assert same_bits(cached_out[0][live.to(device)], replay_x[live])
            if weighted:
                assert same_bits(cached_out[2][live.to(device)], replay_w[live] if expand else replay_w)
            else:
                assert cached_out[2].numel() == 0 and cached_out[2].dtype == torch.float32
        assert same_bits(outputs[0][live.to(device)], want_x[live])  # the fresh result kept its bytes

        # combine: expert outputs with zeros in the gaps, as the oracle's padding is zero
        y = cases.payload(want_x.shape[0], hidden, seed=9)
        y[~live] = 0
        y_w = want_w.clone()
        for with_weights, with_bias in ((False, False), (True, True)):
            (combined, restored), done = buffer.combine(
                y.to(device), seven, y_w.to(device) if with_weights else None, bias.to(device) if with_bias else None, expand=expand)
            want, want_cw = oracle.combine(y, lay.recv_metadata(expand), lay.dst_slots, do_expand=expand,
                                           weights=y_w if with_weights else None, bias=bias if with_bias else None)
            assert done is None and same_bits(combined, want)
            if with_weights:
                assert same_bits(restored, want_cw)
            else:
                assert restored.numel() == 0 and restored.dtype == torch.float32

        # asynchronous calls return a CompletionEvent the consumer stream waits on
        producer = torch.cuda.Stream(device=device)
        with torch.cuda.stream(producer):
            late_x = (x + 3).to(device, non_blocking=False)
            ready = torch.cuda.Event()
            ready.record(producer)
        async_out, _, _, done = buffer.dispatch(late_x, seven[5], None, alignment=alignment, cached=(seven, lay.expanded_capacity),
                                                expand=expand, zero_padding=zero_padding, previous_event=ready, async_op=True)
        assert isinstance(done, native.CompletionEvent)
        done.current_stream_wait()
        late_want, _, _, _ = oracle.dispatch(x + 3, idx, experts, None, do_expand=expand, alignment=alignment)
        assert same_bits(async_out[0][live.to(device)], late_want[live])
        (async_combined, _), done = buffer.combine(y.to(device), seven, None, None, expand=expand, async_op=True)
        done.current_stream_wait()
        want, _ = oracle.combine(y, lay.recv_metadata(expand), lay.dst_slots, do_expand=expand)
        assert same_bits(async_combined, want)
    finally:
        buffer.close()
    with pytest.raises(RuntimeError, match="closed"):
        buffer.dispatch(x.to(device), idx.to(device), None)
    with pytest.raises(RuntimeError, match="closed"):
        buffer.combine(y.to(device), seven, None, None, expand=expand)


def test_native_argument_checks_keep_the_reference_wording(device):
    """The substrings callers of the reference match on (tests/distributed/worker.py:324-341)."""
    native = load_extension()
    tokens, experts, topk, hidden = 16, 4, 2, 256
    buffer = ReferenceShapedBuffer(native, device, experts, topk, hidden, 32)
    try:
        idx = cases.routing("random", tokens, experts, topk).to(device)
        x = cases.payload(tokens, hidden).to(device)
        _, metadata, counts, _ = buffer.dispatch(x, idx, None, expand=True)
        seven = list(metadata[:7])
        with pytest.raises(RuntimeError, match="bfloat16"):
            buffer.dispatch(x.float(), idx, None)
        with pytest.raises(RuntimeError, match="bfloat16"):
            buffer.combine(torch.zeros((counts[1], hidden), device=device), seven, None, None, expand=True)
        with pytest.raises(RuntimeError, match="multiple of 256"):
            buffer.dispatch(x[:, :128].contiguous(), idx, None)
        with pytest.raises(RuntimeError, match="16-byte aligned"):
            flat = torch.zeros(tokens * hidden + 8, dtype=torch.bfloat16, device=device)
            buffer.dispatch(flat[1 : 1 + tokens * hidden].view(tokens, hidden), idx, None)
        with pytest.raises(RuntimeError, match="int64"):
            buffer.dispatch(x, idx.int(), None)
        with pytest.raises(RuntimeError, match="max_tokens"):
            big = torch.zeros((33, hidden), dtype=torch.bfloat16, device=device)
            buffer.dispatch(big, torch.zeros((33, topk), dtype=torch.int64, device=device), None)
        with pytest.raises(RuntimeError, match="float32"):
            buffer.dispatch(x, idx, torch.zeros((tokens, topk), dtype=torch.float64, device=device))
        with pytest.raises(RuntimeError, match="seven prepared"):
            buffer.dispatch(x, idx, None, cached=(seven[:6], counts[1]), expand=True)
        for position, name in ((0, "recv_metadata"), (1, "expert_counts"), (2, "expert_offsets"), (3, "dst_slots"), (4, "send_counts"),
                               (6, "recv_rank_prefix")):
            broken = list(seven)
            broken[position] = seven[position].to(torch.float32)
            with pytest.raises(RuntimeError, match=f"cached {name} has invalid CUDA storage or shape"):
                buffer.dispatch(x, seven[5], None, cached=(broken, counts[1]), expand=True)
            with pytest.raises(RuntimeError, match=f"cached {name} has invalid CUDA storage or shape"):
                buffer.combine(torch.zeros((counts[1], hidden), dtype=torch.bfloat16, device=device), broken, None, None, expand=True)
    finally:
        buffer.close()
