"""CPU doubles check the Python layer only: argument resolution, the positional order handed to the
native module, handle packaging and event keep-alives.  The fake backend's signature IS the operator
boundary, in the order the reference's unit tests pin (tests/unit/test_cuda_dispatch.py:77-94,
tests/unit/test_cuda_combine.py:141-154)."""

from types import SimpleNamespace

import pytest
import torch

from nanoep_amd import EPConfig, buffer as api
from nanoep_amd.config import EPConfig as ConfigAlias


class FakeStream:
    def __init__(self, handle, device=None):
        self.cuda_stream = handle
        self.waited_for = []

    def wait_stream(self, other):
        self.waited_for.append(other.cuda_stream)


class FakeTensor:
    """Shape/dtype carrier that stands in for a device tensor."""

    device = torch.device("cuda", 0)

    def __init__(self, name, payload):
        self.name, self.payload = name, payload

    dtype = property(lambda self: self.payload.dtype)
    shape = property(lambda self: self.payload.shape)

    def is_contiguous(self):
        return self.payload.is_contiguous()


class FakeNativeEvent:
    def __init__(self):
        self.waits = 0

    def current_stream_wait(self):
        self.waits += 1


@pytest.fixture
def context(monkeypatch):
    calls = []

    def i64(name, data):
        return FakeTensor(name, torch.tensor(data, dtype=torch.int64))

    def dispatch(runtime, x, routing, weights, experts, capacity, alignment, cached, cached_capacity, mode, expand, zero_padding,
                 num_sms, comm_stream, previous_event, async_op):
        metadata = cached or [
            FakeTensor("recv_metadata", torch.tensor([[0, 0, 0, 1, -1], [0, 1, -1, -1, 2]], dtype=torch.int32)),
            i64("expert_counts", [1, 1, 1]),
            i64("expert_offsets", [0, alignment, 2 * alignment, 3 * alignment]),
            i64("dst_slots", [[0], [1]]),
            i64("send_counts", [2]),
            FakeTensor("snapshot", routing.payload.clone()),
            i64("recv_rank_prefix", [2]),
        ] + ([FakeTensor("token_slots", torch.zeros((2, 3), dtype=torch.int32))] if expand else [])
        capacity_out = cached_capacity if cached else 3 * alignment
        rows = capacity_out if expand else 2
        outputs = (
            FakeTensor("recv_x", torch.zeros((rows, 256), dtype=x.dtype)),
            FakeTensor("recv_idx", torch.empty(0, dtype=torch.int64) if expand else torch.zeros((2, 3), dtype=torch.int64)),
            FakeTensor("recv_w", torch.zeros((rows,) if expand else (rows, 3)) if weights is not None else torch.empty(0)),
        )
        completed = FakeNativeEvent() if async_op else None
        calls.append(SimpleNamespace(kind="dispatch", args=(runtime, x, routing, weights, experts, capacity, alignment, cached,
                                                           cached_capacity, mode, expand, zero_padding, num_sms, comm_stream,
                                                           previous_event, async_op), metadata=metadata, outputs=outputs,
                                     completed=completed))
        return outputs, metadata, (2, capacity_out), completed

    def combine(*args):
        x, metadata, weights = args[1], args[2], args[3]
        tokens = metadata[5].shape[0]
        outputs = (
            FakeTensor("combined_x", torch.zeros((tokens, x.shape[1]), dtype=x.dtype)),
            FakeTensor("combined_w", torch.zeros((tokens, 3)) if weights is not None else torch.empty(0)),
        )
        completed = FakeNativeEvent() if args[-1] else None
        calls.append(SimpleNamespace(kind="combine", args=args, outputs=outputs, completed=completed))
        return outputs, completed

    monkeypatch.setattr(api.torch.cuda, "device", lambda device: __import__("contextlib").nullcontext())
    buffer = api.CudaBuffer.__new__(api.CudaBuffer)
    buffer._config = EPConfig(3, 3, 256, 5)
    buffer._device = buffer._rank = 0
    buffer._device_sms = 256
    buffer._gpu_uuids = ("gpu-0",)
    buffer._auto_num_sms = None
    buffer._closed = False
    buffer._world_size = 1
    # budgets of 64 compute units and more get a stream of their own from the runtime
    buffer._runtime = SimpleNamespace(budget_stream=lambda cus: 1000 + cus if cus >= 64 else 0)
    monkeypatch.setattr(api.torch.cuda, "ExternalStream", FakeStream)
    buffer._comm_stream = FakeStream(11)
    buffer._budget_streams = {}
    buffer._active_stream = buffer._comm_stream
    buffer._backend = SimpleNamespace(dispatch=dispatch, combine=combine)
    buffer._allow_multiple_reduction = False
    return SimpleNamespace(buffer=buffer, calls=calls, tensor=FakeTensor,
                           indices=i64("indices", [[0, 1, -1], [-1, -1, 2]]))


@pytest.mark.parametrize(
    "layout,weighted,mode,asynchronous,explicit_event",
    [
        pytest.param(None, False, False, False, False, id="default-sync"),
        pytest.param(False, True, True, True, True, id="compact-async-weighted"),
        pytest.param(True, True, False, True, False, id="expanded-async-weighted"),
        pytest.param(True, False, True, False, True, id="expanded-sync-unweighted"),
    ],
)
def test_fresh_dispatch_arguments_and_handle(context, layout, weighted, mode, asynchronous, explicit_event):
    buffer = context.buffer
    buffer._allow_multiple_reduction = mode
    x = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    weights = context.tensor("weights", torch.ones((2, 3))) if weighted else None
    ready = SimpleNamespace(cuda_event=77) if explicit_event else None
    alignment = None if layout is None else 4
    result = buffer.dispatch(x, topk_idx=context.indices, weights=weights, do_expand=layout, alignment=alignment,
                             zero_padding=True, previous_event=ready, async_op=asynchronous)
    call = context.calls[0]
    expand = layout is True
    assert call.args == (buffer._runtime, x, context.indices, weights, 3, 5, 1 if alignment is None else 4, [], 0, mode, expand,
                         True, 256, 11, 77 if explicit_event else -1, asynchronous)
    handle = result.handle
    assert handle.owner is buffer and handle.config == buffer._config
    assert (handle.rank, handle.world_size, handle.x_dtype, handle.do_expand, handle.alignment, handle.num_sms) == (
        0, 1, torch.bfloat16, expand, call.args[6], 256)
    assert (handle.layout.recv_count, handle.layout.expanded_capacity) == (2, 3 * call.args[6])
    assert [handle.layout.recv_metadata, handle.layout.expert_counts, handle.layout.expert_offsets, handle.dst_slots,
            handle.send_counts, handle.topk_idx, handle.layout.recv_rank_prefix] == call.metadata[:7]
    assert handle.token_slots is (call.metadata[7] if expand else None)
    assert result.x is call.outputs[0]
    assert result.topk_idx is (None if expand else call.outputs[1])
    assert result.topk_weights is (call.outputs[2] if weighted else None)
    if asynchronous:
        assert result.event.event is call.completed
        assert any(item is handle for item in result.event.keepalive) and any(item is x for item in result.event.keepalive)
        result.event.current_stream_wait()
        assert call.completed.waits == 1
    else:
        assert result.event is None
    # the handle owns the snapshot returned by the backend, not the caller's tensor
    context.indices.payload.fill_(-1)
    assert handle.topk_idx.payload[0].tolist() == [0, 1, -1]


@pytest.mark.parametrize("expand,weighted,asynchronous", [(False, True, False), (True, False, True)])
def test_cached_dispatch_forwards_the_handle(context, expand, weighted, asynchronous):
    buffer = context.buffer
    x = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    weights = context.tensor("weights", torch.ones((2, 3)))
    first = buffer.dispatch(x, topk_idx=context.indices, weights=weights if weighted else None, do_expand=expand, alignment=4,
                            async_op=True, num_sms=24)
    old_metadata = context.calls[0].metadata
    new_x = context.tensor("new_x", torch.full((2, 256), 7.0, dtype=torch.bfloat16))
    new_weights = None if weighted else weights
    result = buffer.dispatch(new_x, weights=new_weights, handle=first.handle, async_op=asynchronous)
    call = context.calls[-1]
    assert result.handle is first.handle
    (_, got_x, routing, got_w, _, _, alignment, cached, capacity, _, got_expand, zero_padding, num_sms, _, _, got_async) = call.args
    assert routing is first.handle.topk_idx and got_x is new_x and got_w is new_weights
    assert cached == old_metadata and capacity == first.handle.layout.expanded_capacity
    assert alignment == 4 and got_expand is expand and zero_padding is False and got_async is asynchronous
    assert num_sms == 24  # the handle's saved budget is inherited


def test_a_compute_unit_budget_picks_the_stream_and_keeps_the_calls_in_order(context):
    """A call with a budget below the whole device is handed the runtime's stream for that budget
    (sync or async), the others the communication stream; a call whose stream differs from the
    previous call's is ordered behind it."""
    buffer = context.buffer
    x = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    streams = lambda: [call.args[13] if call.kind == "dispatch" else call.args[9] for call in context.calls]
    first = buffer.dispatch(x, topk_idx=context.indices, do_expand=True, num_sms=64, async_op=True)
    assert streams() == [1064] and buffer._budget_streams[64].waited_for == [11]
    buffer.dispatch(x, handle=first.handle)  # inherits the handle's budget
    assert streams() == [1064, 1064] and buffer._budget_streams[64].waited_for == [11]
    payload = context.tensor("y", torch.zeros((first.handle.layout.expanded_capacity, 256), dtype=torch.bfloat16))
    buffer.combine(payload, first.handle, num_sms=256)  # the whole device: the communication stream, behind the budget stream
    assert streams()[-1] == 11 and buffer._comm_stream.waited_for == [1064]
    buffer.combine(payload, first.handle, num_sms=128)
    assert streams()[-1] == 1128 and buffer._budget_streams[128].waited_for == [11]
    buffer.dispatch(x, topk_idx=context.indices, num_sms=24)  # the runtime has no stream for so few: the communication stream
    assert streams()[-1] == 11 and buffer._comm_stream.waited_for == [1064, 1128]
    assert buffer.budget_stream(64) is buffer._budget_streams[64]


def test_dispatch_argument_rules(context):
    buffer = context.buffer
    x = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="requires topk_idx"):
        buffer.dispatch(x)
    for bad in (0, -3, True, 2.0):
        with pytest.raises(ValueError, match="alignment"):
            buffer.dispatch(x, topk_idx=context.indices, alignment=bad)
    with pytest.raises(ValueError, match="do_expand"):
        buffer.dispatch(x, topk_idx=context.indices, do_expand="yes")
    with pytest.raises(ValueError, match="hidden"):
        buffer.dispatch(context.tensor("x", torch.zeros((2, 512), dtype=torch.bfloat16)), topk_idx=context.indices)
    with pytest.raises(ValueError, match="shape"):
        buffer.dispatch(context.tensor("x", torch.zeros((3, 256), dtype=torch.bfloat16)), topk_idx=context.indices)
    for bad in (-1, 257, True, 1.0, "4"):
        with pytest.raises(ValueError, match="num_sms"):
            buffer.dispatch(x, topk_idx=context.indices, num_sms=bad)
    assert buffer.dispatch(x, topk_idx=context.indices, num_sms=0).handle.num_sms == 256
    handle = buffer.dispatch(x, topk_idx=context.indices, do_expand=True, alignment=4).handle
    with pytest.raises(ValueError, match="omit topk_idx"):
        buffer.dispatch(x, topk_idx=context.indices, handle=handle)
    with pytest.raises(ValueError, match="alignment"):
        buffer.dispatch(x, handle=handle, alignment=8)
    with pytest.raises(ValueError, match="layout"):
        buffer.dispatch(x, handle=handle, do_expand=False)
    buffer.dispatch(x, handle=handle, alignment=4, do_expand=True)  # restating the handle's settings is allowed
    handle.owner = object()
    with pytest.raises(ValueError, match="another CudaBuffer"):
        buffer.dispatch(x, handle=handle)
    buffer._closed = True
    with pytest.raises(RuntimeError, match="closed"):
        buffer.dispatch(x, topk_idx=context.indices)


@pytest.mark.parametrize("expand,mode,weighted,biased,asynchronous,explicit_event", [
    (False, False, False, False, False, False),
    (False, True, True, True, True, True),
    (True, False, True, False, True, False),
    (True, True, False, True, False, True),
])
def test_combine_arguments(context, expand, mode, weighted, biased, asynchronous, explicit_event):
    buffer = context.buffer
    buffer._allow_multiple_reduction = mode
    x0 = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    handle = buffer.dispatch(x0, topk_idx=context.indices, do_expand=expand, alignment=4, num_sms=24).handle
    rows = 12 if expand else 2
    y = context.tensor("y", torch.zeros((rows, 256), dtype=torch.bfloat16))
    weights = context.tensor("w", torch.ones((rows,) if expand else (rows, 3))) if weighted else None
    bias = context.tensor("bias", torch.zeros((2, 256), dtype=torch.bfloat16)) if biased else None
    ready = SimpleNamespace(cuda_event=5) if explicit_event else None
    result = buffer.combine(y, handle, weights=weights, bias=bias, previous_event=ready, async_op=asynchronous)
    call = context.calls[-1]
    metadata = [handle.layout.recv_metadata, handle.layout.expert_counts, handle.layout.expert_offsets, handle.dst_slots,
                handle.send_counts, handle.topk_idx, handle.layout.recv_rank_prefix]
    if expand:
        metadata.append(handle.token_slots)
    assert call.args == (buffer._runtime, y, metadata, weights, bias, 5, expand, mode, 24, 11, 5 if explicit_event else -1,
                         asynchronous)
    assert result.x is call.outputs[0] and result.x.shape == (2, 256)
    assert result.topk_weights is (call.outputs[1] if weighted else None)
    if asynchronous:
        assert result.event.event is call.completed and any(item is handle for item in result.event.keepalive)
    else:
        assert result.event is None


def test_combine_argument_rules(context):
    buffer = context.buffer
    x0 = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    handle = buffer.dispatch(x0, topk_idx=context.indices, do_expand=True, alignment=4).handle
    good = context.tensor("y", torch.zeros((12, 256), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="bfloat16"):
        buffer.combine(context.tensor("y", torch.zeros((12, 256), dtype=torch.float32)), handle)
    with pytest.raises(ValueError, match="exact receive shape"):
        buffer.combine(context.tensor("y", torch.zeros((11, 256), dtype=torch.bfloat16)), handle)
    with pytest.raises(ValueError, match="weights"):
        buffer.combine(good, handle, weights=context.tensor("w", torch.ones((12, 3))))
    with pytest.raises(ValueError, match="bias"):
        buffer.combine(good, handle, bias=context.tensor("b", torch.zeros((3, 256), dtype=torch.bfloat16)))
    other = api.CudaBuffer.__new__(api.CudaBuffer)
    other.__dict__.update(buffer.__dict__)
    with pytest.raises(ValueError, match="another CudaBuffer"):
        other.combine(good, handle)
    handle.config = EPConfig(6, 3, 256, 5)
    with pytest.raises(ValueError, match="configuration"):
        buffer.combine(good, handle)
    buffer._closed = True
    with pytest.raises(RuntimeError, match="closed"):
        buffer.combine(good, handle)


def test_config_validation():
    assert ConfigAlias is EPConfig
    config = EPConfig(num_experts=256, num_topk=8, hidden=7168, num_max_tokens_per_rank=4096)
    assert (config.num_experts, config.num_topk, config.hidden, config.num_max_tokens_per_rank) == (256, 8, 7168, 4096)
    with pytest.raises(Exception):
        config.hidden = 1  # frozen
    for bad in ((0, 1, 256, 1), (4, 0, 256, 1), (4, 2, 0, 1), (4, 2, 256, 0), (4, 5, 256, 1), (64, 33, 256, 1)):
        with pytest.raises(ValueError):
            EPConfig(*bad)
    EPConfig(64, 32, 256, 1)


def test_deterministic_fill_refusal(context, monkeypatch):
    monkeypatch.setattr(api.torch, "are_deterministic_algorithms_enabled", lambda: True)
    monkeypatch.setattr(api.deterministic, "fill_uninitialized_memory", True)
    x = context.tensor("x", torch.zeros((2, 256), dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="fill_uninitialized_memory"):
        context.buffer.dispatch(x, topk_idx=context.indices)


def test_construction_checks_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("covers the no-GPU error path")
    with pytest.raises(TypeError):
        api.CudaBuffer(None, EPConfig(2, 2, 256, 4), allow_multiple_reduction="no")
    with pytest.raises(RuntimeError, match="no GPU"):
        api.CudaBuffer(None, EPConfig(2, 2, 256, 4))


def test_control_group_inspection_with_a_real_gloo_group():
    """The group argument of the reference's Buffer is a Gloo control group; with one rank its
    single-member form is accepted and anything else refused (no GPU needed for this part)."""
    import torch.distributed as dist

    assert api.CudaBuffer._inspect_group(None) == (0, 1)
    assert not dist.is_initialized()
    dist.init_process_group("gloo", store=dist.HashStore(), rank=0, world_size=1)
    try:
        assert api.CudaBuffer._inspect_group(dist.group.WORLD) == (0, 1)
        assert api.CudaBuffer._inspect_group(dist.new_group(ranks=[0], backend="gloo")) == (0, 1)
    finally:
        dist.destroy_process_group()

    class FakeDist:
        def __init__(self, backend, size):
            self.backend, self.size = backend, size

    import unittest.mock as mock

    for backend, size, message in (("nccl", 1, "Gloo"), ("gloo", 2, "world_size == 1")):
        with mock.patch.object(dist, "get_backend", lambda group, b=backend: b), \
                mock.patch.object(dist, "get_world_size", lambda group=None, n=size: n):
            with pytest.raises(ValueError, match=message):
                api.CudaBuffer._inspect_group(object())


def test_reference_import_paths():
    """`nano_ep`, `nano_ep.backends` and `nano_ep.backends.cuda` export these names (nano_ep/__init__.py,
    nano_ep/backends/__init__.py); the same import paths exist here and name the same objects."""
    import nanoep_amd
    from nanoep_amd import backends
    from nanoep_amd.backends import cuda

    for name in ("CudaBuffer", "CudaEvent", "NativeCombineResult", "NativeDispatchResult", "NativeHandle", "NativeLayout"):
        assert getattr(backends, name) is getattr(nanoep_amd, name) is getattr(cuda, name)
    assert nanoep_amd.EPConfig is not None and nanoep_amd.__version__
    assert callable(cuda.check_torch_deterministic)


def test_the_benchmark_refuses_more_than_one_gpu():
    """bench.py measures one rank on one GPU; any other --gpus ends at once with a message and a
    non-zero status, before anything touches a device."""
    import pathlib
    import subprocess
    import sys

    bench = pathlib.Path(__file__).resolve().parents[1] / "bench.py"
    done = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0
    assert "ONE GPU" in done.stderr + done.stdout
    assert not any(line.startswith("{") for line in done.stdout.splitlines())
