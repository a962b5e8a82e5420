"""The buffer object: `CudaBuffer.dispatch` / `.combine` / `.close` for one rank on one MI355X.

The call surface is the reference's (`CudaBuffer` in nano_ep/backends/cuda.py:90-444): the same
keyword arguments, the same order of argument checks, `ValueError` for misuse of arguments and
handles, `RuntimeError` for a closed buffer and for the deterministic-fill conflict, `TypeError`
for a non-bool `allow_multiple_reduction`.  What differs is underneath: there is no peer window,
no collective bootstrap and no JIT; every call ends in one native call of `_nanoep_torch`.
"""

from __future__ import annotations

import torch
from torch.utils import deterministic

from ._native import load_extension
from .config import EPConfig
from .handles import CudaEvent, NativeCombineResult, NativeDispatchResult, NativeHandle, NativeLayout

__all__ = [
    "Buffer",
    "CudaBuffer",
    "CudaEvent",
    "NativeCombineResult",
    "NativeDispatchResult",
    "NativeHandle",
    "NativeLayout",
    "check_torch_deterministic",
]

# The reference's row-width contract (nano_ep/backends/cuda.py:104-105); the kernels need H % 8.
HIDDEN_MULTIPLE = 256


def check_torch_deterministic():
    """Deterministic mode fills every new tensor; the outputs here are allocated uninitialised and
    written exactly once by the kernels, so the combination is refused as the reference refuses it
    (nano_ep/backends/cuda.py:16-20)."""
    filling = torch.are_deterministic_algorithms_enabled() and deterministic.fill_uninitialized_memory
    if filling:
        raise RuntimeError(
            "NanoEP does not support deterministic algorithms with fill_uninitialized_memory enabled; "
            "disable one of these PyTorch settings"
        )


def _plain_int(value) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


def _raw_event(previous_event) -> int:
    """Raw event handle for the native call, -1 for none."""
    return previous_event.cuda_event if previous_event is not None else -1


def _handle_metadata(handle: NativeHandle) -> list[torch.Tensor]:
    return NativeHandle.tensors(handle)


class CudaBuffer:
    """One rank's dispatch / combine endpoint.  `Buffer` is the same class."""

    def __init__(self, group, config: EPConfig, *, allow_multiple_reduction: bool = False):
        """`group` is None or a torch.distributed Gloo group with a single member: with one rank
        the reference's collective bootstrap (nano_ep/backends/cuda.py:90-231) comes down to the
        local checks below."""
        self._closed = True  # until everything below has succeeded
        self._runtime = self._comm_stream = None
        self._group, self._config = group, config
        self._allow_multiple_reduction = allow_multiple_reduction
        self._rank, self._world_size = self._inspect_group(group)

        if not isinstance(allow_multiple_reduction, bool):
            raise TypeError("allow_multiple_reduction must be bool")
        if not torch.cuda.is_available():
            raise RuntimeError("CudaBuffer environment check failed: no GPU is visible to PyTorch-ROCm")
        if config.num_experts % self._world_size:
            raise ValueError("num_experts must be divisible by world_size")
        if config.hidden % HIDDEN_MULTIPLE:
            raise ValueError(f"CUDA EP hidden must be a positive multiple of {HIDDEN_MULTIPLE}")

        self._device = torch.cuda.current_device()
        card = torch.cuda.get_device_properties(self._device)
        self._device_sms = card.multi_processor_count
        self._gpu_uuids = (str(getattr(card, "uuid", self._device)),)
        self._auto_num_sms = None

        self._backend = load_extension()
        # The window geometry is computed for callers that ask for it; no window is allocated,
        # since with one rank rows go straight from the source tensor to the exact-shaped outputs.
        offsets = self._backend.window_layout(
            self._world_size, config.num_max_tokens_per_rank, config.hidden, config.num_topk, config.num_experts,
            allow_multiple_reduction,
        )
        self._signal_offset, self._count_offset, self._payload_offset, self._return_offset, self._num_bytes = offsets
        # The runtime owns the device id and the pinned mailbox the layout kernels report N and C in.
        self._runtime = self._backend.PeerRuntime(self._rank, self._world_size, self._num_bytes)
        self._handle = self._runtime.export_local_handle()
        self._runtime.import_peer_handles([self._handle])
        self._comm_stream = torch.cuda.Stream(device=self._device)
        # Calls with a compute-unit budget below the whole device run on a stream of the runtime's whose
        # kernels are confined to that many CUs (see _stream_for); `_active_stream` is the stream the
        # latest call ran on, which the next call's stream is ordered behind.
        self._budget_streams: dict[int, torch.cuda.Stream] = {}
        self._active_stream = self._comm_stream
        self._closed = False

    @staticmethod
    def _inspect_group(group) -> tuple[int, int]:
        """(rank, world_size) of the control group; only a single-member Gloo group is accepted."""
        if group is None:
            return 0, 1
        import torch.distributed as dist

        if dist.get_backend(group) != "gloo":
            raise ValueError("CudaBuffer requires a Gloo control group")
        if dist.get_world_size(group=group) != 1:
            raise ValueError("this build runs one rank on one GPU: the control group must have world_size == 1")
        return dist.get_rank(group=group), 1

    # ------------------------------------------------------------------ shared argument handling

    def _require_open(self) -> None:
        if self._closed:
            raise RuntimeError("CudaBuffer is closed")

    def _resolve_num_sms(self, num_sms, handle) -> int:
        """The compute-unit budget of a call: an explicit number, else the handle's, else the whole
        device.  0 asks for the automatic choice, which without peers is the whole device as well
        (nano_ep/backends/_sms.py:50-51)."""
        whole = self._device_sms
        if num_sms is None:
            inherited = None if handle is None else handle.num_sms
            return whole if inherited is None else inherited
        if not _plain_int(num_sms) or num_sms < 0 or num_sms > whole:
            raise ValueError(f"num_sms must be an integer between 0 and {whole}")
        if num_sms:
            return num_sms
        if self._auto_num_sms is None:
            self._auto_num_sms = whole
        return self._auto_num_sms

    def _stream_for(self, budget: int) -> torch.cuda.Stream:
        """The stream a call with this compute-unit budget is handed.  The whole device: the buffer's
        communication stream.  Less: a stream created with a CU mask of about `budget` compute units,
        the same number on every XCD (the MI355X-native form of the reference's SM budget,
        nano_ep/backends/cuda.py:233-244, csrc/pipeline.cu:20-24); such a call runs there whether it is
        asynchronous or not.  All of a buffer's calls stay ordered one behind the other: a call whose
        stream differs from the previous call's waits for it."""
        stream = self._comm_stream
        if 0 < budget < self._device_sms:
            stream = self._budget_streams.get(budget)
            if stream is None:
                raw = self._runtime.budget_stream(budget)
                stream = torch.cuda.ExternalStream(raw, device=self._device) if raw else self._comm_stream
                self._budget_streams[budget] = stream
        if stream is not self._active_stream:
            stream.wait_stream(self._active_stream)
            self._active_stream = stream
        return stream

    # ------------------------------------------------------------------ dispatch

    def dispatch(
        self,
        x: torch.Tensor,
        *,
        topk_idx: torch.Tensor | None = None,
        weights: torch.Tensor | None = None,
        handle: NativeHandle | None = None,
        do_expand: bool | None = None,
        alignment: int | None = None,
        zero_padding: bool = False,
        previous_event: torch.cuda.Event | None = None,
        async_op: bool = False,
        num_sms: int | None = None,
    ) -> NativeDispatchResult:
        """Send token rows to their experts' receive layout.

        Fresh: pass `topk_idx` (int64 [T, K], ids or -1); the result carries a handle.  Cached:
        pass that `handle` instead; its routing snapshot, layout and alignment are reused and only
        the payload (and weights) are new.  `do_expand=True` gives one row per (token, choice) in
        expert-major slots padded to `alignment`, otherwise one row per received token.
        """
        check_torch_deterministic()
        self._require_open()
        replay = handle is not None
        if replay:
            self._check_replay_arguments(handle, topk_idx, alignment, do_expand)
        elif topk_idx is None:
            raise ValueError("fresh dispatch requires topk_idx")
        if alignment is not None and not (_plain_int(alignment) and alignment > 0):
            raise ValueError("alignment must be a positive integer")
        if not (do_expand is None or isinstance(do_expand, bool)):
            raise ValueError("do_expand must be bool or None")

        geometry = self._config
        routing = handle.topk_idx if replay else topk_idx
        if x.shape[1] != geometry.hidden:
            raise ValueError("x hidden dimension does not match the buffer configuration")
        if tuple(routing.shape) != (x.shape[0], geometry.num_topk):
            raise ValueError("routing snapshot/topk_idx shape must match the buffer configuration")

        if replay:
            expand, slot_alignment = handle.do_expand, handle.alignment
            known_tensors, known_capacity = _handle_metadata(handle), handle.layout.expanded_capacity
        else:
            expand, slot_alignment = bool(do_expand), (alignment or 1)
            known_tensors, known_capacity = [], 0

        budget = self._resolve_num_sms(num_sms, handle)
        outputs, metadata, (received, capacity), completed = self._backend.dispatch(
            self._runtime, x, routing, weights,
            geometry.num_experts, geometry.num_max_tokens_per_rank, slot_alignment,
            known_tensors, known_capacity,
            self._allow_multiple_reduction, expand, zero_padding, budget,
            self._stream_for(budget).cuda_stream, _raw_event(previous_event), async_op,
        )
        if not replay:
            handle = self._new_handle(metadata, received, capacity, expand, slot_alignment, x.dtype, budget)

        payload, local_ids, gate = outputs
        return NativeDispatchResult(
            x=payload,
            topk_idx=None if expand else local_ids,
            topk_weights=None if weights is None else gate,
            handle=handle,
            event=CudaEvent(completed, keepalive=(self, x, routing, weights, handle)) if async_op else None,
        )

    def _check_replay_arguments(self, handle, topk_idx, alignment, do_expand) -> None:
        if handle.owner is not self:
            raise ValueError("cached handle belongs to another CudaBuffer")
        if topk_idx is not None:
            raise ValueError("cached dispatch uses the handle snapshot; omit topk_idx")
        if alignment is not None and alignment != handle.alignment:
            raise ValueError("cached dispatch must retain the handle alignment")
        if do_expand is not None and do_expand != handle.do_expand:
            raise ValueError("cached dispatch must retain the handle layout")

    def _new_handle(self, metadata, received, capacity, expand, slot_alignment, dtype, budget) -> NativeHandle:
        """Wrap what a fresh native dispatch returned: seven tensors in the reference's order
        (nano_ep/backends/cuda.py:328-345), then the private slot table and slot-order list."""
        recv_metadata, counts, offsets, dst_slots, send_counts, snapshot, prefix = metadata[:7]
        private = list(metadata[7:9]) + [None, None]
        return NativeHandle(
            config=self._config,
            rank=self._rank,
            world_size=self._world_size,
            do_expand=expand,
            alignment=slot_alignment,
            topk_idx=snapshot,
            layout=NativeLayout(
                recv_metadata=recv_metadata,
                expert_counts=counts,
                expert_offsets=offsets,
                recv_rank_prefix=prefix,
                recv_count=received,
                expanded_capacity=capacity,
            ),
            dst_slots=dst_slots,
            send_counts=send_counts,
            owner=self,
            x_dtype=dtype,
            num_sms=budget,
            token_slots=private[0],
            slot_order=private[1],
        )

    # ------------------------------------------------------------------ combine

    def combine(
        self,
        x: torch.Tensor,
        handle: NativeHandle,
        *,
        weights: torch.Tensor | None = None,
        bias: torch.Tensor | None = None,
        previous_event: torch.cuda.Event | None = None,
        async_op: bool = False,
        num_sms: int | None = None,
    ) -> NativeCombineResult:
        """Bring expert outputs back to their source tokens: per token the fp32 sum of its valid
        rows in ascending choice order (plus `bias`), rounded to bf16 once.  Gate weights are not
        applied; when given they are returned at their original (token, choice) positions."""
        check_torch_deterministic()
        self._require_open()
        if handle.owner is not self:
            raise ValueError("combine handle belongs to another CudaBuffer")
        if handle.config != self._config:
            raise ValueError("combine handle configuration does not match this CudaBuffer")

        here = torch.device("cuda", self._device)
        hidden, topk = self._config.hidden, self._config.num_topk
        expand = handle.do_expand
        rows = handle.layout.expanded_capacity if expand else handle.layout.recv_count

        def fits(tensor, dtype, shape) -> bool:
            return tensor.device == here and tensor.dtype == dtype and tuple(tensor.shape) == shape and tensor.is_contiguous()

        if not fits(x, torch.bfloat16, (rows, hidden)):
            raise ValueError("combine x must be contiguous CUDA bfloat16 with the handle's exact receive shape")
        if weights is not None and not fits(weights, torch.float32, (rows,) if expand else (rows, topk)):
            raise ValueError("combine weights must be contiguous CUDA float32 with the handle's receive layout")
        if bias is not None and not fits(bias, x.dtype, (handle.topk_idx.shape[0], hidden)):
            raise ValueError("combine bias must be contiguous source [T,H], with the x dtype on this buffer's device")

        metadata = _handle_metadata(handle)
        budget = self._resolve_num_sms(num_sms, handle)
        with torch.cuda.device(self._device):
            (combined, restored), completed = self._backend.combine(
                self._runtime, x, metadata, weights, bias,
                self._config.num_max_tokens_per_rank, expand, self._allow_multiple_reduction, budget,
                self._stream_for(budget).cuda_stream, _raw_event(previous_event), async_op,
            )
            event = CudaEvent(completed, keepalive=(self, x, handle, weights, bias)) if async_op else None
        return NativeCombineResult(x=combined, topk_weights=None if weights is None else restored, event=event)

    # ------------------------------------------------------------------ lifetime

    @property
    def comm_stream(self) -> torch.cuda.Stream:
        """The stream asynchronous dispatch and combine kernels are launched on (calls with a
        compute-unit budget below the whole device: `budget_stream`)."""
        return self._comm_stream

    def budget_stream(self, num_sms: int) -> torch.cuda.Stream:
        """The stream calls with this compute-unit budget run on."""
        self._require_open()
        return self._stream_for(self._resolve_num_sms(num_sms, None))

    def close(self):
        """Drain the GPU and release the runtime.  A second call does nothing; dispatch and combine
        raise afterwards."""
        if self._closed:
            return
        torch.cuda.synchronize(self._device)
        self._budget_streams.clear()
        self._active_stream = self._comm_stream
        self._runtime.close_peer_mappings()
        self._runtime.close()
        self._closed = True

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()


Buffer = CudaBuffer
