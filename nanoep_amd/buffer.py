"""Python surface of the dispatch / combine buffer for one rank on one MI355X.

Keeps the reference's public API (nano_ep/backends/cuda.py:23-444): the result and handle
dataclasses, `CudaBuffer(group, config, *, allow_multiple_reduction)`, `dispatch`, `combine`,
`close`, and `CudaEvent.current_stream_wait()`, with the same keyword arguments, validation order
and exception types, so code written against `nano_ep` runs on PyTorch-ROCm with world_size == 1.
Everything below the `self._backend.dispatch / combine` calls is the native extension.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
from torch.utils import deterministic

from ._native import load_extension
from .config import EPConfig


def check_torch_deterministic():
    """Same refusal as the reference (nano_ep/backends/cuda.py:16-20)."""
    if torch.are_deterministic_algorithms_enabled() and deterministic.fill_uninitialized_memory:
        raise RuntimeError(
            "NanoEP does not support deterministic algorithms with fill_uninitialized_memory enabled; "
            "disable one of these PyTorch settings"
        )


@dataclass
class NativeLayout:
    recv_metadata: torch.Tensor  # int32 [N, K+2]: src_rank, src_token, K x (local expert id | expanded slot | -1)
    expert_counts: torch.Tensor  # int64 [L]
    expert_offsets: torch.Tensor  # int64 [L+1], padded exclusive offsets ending at C
    recv_rank_prefix: torch.Tensor  # int64 [R]
    recv_count: int  # N
    expanded_capacity: int  # C


@dataclass
class NativeHandle:
    config: EPConfig
    rank: int
    world_size: int
    do_expand: bool
    alignment: int
    topk_idx: torch.Tensor  # int64 [T, K] routing snapshot
    layout: NativeLayout
    dst_slots: torch.Tensor  # int64 [T, R]
    send_counts: torch.Tensor  # int64 [R]
    owner: object
    x_dtype: torch.dtype
    num_sms: int | None = None
    # int32 [T, K] slot of every (token, k), -1 when masked: the same mapping as dst_slots +
    # recv_metadata in one lookup.  Only expanded handles made by this package carry it.
    token_slots: torch.Tensor | None = None
    # int64 list of every valid assignment as (slot << 32) | (t * K + k), one segment per block of
    # consecutive tokens, ascending slot inside a segment, -1 in unused entries: the order in which
    # a replayed dispatch walks its work.  Only expanded handles made by this package carry it.
    slot_order: torch.Tensor | None = None


@dataclass
class NativeDispatchResult:
    x: torch.Tensor
    topk_idx: torch.Tensor | None
    topk_weights: torch.Tensor | None
    handle: NativeHandle
    event: "CudaEvent | None"


@dataclass
class NativeCombineResult:
    x: torch.Tensor
    topk_weights: torch.Tensor | None
    event: "CudaEvent | None"


class CudaEvent:
    def __init__(self, event, keepalive: tuple = ()):
        self.event = event
        self.keepalive = keepalive

    def current_stream_wait(self):
        """Wait on the consumer stream and protect tensors used on that stream."""
        self.event.current_stream_wait()


def _handle_metadata(handle: NativeHandle) -> list[torch.Tensor]:
    layout = handle.layout
    metadata = [
        layout.recv_metadata,
        layout.expert_counts,
        layout.expert_offsets,
        handle.dst_slots,
        handle.send_counts,
        handle.topk_idx,
        layout.recv_rank_prefix,
    ]
    if getattr(handle, "token_slots", None) is not None:
        metadata.append(handle.token_slots)
        if getattr(handle, "slot_order", None) is not None:
            metadata.append(handle.slot_order)
    return metadata


class CudaBuffer:
    def __init__(self, group, config: EPConfig, *, allow_multiple_reduction: bool = False):
        """Create the buffer and its communication stream.

        `group` is None or a torch.distributed Gloo group of size 1: this build runs one rank on
        one GPU, so the reference's collective bootstrap (nano_ep/backends/cuda.py:90-231) reduces
        to local checks.
        """
        self._group = group
        self._config = config
        self._allow_multiple_reduction = allow_multiple_reduction
        self._world_size = 1
        self._rank = 0
        self._runtime = None
        self._comm_stream = None
        self._closed = True
        if group is not None:
            import torch.distributed as dist

            if dist.get_backend(group) != "gloo":
                raise ValueError("CudaBuffer requires a Gloo control group")
            if dist.get_world_size(group=group) != 1:
                raise ValueError("this build runs one rank on one GPU: the control group must have world_size == 1")
            self._rank = dist.get_rank(group=group)
        if not isinstance(allow_multiple_reduction, bool):
            raise TypeError("allow_multiple_reduction must be bool")
        if not torch.cuda.is_available():
            raise RuntimeError("CudaBuffer environment check failed: no GPU is visible to PyTorch-ROCm")
        if config.num_experts % self._world_size != 0:
            raise ValueError("num_experts must be divisible by world_size")
        if config.hidden % 256 != 0:
            raise ValueError("CUDA EP hidden must be a positive multiple of 256")

        self._device = torch.cuda.current_device()
        properties = torch.cuda.get_device_properties(self._device)
        self._device_sms = properties.multi_processor_count
        self._gpu_uuids = (str(getattr(properties, "uuid", self._device)),)
        self._auto_num_sms = None

        self._backend = load_extension()
        (
            self._signal_offset,
            self._count_offset,
            self._payload_offset,
            self._return_offset,
            self._num_bytes,
        ) = self._backend.window_layout(
            self._world_size,
            config.num_max_tokens_per_rank,
            config.hidden,
            config.num_topk,
            config.num_experts,
            allow_multiple_reduction,
        )
        # No peer window is allocated: with one rank, rows go straight from the source tensor to
        # the exact-shaped outputs.  The runtime owns the device id and the host count mailbox.
        self._runtime = self._backend.PeerRuntime(self._rank, self._world_size, self._num_bytes)
        self._handle = self._runtime.export_local_handle()
        self._runtime.import_peer_handles([self._handle])
        self._comm_stream = torch.cuda.Stream(device=self._device)
        self._closed = False

    def _resolve_num_sms(self, num_sms: int | None, handle: NativeHandle | None) -> int:
        if num_sms is None:
            return self._device_sms if handle is None or handle.num_sms is None else handle.num_sms
        if isinstance(num_sms, bool) or not isinstance(num_sms, int) or not 0 <= num_sms <= self._device_sms:
            raise ValueError(f"num_sms must be an integer between 0 and {self._device_sms}")
        if num_sms > 0:
            return num_sms
        if self._auto_num_sms is None:
            # The reference's link-bandwidth model returns the whole device when there are no peers
            # (nano_ep/backends/_sms.py:50-51).
            self._auto_num_sms = self._device_sms
        return self._auto_num_sms

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
        "Dispatch payloads using fresh or cached routing; return exact receive layouts."
        check_torch_deterministic()
        if self._closed:
            raise RuntimeError("CudaBuffer is closed")
        if handle is not None:
            if handle.owner is not self:
                raise ValueError("cached handle belongs to another CudaBuffer")
            if topk_idx is not None:
                raise ValueError("cached dispatch uses the handle snapshot; omit topk_idx")
            if alignment is not None and alignment != handle.alignment:
                raise ValueError("cached dispatch must retain the handle alignment")
            if do_expand is not None and do_expand != handle.do_expand:
                raise ValueError("cached dispatch must retain the handle layout")
        elif topk_idx is None:
            raise ValueError("fresh dispatch requires topk_idx")
        if alignment is not None and (isinstance(alignment, bool) or not isinstance(alignment, int) or alignment <= 0):
            raise ValueError("alignment must be a positive integer")
        if do_expand is not None and not isinstance(do_expand, bool):
            raise ValueError("do_expand must be bool or None")

        routing = handle.topk_idx if handle is not None else topk_idx
        if x.shape[1] != self._config.hidden:
            raise ValueError("x hidden dimension does not match the buffer configuration")
        if routing.shape != (x.shape[0], self._config.num_topk):
            raise ValueError("routing snapshot/topk_idx shape must match the buffer configuration")

        if handle is None:
            expand = False if do_expand is None else do_expand
            expert_alignment = 1 if alignment is None else alignment
            cached_metadata = []
            cached_expanded_capacity = 0
        else:
            expand = handle.do_expand
            expert_alignment = handle.alignment
            cached_expanded_capacity = handle.layout.expanded_capacity
            cached_metadata = _handle_metadata(handle)

        main_sms = self._resolve_num_sms(num_sms, handle)
        outputs, metadata, counts, completed = self._backend.dispatch(
            self._runtime,
            x,
            routing,
            weights,
            self._config.num_experts,
            self._config.num_max_tokens_per_rank,
            expert_alignment,
            cached_metadata,
            cached_expanded_capacity,
            self._allow_multiple_reduction,
            expand,
            zero_padding,
            main_sms,
            self._comm_stream.cuda_stream,
            -1 if previous_event is None else previous_event.cuda_event,
            async_op,
        )
        recv_count, expanded_capacity = counts

        if handle is None:
            layout = NativeLayout(
                recv_metadata=metadata[0],
                expert_counts=metadata[1],
                expert_offsets=metadata[2],
                recv_rank_prefix=metadata[6],
                recv_count=recv_count,
                expanded_capacity=expanded_capacity,
            )
            handle = NativeHandle(
                config=self._config,
                rank=self._rank,
                world_size=self._world_size,
                do_expand=expand,
                alignment=expert_alignment,
                topk_idx=metadata[5],
                layout=layout,
                dst_slots=metadata[3],
                send_counts=metadata[4],
                owner=self,
                x_dtype=x.dtype,
                num_sms=main_sms,
                token_slots=metadata[7] if len(metadata) > 7 else None,
                slot_order=metadata[8] if len(metadata) > 8 else None,
            )

        event = CudaEvent(completed, keepalive=(self, x, routing, weights, handle)) if async_op else None

        return NativeDispatchResult(
            x=outputs[0],
            topk_idx=None if expand else outputs[1],
            topk_weights=outputs[2] if weights is not None else None,
            handle=handle,
            event=event,
        )

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
        "Return expert outputs to their source and reduce in FP32, without gate weighting."
        check_torch_deterministic()
        if self._closed:
            raise RuntimeError("CudaBuffer is closed")
        if handle.owner is not self:
            raise ValueError("combine handle belongs to another CudaBuffer")
        if handle.config != self._config:
            raise ValueError("combine handle configuration does not match this CudaBuffer")

        device = torch.device("cuda", self._device)
        layout = handle.layout
        rows = layout.expanded_capacity if handle.do_expand else layout.recv_count
        hidden = self._config.hidden
        if x.device != device or x.dtype != torch.bfloat16 or x.shape != (rows, hidden) or not x.is_contiguous():
            raise ValueError("combine x must be contiguous CUDA bfloat16 with the handle's exact receive shape")
        weight_shape = (rows,) if handle.do_expand else (rows, self._config.num_topk)
        if weights is not None and (
            weights.device != device or weights.dtype != torch.float32 or weights.shape != weight_shape or not weights.is_contiguous()
        ):
            raise ValueError("combine weights must be contiguous CUDA float32 with the handle's receive layout")
        source_tokens = handle.topk_idx.shape[0]
        if bias is not None and (
            bias.device != device or bias.dtype != x.dtype or bias.shape != (source_tokens, hidden) or not bias.is_contiguous()
        ):
            raise ValueError("combine bias must be contiguous source [T,H], with the x dtype on this buffer's device")

        metadata = _handle_metadata(handle)
        main_sms = self._resolve_num_sms(num_sms, handle)
        with torch.cuda.device(self._device):
            outputs, completed = self._backend.combine(
                self._runtime,
                x,
                metadata,
                weights,
                bias,
                self._config.num_max_tokens_per_rank,
                handle.do_expand,
                self._allow_multiple_reduction,
                main_sms,
                self._comm_stream.cuda_stream,
                -1 if previous_event is None else previous_event.cuda_event,
                async_op,
            )

            event = CudaEvent(completed, keepalive=(self, x, handle, weights, bias)) if async_op else None

        return NativeCombineResult(x=outputs[0], topk_weights=outputs[1] if weights is not None else None, event=event)

    @property
    def comm_stream(self) -> torch.cuda.Stream:
        """The stream dispatch and combine kernels are launched on."""
        return self._comm_stream

    def close(self):
        """Drain the GPU and release the runtime.  Idempotent; dispatch/combine fail afterwards."""
        if self._closed:
            return
        torch.cuda.synchronize(self._device)
        self._runtime.close_peer_mappings()
        self._runtime.close()
        self._closed = True

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()


Buffer = CudaBuffer
