"""Single-GPU (world_size == 1) expert-parallel dispatch and combine for PyTorch-ROCm on MI355X."""

from .buffer import (
    Buffer,
    CudaBuffer,
    CudaEvent,
    NativeCombineResult,
    NativeDispatchResult,
    NativeHandle,
    NativeLayout,
)
from .config import EPConfig

__version__ = "0.1.0"

__all__ = [
    "Buffer",
    "CudaBuffer",
    "CudaEvent",
    "EPConfig",
    "NativeCombineResult",
    "NativeDispatchResult",
    "NativeHandle",
    "NativeLayout",
]
