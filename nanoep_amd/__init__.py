"""nanoep_amd: expert-parallel dispatch / combine for one rank on one MI355X (PyTorch-ROCm).

The public names are those of the reference package `nano_ep`, so `from nanoep_amd import
CudaBuffer, EPConfig` is the only line a caller changes; `Buffer` is a shorter alias.
"""

from . import buffer as _buffer
from . import handles as _handles
from .config import EPConfig

__version__ = "0.1.0"

CudaBuffer = _buffer.CudaBuffer
Buffer = _buffer.Buffer
CudaEvent = _handles.CudaEvent
NativeLayout = _handles.NativeLayout
NativeHandle = _handles.NativeHandle
NativeDispatchResult = _handles.NativeDispatchResult
NativeCombineResult = _handles.NativeCombineResult

__all__ = sorted(
    ["Buffer", "CudaBuffer", "CudaEvent", "EPConfig", "NativeLayout", "NativeHandle", "NativeDispatchResult", "NativeCombineResult"]
)
