"""Import path of the reference (`nano_ep.backends`): the same names, served by `nanoep_amd.buffer`."""

from ..buffer import CudaBuffer, CudaEvent, NativeCombineResult, NativeDispatchResult, NativeHandle, NativeLayout

__all__ = ["CudaBuffer", "CudaEvent", "NativeCombineResult", "NativeDispatchResult", "NativeHandle", "NativeLayout"]
