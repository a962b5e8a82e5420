"""Import path of the reference (`nano_ep.backends.cuda`, nano_ep/backends/cuda.py): the same names,
served by `nanoep_amd.buffer`."""

from ..buffer import (  # noqa: F401
    CudaBuffer,
    CudaEvent,
    NativeCombineResult,
    NativeDispatchResult,
    NativeHandle,
    NativeLayout,
    check_torch_deterministic,
)
