"""`nanoep_amd.backends`: the import path callers of the reference use for its buffer classes
(`nano_ep.backends`).  Nothing lives here; the names come from `nanoep_amd.buffer` and
`nanoep_amd.handles`, and importing them compiles nothing."""

import nanoep_amd as _package

_NAMES = ("CudaBuffer", "CudaEvent", "NativeCombineResult", "NativeDispatchResult", "NativeHandle", "NativeLayout")
globals().update({name: getattr(_package, name) for name in _NAMES})
__all__ = list(_NAMES)
