"""Loader of the prebuilt in-tree host extension.

Nothing is compiled here: `python -m nanoep_amd.build` (or __graft_entry__.build()) produces
nanoep_amd/libnanoep_hip.so and nanoep_amd/_nanoep_torch.so ahead of time, and a missing library is
an error, never a reason to fall back to another implementation.  Takes the place of the
reference's load_extension() (nano_ep/backends/_build.py:24-48).
"""

from __future__ import annotations

import importlib
from pathlib import Path

PACKAGE = Path(__file__).resolve().parent
_REQUIRED = ("libnanoep_hip.so", "_nanoep_torch.so")

_module = None


def load_extension():
    """Return the native module exporting dispatch, combine, window_layout, PeerRuntime, CompletionEvent."""
    global _module
    if _module is None:
        missing = [name for name in _REQUIRED if not (PACKAGE / name).exists()]
        if missing:
            raise RuntimeError(
                f"nanoep_amd native libraries are not built ({', '.join(missing)} missing in {PACKAGE}); "
                "run `python -m nanoep_amd.build`"
            )
        import torch  # noqa: F401  (libtorch must be loaded before the extension)

        _module = importlib.import_module("nanoep_amd._nanoep_torch")
    return _module
