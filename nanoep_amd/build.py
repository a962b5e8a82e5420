"""Ahead-of-time build of the two in-tree shared libraries (`python -m nanoep_amd.build`).

  libnanoep_hip.so   hand-written HIP kernels + the C ABI of include/nanoep_hip.h  (hipcc, gfx950)
  _nanoep_torch*.so  the PyTorch-ROCm host extension (g++), linked against the first

This replaces the reference's load_extension() + DeepJIT path (nano_ep/backends/_build.py:24-48):
nothing is compiled at import or call time.
"""

from __future__ import annotations

import os
import shlex
import subprocess
import sys
import sysconfig
from pathlib import Path

PACKAGE = Path(__file__).resolve().parent
ROOT = PACKAGE.parent
CSRC = PACKAGE / "csrc"
INCLUDE = ROOT / "include"

KERNEL_LIBRARY = PACKAGE / "libnanoep_hip.so"
EXTENSION_NAME = "_nanoep_torch"
EXTENSION_LIBRARY = PACKAGE / f"{EXTENSION_NAME}.so"

KERNEL_SOURCES = ["nanoep_layout.hip", "nanoep_dispatch.hip", "nanoep_combine.hip", "nanoep_abi.hip"]

OFFLOAD_ARCH = "gfx950"
# Packed fp32 instructions are disabled for every HIP translation unit of this project.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _run(command: list[str], verbose: bool) -> None:
    if verbose:
        print("+", " ".join(shlex.quote(part) for part in command), flush=True)
    result = subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    output = "\n".join(line for line in result.stdout.splitlines() if noise not in line)
    if result.returncode != 0:
        raise RuntimeError(f"build step failed ({result.returncode}): {' '.join(command)}\n{output}")
    if verbose and output.strip():
        print(output, flush=True)


def hipcc_path() -> str:
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    candidate = Path(rocm) / "bin" / "hipcc"
    return str(candidate) if candidate.exists() else "hipcc"


def build_kernels(verbose: bool = False) -> Path:
    sources = [str(CSRC / name) for name in KERNEL_SOURCES]
    command = [hipcc_path(), *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", *sources, "-o", str(KERNEL_LIBRARY)]
    _run(command, verbose)
    return KERNEL_LIBRARY


def build_extension(verbose: bool = False) -> Path:
    import torch
    from torch.utils import cpp_extension

    include_dirs = [*cpp_extension.include_paths("cuda"), sysconfig.get_paths()["include"], str(INCLUDE)]
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    command = [
        os.environ.get("CXX", "g++"),
        "-O2",
        "-std=c++17",
        "-fPIC",
        "-shared",
        "-fvisibility=hidden",
        "-Wall",
        "-Wno-unused-function",
        "-D__HIP_PLATFORM_AMD__=1",
        "-DUSE_ROCM=1",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-DTORCH_EXTENSION_NAME={EXTENSION_NAME}",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *[f"-I{path}" for path in include_dirs],
        str(CSRC / "nanoep_torch.cpp"),
        "-o",
        str(EXTENSION_LIBRARY),
        f"-L{torch_lib}",
        f"-L{PACKAGE}",
        "-lnanoep_hip",
        "-lc10",
        "-lc10_hip",
        "-ltorch_cpu",
        "-ltorch_hip",
        "-ltorch",
        "-ltorch_python",
        "-lamdhip64",
        "-Wl,-rpath,$ORIGIN",
        f"-Wl,-rpath,{torch_lib}",
    ]
    _run(command, verbose)
    return EXTENSION_LIBRARY


def build_all(verbose: bool = False) -> list[Path]:
    return [build_kernels(verbose), build_extension(verbose)]


if __name__ == "__main__":
    built = build_all(verbose="-q" not in sys.argv)
    for path in built:
        print(f"built {path.relative_to(ROOT)}")
