"""Builds libtlce_gfx950.so, the C-ABI HIP library, in-tree with plain hipcc.

The reference JIT-builds its CUDA extension through torch.utils.cpp_extension
with ``-O3 --use_fast_math -lcublas``
(dllm_parallel/core/kernels/_native_specs.py:63-143).  This library has no
torch or BLAS dependency, so the build is one hipcc command; the result sits
next to this file where the ctypes loader looks for it.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIBRARY_NAME = "libtlce_gfx950.so"
LIBRARY_PATH = PACKAGE_DIR / LIBRARY_NAME
SOURCES = ("tlce_compact.hip", "tlce_linear_ce.hip")
OFFLOAD_ARCH = "gfx950"

HIPCC_FLAGS = (
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-munsafe-fp-atomics",
    # the direct-to-LDS loads name m0 (reserved) in their inline-asm clobber list
    "-Wno-inline-asm",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return str(candidate)
    raise RuntimeError("hipcc not found; install ROCm or set HIPCC")


def build_library(verbose: bool = False) -> Path:
    """Compiles every HIP source for gfx950 and links the shared library."""
    command = [find_hipcc(), *HIPCC_FLAGS]
    command += [str(CSRC_DIR / name) for name in SOURCES]
    command += ["-o", str(LIBRARY_PATH)]
    if verbose:
        print(" ".join(command), flush=True)
    result = subprocess.run(command, capture_output=True, text=True)
    # the host pass warns that it does not know the device-only feature flag
    stderr = "\n".join(
        line for line in result.stderr.splitlines() if "packed-fp32-ops" not in line
    )
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed ({result.returncode}):\n{stderr}")
    if verbose and stderr.strip():
        print(stderr, file=sys.stderr)
    return LIBRARY_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
