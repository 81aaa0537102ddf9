"""Builds libtlce_gfx950.so, the C-ABI HIP library, in-tree with plain hipcc.

The reference JIT-builds its CUDA extension through torch.utils.cpp_extension
with ``-O3 --use_fast_math -lcublas``
(dllm_parallel/core/kernels/_native_specs.py:63-143).  This library has no
torch or BLAS dependency: every source is compiled to an object with one hipcc
command (in parallel, one translation unit per tile engine) and the objects
are linked into a shared library that sits next to this file, where the ctypes
loader looks for it.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
OBJECT_DIR = CSRC_DIR / "build"
LIBRARY_NAME = "libtlce_gfx950.so"
LIBRARY_PATH = PACKAGE_DIR / LIBRARY_NAME
# (object name, source, extra definitions).  tlce_engine_unit.hip is compiled once
# per engine, and once per kernel family for the two direct-to-LDS MFMA engines,
# whose kernels take the longest to compile.
_SPLIT_ENGINES = {"direct_bf16": "MfmaDirect4Engine<__bf16>",
                  "direct_f16": "MfmaDirect4Engine<_Float16>"}
_WHOLE_ENGINES = {"staged_bf16": "MfmaEngine<__bf16>", "staged_f16": "MfmaEngine<_Float16>",
                  "generic_f32": "SimtEngine<float>", "generic_bf16": "SimtEngine<__bf16>",
                  "generic_f16": "SimtEngine<_Float16>"}
_PARTS = {2: "grad_logits", 7: "grad_logits_cap", 8: "grad_logits_bias", 9: "grad_logits_cap_bias",
          1: "forward", 3: "gemm", 4: "kl", 5: "logits", 6: "sequences",
          10: "forward_dim_first", 11: "grad_logits_dim_first", 12: "exp_panel"}
# the forward that leaves the gradients (part 12 and its launch sequence) exists for bf16 only
_FUSED_ENGINES = ("direct_bf16",)
UNITS = (
    [(f"engine_{tag}_{name}", "tlce_engine_unit.hip",
      (f"-DTLCE_UNIT_ENGINE={engine}", f"-DTLCE_UNIT_PART={part}")
      + (("-DTLCE_UNIT_FUSED=1",) if tag in _FUSED_ENGINES else ()))
     for tag, engine in _SPLIT_ENGINES.items() for part, name in _PARTS.items()
     if part != 12 or tag in _FUSED_ENGINES]
    + [(f"engine_{tag}", "tlce_engine_unit.hip",
        (f"-DTLCE_UNIT_ENGINE={engine}", "-DTLCE_UNIT_PART=0"))
       for tag, engine in _WHOLE_ENGINES.items()]
    + [("linear_ce", "tlce_linear_ce.hip", ()), ("compact", "tlce_compact.hip", ())]
)
OFFLOAD_ARCH = "gfx950"

HIPCC_FLAGS = (
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
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


def _run(command: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(command), flush=True)
    result = subprocess.run(command, capture_output=True, text=True)
    # the host pass warns that it does not know the device-only feature flag
    stderr = "\n".join(
        line for line in result.stderr.splitlines() if "packed-fp32-ops" not in line
    )
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed ({result.returncode}): {' '.join(command)}\n{stderr}")
    if verbose and stderr.strip():
        print(stderr, file=sys.stderr)


def _newest_source_time() -> float:
    sources = [*CSRC_DIR.glob("*.h"), *CSRC_DIR.glob("*.hip"),
               PACKAGE_DIR.parent / "include" / "tlce.h", Path(__file__)]
    return max(path.stat().st_mtime for path in sources)


def build_library(verbose: bool = False, jobs: int | None = None,
                  incremental: bool = False) -> Path:
    """Compiles every HIP source for gfx950 and links the shared library.
    ``incremental`` skips objects newer than every source and header (for the
    edit-compile loop; the default recompiles everything)."""
    hipcc = find_hipcc()
    OBJECT_DIR.mkdir(exist_ok=True)
    objects = [OBJECT_DIR / (name + ".o") for name, _, _ in UNITS]
    commands = [
        [hipcc, *HIPCC_FLAGS, *defines, "-c", str(CSRC_DIR / source), "-o", str(obj)]
        for (_, source, defines), obj in zip(UNITS, objects)
    ]
    if incremental:
        newest = _newest_source_time()
        commands = [command for command, obj in zip(commands, objects)
                    if not obj.exists() or obj.stat().st_mtime < newest]
    if jobs is None:
        jobs = min(len(commands), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=max(int(jobs), 1)) as pool:
        list(pool.map(lambda command: _run(command, verbose), commands))
    _run([hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC",
          *[str(obj) for obj in objects], "-o", str(LIBRARY_PATH)], verbose)
    return LIBRARY_PATH


if __name__ == "__main__":
    print(build_library(verbose=True, incremental="--incremental" in sys.argv[1:]))
