"""Build ``libiron_hip.so``: every HIP source of ``csrc/`` compiled for gfx950.

``python -m iron_amd.build`` or ``build()``; hipcc cross-compiles without a GPU.
The library is written beside this file so it travels with the source tree.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libiron_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops off: the compiler is not to form v_pk_*_f32 from float code.
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    # The first 16 dwords of a kernel's arguments arrive in SGPRs with the wave instead of by a
    # scalar load the kernel's first instructions wait for: about a memory trip off every launch of a
    # chain of short dependent kernels.  (A kernel keeps a prologue that loads them for hardware
    # that does not preload.)
    "-mllvm",
    "-amdgpu-kernarg-preload-count=16",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(found).exists():
        raise RuntimeError("hipcc not found: libiron_hip.so cannot be built here")
    return found


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{err}")
    if err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False) -> Path:
    """Compile every source and link the shared library; always recompiles."""
    hipcc = _hipcc()
    objdir = HERE / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [objdir / (s.stem + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"hipcc {src.name}")
        _run([hipcc, *FLAGS, "-c", str(src), "-o", str(obj)])

    jobs = min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
