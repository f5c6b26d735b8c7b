"""Builds libxma_hip.so (the C-ABI kernel library) for gfx950 with hipcc.

The reference compiles its native code at first use through torch's JIT extension loader
(xma/jit.py:22-87).  Here the library is built ahead of time, in-tree, so that a machine without
a compiler (or without the sources' include paths) can load the shared object directly:

    python -m flash_model_architectures_amd.build
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor


_PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_PACKAGE_DIR, "csrc")
LIB_DIR = os.path.join(_PACKAGE_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libxma_hip.so")

SOURCES = ["common.hip", "routing.hip", "rowmove.hip", "seqpack.hip", "bias.hip", "swiglu.hip", "router_wgrad.hip", "grouped_gemm.hip", "grouped_gemm_dma.hip"]

# packed-fp32 VALU forms are switched off for every kernel in this library
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built on this machine")
    return path


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}")
    noise = "'-packed-fp32-ops' is not a recognized feature"
    out = "\n".join(line for line in proc.stdout.splitlines() if noise not in line and line.strip())
    if out:
        print(out, file=sys.stderr)


def _up_to_date(src: str, obj: str) -> bool:
    """True if `obj` is newer than the source, every header in csrc/ and the public header."""

    if not os.path.exists(obj):
        return False
    deps = [os.path.join(CSRC_DIR, src)]
    deps += [os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".h")]
    deps.append(os.path.join(os.path.dirname(_PACKAGE_DIR), "include", "xma_hip.h"))
    return all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps if os.path.exists(d))


def build(verbose: bool = False, jobs: int | None = None, incremental: bool = False) -> str:
    """Compile every source in csrc/ and link lib/libxma_hip.so; returns the library path.  `incremental` (the
    command line's -i) skips sources whose object file is newer than everything it is built from."""

    hipcc = _hipcc()
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        if incremental and _up_to_date(src, obj):
            return obj
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC_DIR, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        _run(cmd)
        return obj

    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(compile_one, SOURCES))

    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objects])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, incremental="-i" in sys.argv))
