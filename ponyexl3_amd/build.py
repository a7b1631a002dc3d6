"""Builds libexl3_hip.so (gfx950) in-tree with hipcc.

``python -m ponyexl3_amd.build`` or ``ponyexl3_amd.build.build()``. Each .hip
file is one translation unit compiled in parallel; the objects are linked into
``ponyexl3_amd/libexl3_hip.so``, the C-ABI library declared in
``include/exl3_hip.h``, and (``diag.hip`` alone) ``ponyexl3_amd/libexl3_diag.so``,
the measurement probes declared in ``include/exl3_diag.h``.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(PKG_DIR, "libexl3_hip.so")

SOURCES = ["decode.hip", "hadamard.hip", "gemv.hip", "linear_mid.hip", "gemm.hip", "moe.hip", "search.hip", "capi.hip"]
# measurement probes (include/exl3_diag.h): a library of their own, kept out of the product ABI
DIAG_SOURCES = ["diag.hip"]
DIAG_LIB_PATH = os.path.join(PKG_DIR, "libexl3_diag.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU ops are kept out of the generated code on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the EXL3 kernels need the ROCm toolchain")
    return exe


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stderr[-8000:]}")
    noise = "packed-fp32-ops"  # host pass does not know -packed-fp32-ops; harmless
    warn = "\n".join(l for l in proc.stderr.splitlines() if noise not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = False, jobs: int | None = None, extra_flags: list[str] | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    extra = list(extra_flags or [])
    every = SOURCES + DIAG_SOURCES
    jobs = jobs or min(len(every), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra), every))
    for path, group in ((LIB_PATH, objs[: len(SOURCES)]), (DIAG_LIB_PATH, objs[len(SOURCES):])):
        cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path, *group]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr[-4000:]}")
        if verbose:
            print(f"built {path} ({os.path.getsize(path)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
