"""Compiles the HIP library in-tree for gfx950.

``python -m aristos_amd.build`` or ``build_library()``; the result is ``aristos_amd/libkleos_amd.so``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libkleos_amd.so")
DRIVER_PATH = os.path.join(CSRC, "kleos_main")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 arithmetic is kept off for every device function of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-pass-failed",
]
SOURCES = ["config.cpp", "capi.hip", "kernels.hip", "kernels_f32.hip", "kernels_tf32.hip", "kernels_bf16.hip", "kernels_f16.hip"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the library can only be built with the ROCm toolchain")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"build failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_library(driver: bool = True, jobs: int = 6) -> str:
    """Compiles every HIP source into libkleos_amd.so (and the C++ driver); returns the library path.
    The sources are compiled side by side (one hipcc process each, objects under aristos_amd/build/),
    then linked."""
    from concurrent.futures import ThreadPoolExecutor
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.splitext(src)[0] + ".o") for src in SOURCES]
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(SOURCES)))) as pool:
        list(pool.map(lambda so: _run([_hipcc(), *HIPCC_FLAGS, "-c", so[0], "-o", so[1]]), zip(SOURCES, objs)))
    tmp = LIB_PATH + ".tmp"
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", *objs, "-o", tmp])
    os.replace(tmp, LIB_PATH)
    if driver:
        _run([_hipcc(), *HIPCC_FLAGS, "main.cpp", "-o", DRIVER_PATH, f"-L{PKG_DIR}", "-lkleos_amd",
              f"-Wl,-rpath,{PKG_DIR}"])
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
