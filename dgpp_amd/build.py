"""Builds libdgpp_amd.so (HIP kernels for gfx950 + the C ABI + host encoders) in-tree.

hipcc cross-compiles without a GPU. Objects go to dgpp_amd/_build/, the library to
dgpp_amd/lib/libdgpp_amd.so. Run as `python -m dgpp_amd.build`.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
BUILD = PKG / "_build"
LIB_DIR = PKG / "lib"
LIB = LIB_DIR / "libdgpp_amd.so"
# A C++ host program over include/dgpp_amd.hpp (reference-style host code calling the dgpp::launch_* names), run by
# the GPU tests as a subprocess.
HOST_PROGRAM_SRC = PKG.parent / "tests" / "cpp" / "host_program.cpp"
HOST_PROGRAM = LIB_DIR / "dgpp_host_program"

HIP_SOURCES = [
    "gemv_mxfp4.hip",
    "gemv_nvfp4.hip",
    "gemv_mixed.hip",
    "gemv_fp8f32.hip",
    "gemv_fp8e8m0.hip",
    "moe_router.hip",
    "moe_grouping.hip",
    "moe_elementwise.hip",
    "mxfp8_gemm.hip",
    "nvfp4_act.hip",
    "qwen_tail.hip",
    "capi.hip",
]
HOST_SOURCES = ["host_codec.cpp", "loader.cpp"]
# Host C++ that needs the HIP runtime headers (compiled by hipcc as plain host code).
HIP_HOST_SOURCES = ["moe_layer.cpp", "moe_resident.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-FP32 instruction selection is switched off for all device code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]
HIP_FLAGS += os.environ.get("DGPP_EXTRA_HIP_FLAGS", "").split()   # e.g. -D switches for an experiment
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-ffp-contract=off", "-pthread"]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def _stale(obj: Path, src: Path) -> bool:
    if not obj.exists():
        return True
    newest = max(p.stat().st_mtime for p in list(CSRC.glob("*.hpp")) + [src] + list((PKG.parent / "include").glob("*.h*")))
    return obj.stat().st_mtime < newest


def build(force: bool = True, jobs: int = 6) -> Path:
    """Compiles every source (always, when force) and links the shared library."""
    BUILD.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    tasks = []
    objs = []
    for name in HIP_SOURCES:
        src, obj = CSRC / name, BUILD / (name + ".o")
        objs.append(obj)
        if force or _stale(obj, src):
            tasks.append([HIPCC, *HIP_FLAGS, "-c", str(src), "-o", str(obj)])
    for name in HIP_HOST_SOURCES:
        src, obj = CSRC / name, BUILD / (name + ".o")
        objs.append(obj)
        if force or _stale(obj, src):
            tasks.append([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-c", str(src),
                          "-o", str(obj)])
    for name in HOST_SOURCES:
        src, obj = CSRC / name, BUILD / (name + ".o")
        objs.append(obj)
        if force or _stale(obj, src):
            tasks.append([shutil.which("g++") or "g++", *HOST_FLAGS, "-c", str(src), "-o", str(obj)])
    with cf.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, tasks))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)])
    if HOST_PROGRAM_SRC.exists() and (force or not HOST_PROGRAM.exists() or
                                      HOST_PROGRAM.stat().st_mtime < max(HOST_PROGRAM_SRC.stat().st_mtime, LIB.stat().st_mtime)):
        # host code only (no kernels of its own): it finds the library next to itself
        _run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", str(HOST_PROGRAM_SRC), "-o", str(HOST_PROGRAM),
              f"-L{LIB_DIR}", "-ldgpp_amd", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv))
