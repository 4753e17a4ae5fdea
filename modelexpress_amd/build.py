"""Builds libmxplace.so (HIP kernels + C++ host engine) for gfx950 with hipcc.

Run as ``python -m modelexpress_amd.build``.  hipcc cross-compiles without a GPU, so
this works on a build host; the resulting library sits next to this file.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libmxplace.so"

SOURCES = (
    "mxp_kernels.hip",
    "mxp_synth.hip",
    "mxp_permute.hip",
    "mxp_ckpt.cpp",
    "mxp_plan.cpp",
    "mxp_engine.cpp",
    "mxp_crc32c.cpp",
)

# -packed-fp32-ops is switched off on purpose for every device compile: the packed fp32
# instruction forms are not wanted in this library's kernels.
DEVICE_FLAGS = (
    "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)
COMMON_FLAGS = (
    "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
    "-Wno-unknown-attributes", "-Wno-unused-command-line-argument",
    "-D__HIP_PLATFORM_AMD__",
)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def _compile(hipcc: str, src: Path, obj: Path) -> None:
    cmd = [hipcc, *COMMON_FLAGS, *DEVICE_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-x", "hip", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_library(force: bool = True, jobs: int = 4) -> Path:
    """Compile every source and link the shared library. Returns its path."""
    hipcc = _hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    headers = list(CSRC.glob("*.h")) + list(CSRC.glob("*.hpp")) + [INCLUDE / "mxp.h", INCLUDE / "mxp_bench.h"]
    newest_header = max(h.stat().st_mtime for h in headers)
    todo = []
    objs = []
    for name in SOURCES:
        src = CSRC / name
        obj = obj_dir / (name + ".o")
        objs.append(obj)
        if force or not obj.exists() or obj.stat().st_mtime < max(src.stat().st_mtime, newest_header):
            todo.append((src, obj))
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for fut in [pool.submit(_compile, hipcc, s, o) for s, o in todo]:
            fut.result()
    if todo or not LIB_PATH.exists():
        cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *map(str, objs), "-o", str(LIB_PATH), "-lpthread"]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


ABI_DRIVER_SRC = PKG_DIR.parent / "tests" / "c" / "abi_driver.c"
ABI_DRIVER = ABI_DRIVER_SRC.with_suffix("")


def build_abi_driver() -> Path:
    """Compile the plain-C caller of the library (tests/c/abi_driver.c) with gcc: it includes
    only include/mxp.h and the HIP runtime API header, and links libmxplace.so and libamdhip64."""
    rocm = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
    cmd = ["gcc", "-std=c11", "-O1", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", f"-I{INCLUDE}", f"-I{rocm / 'include'}",
           str(ABI_DRIVER_SRC), "-o", str(ABI_DRIVER), f"-L{PKG_DIR}", "-lmxplace", f"-L{rocm / 'lib'}", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../modelexpress_amd", f"-Wl,-rpath,{rocm / 'lib'}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed on {ABI_DRIVER_SRC.name}:\n{proc.stderr}")
    if proc.stderr.strip():
        sys.stderr.write(proc.stderr)
    return ABI_DRIVER


if __name__ == "__main__":
    path = build_library(force="--incremental" not in sys.argv)
    print(path)
    if "--abi-driver" in sys.argv:
        print(build_abi_driver())
