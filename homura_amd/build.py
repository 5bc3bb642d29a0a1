"""Builds libhomura_amd.so (HIP kernels + C boundary + host plan) for gfx950, in-tree.

`python -m homura_amd.build` or `homura_amd.build.build_library()`. hipcc cross-compiles, so
this works on a machine without a GPU. Objects go to homura_amd/_build/, the library to
homura_amd/libhomura_amd.so.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
BUILD_DIR = PKG_DIR / "_build"
LIB_PATH = PKG_DIR / "libhomura_amd.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-pthread"]


def _sources() -> list[Path]:
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")) +
                  list((CSRC / "host").glob("*.hip")) + list((CSRC / "host").glob("*.cpp")))


def _compile(src: Path) -> Path:
    obj = BUILD_DIR / (src.stem + ".o")
    if src.suffix == ".hip":
        cmd = [HIPCC, *HIP_FLAGS, "-c", str(src), "-o", str(obj)]
    else:
        cmd = ["g++", *HOST_FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"compile failed: {' '.join(cmd)}\n{res.stdout}\n{res.stderr}")
    # hipcc's host pass does not know the packed-fp32 feature and says so; everything else is shown
    noise = ("packed-fp32-ops", "is not a recognized feature")
    for line in res.stderr.splitlines():
        if line.strip() and not any(n in line for n in noise):
            print(line, file=sys.stderr)
    return obj


def build_library(jobs: int | None = None, verbose: bool = True) -> Path:
    BUILD_DIR.mkdir(exist_ok=True)
    srcs = _sources()
    if not srcs:
        raise RuntimeError(f"no sources under {CSRC}")
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH),
           *map(str, objs), "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed: {' '.join(cmd)}\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
