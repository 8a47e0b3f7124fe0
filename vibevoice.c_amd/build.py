"""Builds libvibevoice_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python vibevoice.c_amd/build.py            # or: __graft_entry__.build()

Each .hip file is compiled to an object in parallel, then linked into
vibevoice.c_amd/lib/libvibevoice_hip.so. Nothing is downloaded or installed.
"""
from __future__ import annotations

import concurrent.futures as cf
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libvibevoice_hip.so")
ARCH = "gfx950"

# -packed-fp32-ops off: scalar FP32 arithmetic is never fused into v_pk_*_f32.
# -amdgpu-kernarg-preload-count: the first 16 dwords of a kernel's arguments arrive in scalar registers with the
# wave instead of being fetched by its first instructions - one memory round trip less before a kernel's first
# load (a 512-row add+norm 4.20 -> 3.95 us, a one-row launch 2.4 -> 2.1 us; long kernels do not notice).
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-mllvm", "-amdgpu-kernarg-preload-count=16"]
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
            "-Wno-unused-parameter", f"--offload-arch={ARCH}"] + DEVICE_FLAGS


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP backend cannot be built here")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    cmd = [hipcc(), *CXXFLAGS, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
    err = "\n".join(l for l in res.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    with cf.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(_compile, sources))
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB, *objs]
    subprocess.check_call(cmd)
    stale = os.path.join(LIBDIR, "libvibevoice_hip_unsupported.so")      # an older build's second library
    if os.path.exists(stale):
        os.remove(stale)
    if verbose:
        print(f"built {LIB} from {len(sources)} sources for {ARCH}")
    return LIB


if __name__ == "__main__":
    build()
