"""Builds libqvb8_amd.so (HIP, gfx950 only) in-tree with hipcc.

    python -m qvb8_amd.build            # compile every source into qvb8_amd/lib/libqvb8_amd.so

The library is loaded by qvb8_amd._lib with ctypes.  There is no other backend: if the
library is missing and cannot be built, every operator raises.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libqvb8_amd.so")
SOURCES = ["qvb8_kernels.hip", "qvb8_tile.hip", "qvb8_mlp.hip", "qvb8_moe.hip", "qvb8r.hip", "qvb8_attn.hip"]
ARCH = "gfx950"
# packed-fp32 VALU forms are switched off for every device compile of this library
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                # the first 16 dwords of a kernel's arguments arrive in registers instead of being fetched by the first
                # instructions (measured: about 1 % on the decode step)
                "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def sources() -> list[str]:
    return [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]


def build(verbose: bool = True) -> str:
    """Compiles every source to an object (in parallel, one hipcc each) and links them into the library."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    common = [hipcc_path(), f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-sanitize", *DEVICE_FLAGS,
              "-I", os.path.join(os.path.dirname(HERE), "include")]

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed ({r.returncode}):\n{out}")
        if verbose and out.strip():
            print(out)

    srcs = sources()
    objs = [os.path.join(obj_dir, os.path.basename(s) + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(lambda so: run([*common, "-c", so[0], "-o", so[1]]), zip(srcs, objs)))
    tmp = LIB_PATH + ".tmp"
    run([hipcc_path(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-sanitize", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    deps.append(os.path.join(os.path.dirname(HERE), "include", "qvb8_amd.h"))
    return any(os.path.getmtime(d) > t for d in deps if os.path.isfile(d))


if __name__ == "__main__":
    print(build())
    sys.exit(0)
