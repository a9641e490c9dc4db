"""Builds libskainet_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m skainet_amd.build            # compile every csrc/*.hip and link skainet_amd/libskainet_hip.so

hipcc cross-compiles for gfx950 without a GPU.  The library has no dependency beyond the HIP runtime.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libskainet_hip.so")

ARCH = "gfx950"
# packed-fp32 VALU forms are kept off: scalar fp32 code must not be fused into v_pk_* instructions
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libskainet_hip needs the ROCm toolchain")
    return exe


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"command failed ({p.returncode}): {' '.join(cmd)}\n{out}")
    return out


def build_library(jobs=8, verbose=False, save_temps=False):
    os.makedirs(OBJ, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources found")
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        extra = ["-save-temps=obj"] if save_temps else []
        return _run([hipcc(), *FLAGS, *extra, "-c", src, "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, out in zip(sources, ex.map(compile_one, zip(sources, objs))):
            if verbose and out.strip():
                print(f"--- {os.path.basename(src)}\n{out}")
    _run([hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True, save_temps="--save-temps" in sys.argv))
