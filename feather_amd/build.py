"""Build libfeather_hip.so (gfx950 only) with hipcc.

    python -m feather_amd.build            # compile every csrc/*.hip, link in-tree
    python -m feather_amd.build --if-stale # only when a source is newer than the library

hipcc cross-compiles for gfx950 without a GPU present.  The library lands in
``feather_amd/lib/`` next to the sources so that it travels with the tree.
"""
from __future__ import annotations

import argparse
import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfeather_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: v_pk_*_f32 forms are not used.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-fno-gpu-rdc", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators stay in architectural VGPRs: the kernels rescale them with VALU ops, and
    # every such touch of an AGPR accumulator costs a v_accvgpr_read/write pair
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # the first 16 dwords of kernel arguments arrive in SGPRs with the wave instead of through s_load
    # (a cold scalar-cache miss at the start of every kernel); code objects keep a loader prologue for
    # firmware without the feature
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")
    return exe


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def headers() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.h"))) + [os.path.join(HERE, "..", "include", "feather_hip.h")]


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in sources() + headers())


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    noise = "is not a recognized feature for this target"
    warn = "\n".join(l for l in r.stderr.splitlines() if l.strip() and noise not in l)
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--if-stale", action="store_true")
    args = ap.parse_args()
    if args.if_stale and not is_stale():
        print(f"{LIB_PATH} is up to date")
        return
    build()


if __name__ == "__main__":
    main()
