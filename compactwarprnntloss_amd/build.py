"""Builds libcwarp_rnnt_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage:  python -m compactwarprnntloss_amd.build
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libcwarp_rnnt_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["api.hip", "lattice.hip", "rows.hip", "pack.hip", "join.hip", "joint.hip"]
ARCH = "gfx950"
# -packed-fp32-ops is switched off: hipcc would otherwise pair fp32 operations into packed
# instructions, which have produced sporadic wrong results on the target machines.
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         # "#pragma unroll N" on loops with run-time bounds is a request, not a promise
         "-Wno-pass-failed"]


# The streaming kernels take row maxima with fmaxf; without this the compiler adds one
# canonicalising v_max per input element to quiet signalling NaNs.
EXTRA_FLAGS = {"rows.hip": ["-fno-honor-nans"]}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build " + LIB_NAME)
    return exe


def build(verbose: bool = True) -> str:
    """Compile every translation unit and link the shared library.  Returns its path."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in res.stderr.splitlines() if "not a recognized feature" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
