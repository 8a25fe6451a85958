"""Builds libcwarp_rnnt_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage:  python -m compactwarprnntloss_amd.build
"""
from __future__ import annotations

import os
import re
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


# A scalar select or branch reads the scalar condition code (SCC).  hipcc 7.2 has been seen to emit,
# for a select on a wave-uniform loop counter that register pressure had pushed into a vector
# register, a v_cmp (which sets VCC) followed by an s_cselect that reads an SCC nobody set: the
# lattice kernel then published a wrong progress count and a neighbouring wave waited for good.
# The device assembly of every translation unit is therefore checked for SCC readers whose last SCC
# writer is not a compare although a vector compare sits between the two.
_SCC_WRITER = re.compile(r"^\s*(s_cmp|s_and|s_or|s_xor|s_andn2|s_orn2|s_nand|s_nor|s_xnor|s_add_|s_sub_|s_addc|s_subb|"
                         r"s_lshl|s_lshr|s_ashr|s_bfe|s_min|s_max|s_abs|s_not|s_bitcmp|s_absdiff|s_addk|s_cmpk|s_wqm|"
                         r"s_quadmask|s_bcnt|s_ff|s_flbit|s_sext|s_bitset)")
_SCC_READER = re.compile(r"^\s*(s_cselect|s_cbranch_scc|s_cmov)")
_SCC_COMPARE = ("s_cmp", "s_and_b64", "s_bitcmp", "s_cmpk")


def stale_scc_reads(asm_text: str):
    """Lines (1-based number, text) of the device assembly whose scalar select / branch looks like it
    reads a condition code left by an unrelated instruction."""
    found = []
    last_writer = None
    vcmp_since = False
    for i, line in enumerate(asm_text.split("\n")):
        if line.startswith(".LBB") or re.match(r"^\S.*:$", line):
            last_writer, vcmp_since = None, False
            continue
        if _SCC_READER.match(line):
            if last_writer is None or (vcmp_since and not last_writer.strip().startswith(_SCC_COMPARE)):
                found.append((i + 1, line.strip()))
        if re.match(r"^\s*v_cmp", line):
            vcmp_since = True
        if _SCC_WRITER.match(line):
            last_writer, vcmp_since = line, False
    return found


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
        # -save-temps=obj leaves the device assembly next to the object, for the check below
        cmd = [hipcc, *FLAGS, *EXTRA_FLAGS.get(src, []), "-save-temps=obj", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in res.stderr.splitlines() if "not a recognized feature" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        asm = os.path.join(objdir, src.replace(".hip", f"-hip-amdgcn-amd-amdhsa-{ARCH}.s"))
        with open(asm) as f:
            bad = stale_scc_reads(f.read())
        if bad:
            raise RuntimeError(f"{src}: scalar condition code read without a matching compare at {asm}: {bad[:5]}")
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
