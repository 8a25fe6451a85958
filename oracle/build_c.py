"""Builds oracle/_build/librnnt_oracle_c.so from oracle/rnnt_oracle_c.c with gcc (-O2, OpenMP).

Test infrastructure: the library is loaded by tests/ and by bench.py's cpu_baseline leg only.

Usage:  python -m oracle.build_c
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "rnnt_oracle_c.c")
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "librnnt_oracle_c.so")


def build(verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ["gcc", "-O2", "-fopenmp", "-fPIC", "-shared", "-std=c11", "-Wall", SRC, "-o", LIB + ".tmp", "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed on rnnt_oracle_c.c:\n" + res.stderr)
    os.replace(LIB + ".tmp", LIB)
    return LIB


def load():
    """ctypes handle of the built library (built on first use when missing)."""
    if not os.path.exists(LIB):
        build(verbose=False)
    lib = C.CDLL(LIB)
    p, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
    lib.rnnt_oracle_c_threads.restype = C.c_int
    lib.rnnt_oracle_c_loss_grad.restype = C.c_int
    lib.rnnt_oracle_c_loss_grad.argtypes = [p, i64, i64, p, p, p, i64, i32, i32, C.c_int, p, p, p, p]
    return lib


def loss_and_grad(lib, x, lx, y, ly, blank=0, fused=True, grad_out=None, want_G=True, want_grad=True):
    """NumPy front of rnnt_oracle_c_loss_grad: x (R,V) float32, lx / ly (N,) int32, y padded (N,Umax) or
    concatenated (sum U,) int32.  Returns dict(costs, G, grad)."""
    import numpy as np
    x = np.ascontiguousarray(x, dtype=np.float32)
    lx = np.ascontiguousarray(lx, dtype=np.int32)
    ly = np.ascontiguousarray(ly, dtype=np.int32)
    y = np.ascontiguousarray(y, dtype=np.int32)
    R, V = x.shape
    N = len(lx)
    stride = y.shape[1] if y.ndim == 2 else -1
    costs = np.zeros(N)
    G = np.zeros((R, 2)) if want_G else None
    grad = np.empty((R, V), dtype=np.float32) if want_grad else None
    go = None if grad_out is None else np.ascontiguousarray(grad_out, dtype=np.float64)
    ptr = lambda a: None if a is None else a.ctypes.data
    rc = lib.rnnt_oracle_c_loss_grad(ptr(x), R, V, ptr(lx), ptr(ly), ptr(y), stride, N, blank, 1 if fused else 0,
                                     ptr(go), ptr(costs), ptr(G), ptr(grad))
    if rc != 0:
        raise RuntimeError(f"rnnt_oracle_c_loss_grad returned {rc}")
    return dict(costs=costs, G=G, grad=grad)


if __name__ == "__main__":
    print(build())
