"""Writes the golden fixtures tests/golden/*.npz.

The reference repository holds no golden vectors and cannot be built or run without CUDA, so the
fixtures are produced by the float64 oracle (oracle/rnnt_oracle.py), which tests/test_oracle_pins.py
pins against brute-force path enumeration, closed forms, finite differences and autograd.  Each
file stores inputs (x, lx, ly, y, blank, mode, grad_out) and expected outputs (costs, G, grad,
int32 row offsets).  The join_*.npz files hold the compact joiner front instead: inputs (f, g, lx,
ly, act, dh) and expected outputs (h, df, dg) from the oracle's join_rows / join_rows_backward.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import rnnt_oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = [
    # name, lx, ly, V, blank, mode, seed, label_equals_blank_at
    ("ragged_fused", [7, 1, 12, 2, 5], [3, 4, 0, 2, 5], 12, 0, "fused", 1, None),
    ("ragged_logprob", [7, 1, 12, 2, 5], [3, 4, 0, 2, 5], 12, 0, "logprob", 2, None),
    ("blank_last_fused", [4, 9], [3, 2], 8, 7, "fused", 3, None),
    ("blank_mid_logprob", [4, 9], [3, 2], 8, 3, "logprob", 4, None),
    ("label_is_blank_logprob", [4, 3], [2, 2], 8, 0, "logprob", 5, (0, 0)),
    ("two_strips_fused", [6, 3], [70, 64], 16, 0, "fused", 6, None),
]


def main():
    for name, lx, ly, V, blank, mode, seed, lb in CASES:
        rng = np.random.default_rng(seed)
        lx = np.asarray(lx, dtype=np.int32)
        ly = np.asarray(ly, dtype=np.int32)
        N = len(lx)
        R = int(orc.row_offsets_i64(lx, ly)[-1])
        x = rng.standard_normal((R, V)).astype(np.float32)
        if mode == "logprob":
            x = orc.log_softmax(x).astype(np.float32)
        y = np.zeros((N, int(ly.max())), dtype=np.int32)
        for n in range(N):
            lab = rng.integers(0, V - 1, int(ly[n])).astype(np.int32)
            lab[lab >= blank] += 1
            y[n, : ly[n]] = lab
        if lb is not None:
            y[lb] = blank
        go = rng.uniform(-1.5, 1.5, N)
        out = orc.loss_and_grad(x.astype(np.float64), lx, y, ly, blank, mode, grad_out=go)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, lx=lx, ly=ly, y=y, blank=np.int32(blank),
                            mode=np.array(mode), grad_out=go, costs=out["costs"], G=out["G"],
                            grad=out["grad"], row_off_i32=orc.row_offsets(lx, ly))
        print(name, "R =", R, "costs", np.round(out["costs"], 4))


JOIN_CASES = [
    # name, lx, ly, H, activation, seed, padding of (T, U+1) beyond the longest sequence
    ("join_tanh", [5, 1, 7, 3], [2, 4, 0, 6], 24, "tanh", 7, (1, 2)),
    ("join_sum", [3, 6], [5, 1], 10, "none", 8, (0, 0)),
]


def main_join():
    for name, lx, ly, H, act, seed, (tp, up) in JOIN_CASES:
        rng = np.random.default_rng(seed)
        lx = np.asarray(lx, dtype=np.int32)
        ly = np.asarray(ly, dtype=np.int32)
        N = len(lx)
        f = rng.standard_normal((N, int(lx.max()) + tp, H)).astype(np.float32)
        g = rng.standard_normal((N, int(ly.max()) + 1 + up, H)).astype(np.float32)
        h = orc.join_rows(f, g, lx, ly, act)
        dh = rng.standard_normal(h.shape).astype(np.float32)
        df, dg = orc.join_rows_backward(dh, f, g, lx, ly, act)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), f=f, g=g, lx=lx, ly=ly, act=np.array(act), dh=dh,
                            h=h, df=df, dg=dg)
        print(name, "rows =", h.shape[0], "H =", H)


if __name__ == "__main__":
    main_join()
    main()
