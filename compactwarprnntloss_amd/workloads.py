"""Seeded synthetic batches: the five benchmark configurations of the compact RNN-T loss.

Shared by the benchmark, the smoke check and the tests, so that all of them draw exactly the same
lengths, labels and logits.  NumPy only.
"""
from __future__ import annotations

import math

import numpy as np


def make_config(idx, seed=None, scale=1.0):
    """Seeded synthetic batch for configuration idx in 1..5.

    Returns dict(N, V, lx, ly (int32), y_padded (N,Umax) int32, y_cat (sum U,) int32, sigma,
    dtype ('f32'|'f16'), R).  Logits are NOT generated here (they are large); use
    make_logits().  `scale` < 1 shrinks the T/U ranges for quick tests.
    """
    rng = np.random.default_rng(idx if seed is None else seed)

    def s(v, lo=1):
        return max(lo, int(round(v * scale)))

    if idx == 1:
        N, V, sigma, dt = 4, 32, 1.0, "f32"
        lx = rng.integers(8, 33, N)
        ly = rng.integers(2, 11, N)
    elif idx == 2:
        N, V, sigma, dt = 32, 1024, 2.0, "f32"
        lx = rng.integers(s(100), s(250) + 1, N)
        ly = rng.integers(s(20), s(80) + 1, N)
    elif idx == 3:
        N, V, sigma, dt = 16, 4096, 1.0, "f16"
        lx = rng.integers(s(150), s(300) + 1, N)
        ly = rng.integers(s(40), s(120) + 1, N)
    elif idx == 4:
        N, V, sigma, dt = 64, 512, 1.0, "f32"
        lx = np.clip(np.round(rng.lognormal(math.log(120 * scale), 0.6, N)), 1, s(600)).astype(np.int64)
        ly = np.clip(np.round(rng.lognormal(math.log(max(30 * scale, 1.0)), 0.7, N)), 0, lx).astype(np.int64)
        ly[3] = 0          # forced: a sequence with no labels
        lx[7] = 1          # forced: a single-frame sequence
        ly[7] = min(ly[7], 1)
    elif idx == 5:
        N, V, sigma, dt = 4, 128, 1.5, "f32"
        lx = rng.integers(s(1000), s(1500) + 1, N)
        ly = rng.integers(s(200), s(400) + 1, N)
    else:
        raise ValueError(idx)
    lx = lx.astype(np.int32)
    ly = ly.astype(np.int32)
    Umax = int(ly.max())
    yp = np.zeros((N, max(Umax, 1)), dtype=np.int32)
    cat = []
    for n in range(N):
        lab = rng.integers(1, V, int(ly[n])).astype(np.int32)
        yp[n, : ly[n]] = lab
        cat.append(lab)
    yc = np.concatenate(cat) if cat else np.zeros(0, dtype=np.int32)
    yp = yp[:, :Umax] if Umax > 0 else yp[:, :0]
    R = int((lx.astype(np.int64) * (ly.astype(np.int64) + 1)).sum())
    return dict(N=N, V=V, lx=lx, ly=ly, y_padded=yp, y_cat=yc, sigma=sigma, dtype=dt, R=R, idx=idx)


def make_logits(cfg, seed=None):
    """float32 (or float16 for config 3) compact logits N(0, sigma) of shape (R, V)."""
    rng = np.random.default_rng(1000 + cfg["idx"] if seed is None else seed)
    x = rng.standard_normal((cfg["R"], cfg["V"]), dtype=np.float32) * np.float32(cfg["sigma"])
    if cfg["dtype"] == "f16":
        x = x.astype(np.float16)
    return x
