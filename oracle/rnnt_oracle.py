"""CPU oracle for the compact-layout RNN-T loss and gradient (float64 NumPy).

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it; the shipped package never does.

It restates, on the CPU and in float64, the algorithm of the reference files (paths relative to
the CompactWarpRNNTLoss checkout):

  cwarp_cuda.cpp:72-77                  row offsets = exclusive cumsum of lx*(ly+1)
  cwarp_cuda_gather_kernel.cu:29-42     gather of the blank / label log-probability of each row
  cwarp_cuda_gather_kernel.cu:62-73     scatter of the (R,2) gradient back into (R,V)
  cwarp_cuda_rnnt_kernel.cu:59-125      alpha recursion
  cwarp_cuda_rnnt_kernel.cu:165-231     beta recursion
  cwarp_cuda_rnnt_kernel.cu:286-307     gradient w.r.t. the blank log-probability
  cwarp_cuda_rnnt_kernel.cu:321-331     gradient w.r.t. the label log-probability
  cwarp_cuda_rnnt_kernel.cu:345-366     cost = -beta[0][0] (+ forward/backward mismatch rule)
  cwarp_cuda_rnnt_kernel.cu:518-519     per-sequence rescale by grad_out
  cwarp_rnnt/__init__.py:66-71          reductions
  test/test.py:34-48                    definition of the compact layout (slice + concatenate)

The reference itself cannot be built or imported without CUDA, and its repository holds no golden
vectors, so every function here is pinned by what the mathematics fixes; the checks live in
tests/test_oracle_pins.py:

  row_offsets / label_offsets   closed form vs. a Python running sum; int32 result dtype
  compact_from_padded           re-pack vs. element-wise indexing
  gather                        direct indexing of x[row, blank], x[row, y[n,u]]
  alphas / betas / costs        brute-force enumeration of every alignment path; closed forms for
                                U=0, T=1 and uniform log-probs; alpha-terminal == beta[0,0];
                                an independent triple-loop restatement
  sparse_grads                  central finite differences of the brute-force loss; occupancy sums;
                                torch.autograd through an independent torch restatement
  dense gradients (both modes)  finite differences of the full function; rows sum to zero (fused
                                mode); linearity in grad_out
  join_rows / join_rows_backward  (no reference counterpart: the repository has no joiner)
                                padded broadcast sum packed by compact_from_padded; central finite
                                differences

Two gradient definitions are provided:
  mode "logprob"  x already holds log-probabilities (what the reference computes): the gradient
                  is non-zero only in the blank and label columns.
  mode "fused"    x holds raw logits; log-softmax over V is part of the function; the gradient is
                  dense: dL/dx[r,v] = softmax(x_r)[v] * gamma_r + G[r,0][v==blank] + G[r,1][v==label].
"""
from __future__ import annotations

import itertools
import math

import numpy as np

NEG_INF = -np.inf


# ---------------------------------------------------------------------------------------------
# layout
# ---------------------------------------------------------------------------------------------
def row_offsets(lx, ly):
    """Exclusive cumsum of lx*(ly+1), int32 like the reference (cwarp_cuda.cpp:72-77: int32
    product, int64 cumsum, stored back into an int32 tensor)."""
    lx = np.asarray(lx, dtype=np.int32)
    ly = np.asarray(ly, dtype=np.int32)
    prod = (lx * (ly + np.int32(1))).astype(np.int32)
    cs = np.cumsum(prod.astype(np.int64))
    off = np.zeros(lx.shape[0], dtype=np.int32)
    off[1:] = cs[:-1].astype(np.int32)
    return off


def row_offsets_i64(lx, ly):
    """N+1 exclusive offsets in int64 (entry N is the total row count)."""
    lx = np.asarray(lx, dtype=np.int64)
    ly = np.asarray(ly, dtype=np.int64)
    return np.concatenate([[0], np.cumsum(lx * (ly + 1))]).astype(np.int64)


def label_offsets_i64(ly):
    """N+1 exclusive offsets of concatenated labels (sum of ly before each sequence)."""
    ly = np.asarray(ly, dtype=np.int64)
    return np.concatenate([[0], np.cumsum(ly)]).astype(np.int64)


def compact_from_padded(xp, lx, ly):
    """(N,Tmax,Umax+1,V) -> (R,V): sequence-major, then t, then u (test/test.py:44-46)."""
    out = []
    for n in range(xp.shape[0]):
        out.append(xp[n, : lx[n], : ly[n] + 1, :].reshape(-1, xp.shape[-1]))
    return np.concatenate(out, axis=0)


def _activation(z, act):
    if act in (None, "none"):
        return z
    if act == "tanh":
        return np.tanh(z)
    if act == "relu":
        return np.maximum(z, 0.0)
    raise ValueError(act)


def join_rows(f, g, lx, ly, act=None):
    """Compact joiner front: one (H,) row act(f[n,t] + g[n,u]) per lattice cell, in the compact row
    order (test/test.py:44-46).  The reference repository has no joiner; this restates what its
    callers feed cwarp_rnnt/__init__.py:52-59 (a padded broadcast sum), restricted to valid cells.
    f: (N,Tmax,H), g: (N,Umax+1,H).  Written cell by cell; pinned against the padded broadcast sum
    packed by compact_from_padded."""
    f = np.asarray(f, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    rows = []
    for n in range(f.shape[0]):
        for t in range(int(lx[n])):
            for u in range(int(ly[n]) + 1):
                rows.append(_activation(f[n, t] + g[n, u], act))
    if not rows:
        return np.zeros((0, f.shape[-1]))
    return np.stack(rows)


def join_rows_backward(dh, f, g, lx, ly, act=None):
    """Gradient of sum(dh * join_rows(f, g)) w.r.t. f and g: dz = dh * act'(z) summed over u for f
    and over t for g, zeros in the padding.  Pinned by central finite differences."""
    f = np.asarray(f, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    dh = np.asarray(dh, dtype=np.float64)
    df, dg = np.zeros_like(f), np.zeros_like(g)
    r = 0
    for n in range(f.shape[0]):
        for t in range(int(lx[n])):
            for u in range(int(ly[n]) + 1):
                z = f[n, t] + g[n, u]
                if act == "tanh":
                    dz = dh[r] * (1.0 - np.tanh(z) ** 2)
                elif act == "relu":
                    dz = dh[r] * (z > 0)
                else:
                    dz = dh[r]
                df[n, t] += dz
                dg[n, u] += dz
                r += 1
    return df, dg


def joint_logits(h, w, bias=None):
    """Output layer of a joiner in float64: logits[r, v] = sum_k h[r, k] * w[v, k] + bias[v], for
    compact joint activations h (R, H) and a weight w (V, H) laid out as torch.nn.Linear keeps it.
    (The reference repository has no joiner; its callers feed such logits, after log_softmax, to
    cwarp_rnnt/__init__.py:32-73, test/test.py:19-20.)"""
    z = np.asarray(h, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    if bias is not None:
        z = z + np.asarray(bias, dtype=np.float64)[None, :]
    return z


def joint_backward(dlogits, h, w):
    """Backward of joint_logits: (dh (R,H), dw (V,H), dbias (V,)) for dlogits (R,V)."""
    d = np.asarray(dlogits, dtype=np.float64)
    return d @ np.asarray(w, dtype=np.float64), d.T @ np.asarray(h, dtype=np.float64), d.sum(axis=0)


def labels_of(y, ly, n):
    """Labels of sequence n from either padded (N,Umax) or concatenated (sum U,) labels."""
    y = np.asarray(y)
    if y.ndim == 2:
        return y[n, : ly[n]]
    off = label_offsets_i64(ly)
    return y[off[n] : off[n + 1]]


def gather(x, lx, y, ly, blank):
    """(R,V) -> (R,2): column 0 = x[row, blank]; column 1 = x[row, y[n,u]] for u < U_n, else 0
    (cwarp_cuda_gather_kernel.cu:29-42; output zero-initialised at :87)."""
    x = np.asarray(x)
    off = row_offsets_i64(lx, ly)
    out = np.zeros((x.shape[0], 2), dtype=x.dtype)
    for n in range(len(lx)):
        T, U = int(lx[n]), int(ly[n])
        lab = labels_of(y, ly, n)
        rows = off[n] + np.arange(T * (U + 1))
        u = np.arange(T * (U + 1)) % (U + 1)
        out[rows, 0] = x[rows, blank]
        m = u < U
        out[rows[m], 1] = x[rows[m], lab[u[m]]]
    return out


def log_softmax(x):
    x = np.asarray(x, dtype=np.float64)
    m = x.max(axis=-1, keepdims=True)
    z = x - m
    return z - np.log(np.exp(z).sum(axis=-1, keepdims=True))


# ---------------------------------------------------------------------------------------------
# lattice (one sequence; lp has shape (T, U+1, 2): [...,0]=blank, [...,1]=label)
# ---------------------------------------------------------------------------------------------
def row_lse(xs, chunk=2048):
    """float64 log-sum-exp of every row of xs (any float type), as max + log(sum(exp(x - max))).
    Walks the rows in chunks so that the float64 temporaries stay small."""
    out = np.empty(xs.shape[0])
    for i in range(0, xs.shape[0], chunk):
        c = np.asarray(xs[i : i + chunk], dtype=np.float64)
        m = c.max(axis=-1)
        out[i : i + chunk] = m + np.log(np.exp(c - m[:, None]).sum(axis=-1))
    return out


def _lse(a, b):
    """max + log1p(exp(-|a-b|)) (cwarp_cuda_rnnt_kernel.cu:22-29), float64, -inf safe."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    mx = np.maximum(a, b)
    mn = np.minimum(a, b)
    with np.errstate(invalid="ignore"):
        d = np.where(np.isneginf(mx), 0.0, mn - mx)
    return mx + np.log1p(np.exp(d))


def alphas(lp):
    """alpha[0,0]=0; alpha[0,u]=alpha[0,u-1]+L(0,u-1); alpha[t,0]=alpha[t-1,0]+B(t-1,0);
    alpha[t,u]=lse(alpha[t-1,u]+B(t-1,u), alpha[t,u-1]+L(t,u-1))
    (cwarp_cuda_rnnt_kernel.cu:59-125).  Vectorised over anti-diagonals."""
    T, Up, _ = lp.shape
    B = lp[..., 0].astype(np.float64)
    L = lp[..., 1].astype(np.float64)
    a = np.full((T, Up), NEG_INF)
    a[0, 0] = 0.0
    for k in range(1, T + Up - 1):
        u = np.arange(max(0, k - (T - 1)), min(k, Up - 1) + 1)
        t = k - u
        skip = np.full(u.shape, NEG_INF)
        emit = np.full(u.shape, NEG_INF)
        ms = t > 0
        skip[ms] = a[t[ms] - 1, u[ms]] + B[t[ms] - 1, u[ms]]
        me = u > 0
        emit[me] = a[t[me], u[me] - 1] + L[t[me], u[me] - 1]
        a[t, u] = _lse(skip, emit)
    return a


def betas(lp):
    """beta[T-1,U]=B(T-1,U); beta[T-1,u]=beta[T-1,u+1]+L(T-1,u); beta[t,U]=beta[t+1,U]+B(t,U);
    beta[t,u]=lse(beta[t+1,u]+B(t,u), beta[t,u+1]+L(t,u)) (cwarp_cuda_rnnt_kernel.cu:165-231)."""
    T, Up, _ = lp.shape
    B = lp[..., 0].astype(np.float64)
    L = lp[..., 1].astype(np.float64)
    b = np.full((T, Up), NEG_INF)
    b[T - 1, Up - 1] = B[T - 1, Up - 1]
    for k in range(T + Up - 3, -1, -1):
        u = np.arange(max(0, k - (T - 1)), min(k, Up - 1) + 1)
        t = k - u
        skip = np.full(u.shape, NEG_INF)
        emit = np.full(u.shape, NEG_INF)
        ms = t < T - 1
        skip[ms] = b[t[ms] + 1, u[ms]] + B[t[ms], u[ms]]
        me = u < Up - 1
        emit[me] = b[t[me], u[me] + 1] + L[t[me], u[me]]
        b[t, u] = _lse(skip, emit)
    return b


def sparse_grads(lp, a, b):
    """G[t,u,0] = -exp(alpha[t,u] + [t<T-1] beta[t+1,u] + B(t,u) - beta[0,0]), left 0 where
    t==T-1 and u<U (cwarp_cuda_rnnt_kernel.cu:286-307);
    G[t,u,1] = -exp(alpha[t,u] + beta[t,u+1] + L(t,u) - beta[0,0]) for u<U (:321-331)."""
    T, Up, _ = lp.shape
    B = lp[..., 0].astype(np.float64)
    L = lp[..., 1].astype(np.float64)
    G = np.zeros((T, Up, 2))
    b00 = b[0, 0]
    if T > 1:
        G[: T - 1, :, 0] = -np.exp(a[: T - 1] + b[1:] + B[: T - 1] - b00)
    G[T - 1, Up - 1, 0] = -np.exp(a[T - 1, Up - 1] + B[T - 1, Up - 1] - b00)
    if Up > 1:
        G[:, : Up - 1, 1] = -np.exp(a[:, : Up - 1] + b[:, 1:] + L[:, : Up - 1] - b00)
    return G


def cost_with_check(lp, a, b):
    """cost = -beta[0,0]; when the alpha-terminal and beta[0,0] differ by more than 0.1 % the
    reference averages them (cwarp_cuda_rnnt_kernel.cu:345-366).  Returns (cost, mismatch)."""
    T, Up, _ = lp.shape
    fa = a[T - 1, Up - 1] + float(lp[T - 1, Up - 1, 0])
    fb = b[0, 0]
    with np.errstate(invalid="ignore", divide="ignore"):
        ratio = abs(fa - fb) / abs(max(fa, fb))
    mismatch = bool(ratio > 1e-3)
    if mismatch:
        fb = (fa + fb) / 2.0
    return -fb, mismatch


# ---------------------------------------------------------------------------------------------
# whole batch
# ---------------------------------------------------------------------------------------------
def loss_and_grad(x, lx, y, ly, blank=0, mode="logprob", grad_out=None, want_dense=True):
    """Full restatement of forward + backward on a compact batch.

    Returns dict(costs (N,), gathered (R,2) log-probs, G (R,2) unscaled sparse gradient,
    lse (R,) [fused mode], grad (R,V) dense gradient scaled by grad_out [if want_dense],
    alphas / betas: lists of (T,U+1) arrays, mismatch (N,) bool).
    """
    x = np.asarray(x)
    N = len(lx)
    R, V = x.shape
    off = row_offsets_i64(lx, ly)
    assert off[-1] == R, "sum of lx*(ly+1) must equal the number of rows"
    if grad_out is None:
        grad_out = np.ones(N)
    grad_out = np.asarray(grad_out, dtype=np.float64)

    costs = np.zeros(N)
    mism = np.zeros(N, dtype=bool)
    Gall = np.zeros((R, 2))
    gathered = np.zeros((R, 2))
    lse_all = np.zeros(R) if mode == "fused" else None
    grad = np.zeros((R, V)) if want_dense else None
    A, Bt = [], []
    for n in range(N):
        T, U = int(lx[n]), int(ly[n])
        Up = U + 1
        lab = np.asarray(labels_of(y, ly, n), dtype=np.int64)
        xs = np.asarray(x[off[n] : off[n + 1]])  # storage type; widened to float64 where it is used
        if mode == "fused":
            lse = row_lse(xs)
            lse_all[off[n] : off[n + 1]] = lse
        else:
            lse = np.zeros(xs.shape[0])
        u_of_row = np.arange(T * Up) % Up
        lp = np.zeros((T * Up, 2))
        lp[:, 0] = xs[:, blank].astype(np.float64) - lse
        ml = u_of_row < U
        lp[ml, 1] = xs[ml, lab[u_of_row[ml]]].astype(np.float64) - lse[ml]
        gathered[off[n] : off[n + 1]] = lp
        lp3 = lp.reshape(T, Up, 2)
        a = alphas(lp3)
        b = betas(lp3)
        c, mm = cost_with_check(lp3, a, b)
        costs[n] = c
        mism[n] = mm
        G = sparse_grads(lp3, a, b).reshape(T * Up, 2)
        Gall[off[n] : off[n + 1]] = G
        A.append(a)
        Bt.append(b)
        if want_dense:
            g = grad[off[n] : off[n + 1]]
            rows = np.arange(T * Up)
            if mode == "fused":
                gamma = -(G[:, 0] + G[:, 1])
                g[:] = np.exp(xs.astype(np.float64) - lse[:, None]) * gamma[:, None]
                g[rows, blank] += G[:, 0]
                np.add.at(g, (rows[ml], lab[u_of_row[ml]]), G[ml, 1])
            else:
                # reference scatter: blank first, then the label column overwrites
                # (cwarp_cuda_gather_kernel.cu:70-73)
                g[rows, blank] = G[:, 0]
                g[rows[ml], lab[u_of_row[ml]]] = G[ml, 1]
            g *= grad_out[n]
    return dict(costs=costs, gathered=gathered, G=Gall, lse=lse_all, grad=grad,
                alphas=A, betas=Bt, mismatch=mism, row_off=off)


def reduce_costs(costs, reduction):
    """cwarp_rnnt/__init__.py:66-71."""
    if reduction == "mean":
        return costs.mean()
    if reduction == "sum":
        return costs.sum()
    if reduction == "none" or reduction is None:
        return costs
    raise ValueError(reduction)


# ---------------------------------------------------------------------------------------------
# independent checks used to pin the functions above (small inputs only)
# ---------------------------------------------------------------------------------------------
def brute_force_cost(lp):
    """-log of the sum over every monotone alignment path of exp(sum of its log-probs).
    A path makes T-1 blank moves (t -> t+1) and U label moves (u -> u+1) in any order from (0,0)
    to (T-1,U) and ends with the final blank at (T-1,U)."""
    T, Up, _ = lp.shape
    U = Up - 1
    total = []
    for labels_at in itertools.combinations(range(T - 1 + U), U):
        labels_at = set(labels_at)
        t = u = 0
        s = 0.0
        for i in range(T - 1 + U):
            if i in labels_at:
                s += float(lp[t, u, 1])
                u += 1
            else:
                s += float(lp[t, u, 0])
                t += 1
        s += float(lp[T - 1, U, 0])
        total.append(s)
    total = np.array(total)
    m = total.max()
    return -(m + math.log(np.exp(total - m).sum()))


def loops_alpha_beta(lp):
    """Plain triple-loop alpha/beta (no vectorisation), math.log/exp only."""
    T, Up, _ = lp.shape

    def lse(p, q):
        if p == NEG_INF:
            return q
        if q == NEG_INF:
            return p
        m = max(p, q)
        return m + math.log(math.exp(p - m) + math.exp(q - m))

    a = [[NEG_INF] * Up for _ in range(T)]
    b = [[NEG_INF] * Up for _ in range(T)]
    for t in range(T):
        for u in range(Up):
            if t == 0 and u == 0:
                a[t][u] = 0.0
                continue
            p = a[t - 1][u] + float(lp[t - 1, u, 0]) if t > 0 else NEG_INF
            q = a[t][u - 1] + float(lp[t, u - 1, 1]) if u > 0 else NEG_INF
            a[t][u] = lse(p, q)
    for t in range(T - 1, -1, -1):
        for u in range(Up - 1, -1, -1):
            if t == T - 1 and u == Up - 1:
                b[t][u] = float(lp[t, u, 0])
                continue
            p = b[t + 1][u] + float(lp[t, u, 0]) if t < T - 1 else NEG_INF
            q = b[t][u + 1] + float(lp[t, u, 1]) if u < Up - 1 else NEG_INF
            b[t][u] = lse(p, q)
    return np.array(a), np.array(b)


def uniform_cost(T, U, V):
    """Closed form when every log-prob equals -log V:
    (T+U) log V - log C(T+U-1, U)."""
    return (T + U) * math.log(V) - math.log(math.comb(T + U - 1, U))
