"""Pins the float64 NumPy oracle with checks the mathematics fixes (the reference ships no
golden vectors and cannot be built without CUDA).  Each check is chosen so that a plausible slip
(dropped term, wrong sign or index, transposed operand) fails it."""
import math

import numpy as np
import pytest
import torch

from compactwarprnntloss_amd import workloads as wl
from oracle import rnnt_oracle as orc


def rand_lp(rng, T, U, V=5, normalised=True):
    """Random per-sequence (T,U+1,2) log-probs taken from a real softmax over V symbols."""
    x = rng.standard_normal((T, U + 1, V))
    lpv = orc.log_softmax(x) if normalised else x
    y = rng.integers(1, V, U)
    lp = np.zeros((T, U + 1, 2))
    lp[..., 0] = lpv[..., 0]
    for u in range(U):
        lp[:, u, 1] = lpv[:, u, y[u]]
    return lp


# ----------------------------------------------------------------------------- layout
def test_row_offsets_closed_form_and_dtype():
    rng = np.random.default_rng(0)
    for _ in range(20):
        N = int(rng.integers(1, 40))
        lx = rng.integers(1, 300, N).astype(np.int32)
        ly = rng.integers(0, 90, N).astype(np.int32)
        off = orc.row_offsets(lx, ly)
        assert off.dtype == np.int32 and off.shape == (N,)
        run = 0
        for n in range(N):
            assert off[n] == run
            run += int(lx[n]) * (int(ly[n]) + 1)
        off64 = orc.row_offsets_i64(lx, ly)
        assert off64.dtype == np.int64 and off64[-1] == run
        assert np.array_equal(off64[:-1], off.astype(np.int64))
        lo = orc.label_offsets_i64(ly)
        assert lo[-1] == int(ly.astype(np.int64).sum()) and lo[0] == 0
        assert np.array_equal(np.diff(lo), ly.astype(np.int64))


def test_compact_layout_is_slice_and_concatenate():
    rng = np.random.default_rng(1)
    N, T, Up, V = 3, 6, 5, 4
    xp = rng.standard_normal((N, T, Up, V))
    lx = np.array([6, 2, 4], dtype=np.int32)
    ly = np.array([1, 4, 0], dtype=np.int32)
    xc = orc.compact_from_padded(xp, lx, ly)
    off = orc.row_offsets_i64(lx, ly)
    assert xc.shape[0] == off[-1]
    for n in range(N):
        for t in range(lx[n]):
            for u in range(ly[n] + 1):
                r = off[n] + t * (ly[n] + 1) + u
                assert np.array_equal(xc[r], xp[n, t, u])


def test_gather_is_direct_indexing_2d_and_1d_labels():
    rng = np.random.default_rng(2)
    lx = np.array([3, 5, 1, 4], dtype=np.int32)
    ly = np.array([2, 0, 3, 1], dtype=np.int32)
    V, blank = 7, 2
    R = int(orc.row_offsets_i64(lx, ly)[-1])
    x = rng.standard_normal((R, V))
    yp = rng.integers(0, V, (4, 3)).astype(np.int32)
    yc = np.concatenate([yp[n, : ly[n]] for n in range(4)])
    g2 = orc.gather(x, lx, yp, ly, blank)
    g1 = orc.gather(x, lx, yc, ly, blank)
    assert np.array_equal(g1, g2)
    off = orc.row_offsets_i64(lx, ly)
    for n in range(4):
        for t in range(lx[n]):
            for u in range(ly[n] + 1):
                r = off[n] + t * (ly[n] + 1) + u
                assert g2[r, 0] == x[r, blank]
                assert g2[r, 1] == (x[r, yp[n, u]] if u < ly[n] else 0.0)


# ----------------------------------------------------------------------------- lattice
@pytest.mark.parametrize("T,U", [(1, 0), (1, 3), (4, 0), (2, 1), (3, 3), (5, 2), (2, 6), (6, 5)])
def test_cost_matches_brute_force_path_enumeration(T, U):
    rng = np.random.default_rng(10 * T + U)
    for normalised in (True, False):
        lp = rand_lp(rng, T, U, normalised=normalised)
        a, b = orc.alphas(lp), orc.betas(lp)
        bf = orc.brute_force_cost(lp)
        assert -b[0, 0] == pytest.approx(bf, rel=1e-12, abs=1e-12)
        assert -(a[T - 1, U] + lp[T - 1, U, 0]) == pytest.approx(bf, rel=1e-12, abs=1e-12)
        c, mm = orc.cost_with_check(lp, a, b)
        assert not mm and c == pytest.approx(bf, rel=1e-12)


def test_closed_forms():
    rng = np.random.default_rng(3)
    # U = 0: only blanks
    lp = rand_lp(rng, 9, 0)
    assert -orc.betas(lp)[0, 0] == pytest.approx(-lp[:, 0, 0].sum(), rel=1e-13)
    # T = 1: all labels then the final blank
    lp = rand_lp(rng, 1, 6)
    assert -orc.betas(lp)[0, 0] == pytest.approx(-(lp[0, :6, 1].sum() + lp[0, 6, 0]), rel=1e-13)
    # uniform log-probs: count of paths is C(T+U-1, U)
    for T, U, V in [(7, 3, 11), (20, 20, 5), (64, 17, 1000), (3, 70, 2)]:
        lp = np.full((T, U + 1, 2), -math.log(V))
        assert -orc.betas(lp)[0, 0] == pytest.approx(orc.uniform_cost(T, U, V), rel=1e-12)
        a = orc.alphas(lp)
        assert -(a[T - 1, U] + lp[T - 1, U, 0]) == pytest.approx(orc.uniform_cost(T, U, V), rel=1e-12)


def test_vectorised_recursions_equal_plain_loops():
    rng = np.random.default_rng(4)
    for T, U in [(1, 0), (1, 5), (7, 0), (9, 4), (5, 11), (33, 17)]:
        lp = rand_lp(rng, T, U)
        a, b = orc.alphas(lp), orc.betas(lp)
        a2, b2 = orc.loops_alpha_beta(lp)
        np.testing.assert_allclose(a, a2, rtol=1e-13, atol=1e-13)
        np.testing.assert_allclose(b, b2, rtol=1e-13, atol=1e-13)


def test_mismatch_rule_averages():
    lp = np.full((2, 2, 2), -1.0)
    a, b = orc.alphas(lp), orc.betas(lp)
    b = b.copy()
    b[0, 0] *= 1.01  # 1 % apart -> averaged
    fa = a[1, 1] + lp[1, 1, 0]
    c, mm = orc.cost_with_check(lp, a, b)
    assert mm and c == pytest.approx(-(fa + b[0, 0]) / 2)


# ----------------------------------------------------------------------------- sparse gradient
def test_sparse_grads_match_finite_differences_of_brute_force():
    rng = np.random.default_rng(5)
    for T, U in [(1, 0), (1, 2), (3, 0), (3, 2), (4, 3), (2, 4)]:
        lp = rand_lp(rng, T, U, normalised=False)
        a, b = orc.alphas(lp), orc.betas(lp)
        G = orc.sparse_grads(lp, a, b)
        eps = 1e-6
        for t in range(T):
            for u in range(U + 1):
                for c in range(2):
                    p, m = lp.copy(), lp.copy()
                    p[t, u, c] += eps
                    m[t, u, c] -= eps
                    fd = (orc.brute_force_cost(p) - orc.brute_force_cost(m)) / (2 * eps)
                    assert G[t, u, c] == pytest.approx(fd, abs=2e-8), (T, U, t, u, c)
        # cells the reference leaves at zero really do not influence the loss
        if U > 0:
            assert np.all(G[T - 1, :U, 0] == 0)
            assert np.all(G[:, U, 1] == 0)


def test_occupancy_invariants():
    rng = np.random.default_rng(6)
    for T, U in [(5, 3), (17, 9), (40, 1), (3, 30), (12, 0)]:
        lp = rand_lp(rng, T, U)
        a, b = orc.alphas(lp), orc.betas(lp)
        G = orc.sparse_grads(lp, a, b)
        # every path leaves each frame with exactly one blank
        np.testing.assert_allclose(-G[..., 0].sum(axis=1), np.ones(T), rtol=1e-11)
        # every path emits each label exactly once
        if U > 0:
            np.testing.assert_allclose(-G[:, :U, 1].sum(axis=0), np.ones(U), rtol=1e-11)


def _torch_costs(lp):
    """Independent restatement in torch float64 so autograd supplies the gradient."""
    T, Up, _ = lp.shape
    ninf = torch.tensor(-float("inf"), dtype=torch.float64)
    a = [[None] * Up for _ in range(T)]
    for t in range(T):
        for u in range(Up):
            if t == 0 and u == 0:
                a[t][u] = torch.zeros((), dtype=torch.float64)
                continue
            terms = []
            if t > 0:
                terms.append(a[t - 1][u] + lp[t - 1, u, 0])
            if u > 0:
                terms.append(a[t][u - 1] + lp[t, u - 1, 1])
            a[t][u] = torch.logsumexp(torch.stack(terms), 0)
    return -(a[T - 1][Up - 1] + lp[T - 1, Up - 1, 0])


def test_sparse_grads_match_torch_autograd():
    rng = np.random.default_rng(7)
    for T, U in [(6, 4), (3, 7), (9, 1)]:
        lp = rand_lp(rng, T, U)
        lpt = torch.tensor(lp, dtype=torch.float64, requires_grad=True)
        c = _torch_costs(lpt)
        c.backward()
        a, b = orc.alphas(lp), orc.betas(lp)
        G = orc.sparse_grads(lp, a, b)
        g = lpt.grad.numpy().copy()
        g[:, U, 1] = 0  # never read
        np.testing.assert_allclose(G, g, rtol=1e-10, atol=1e-12)
        assert float(c.detach()) == pytest.approx(-b[0, 0], rel=1e-13)


# ----------------------------------------------------------------------------- whole batch
def _tiny_batch(seed, V=6, blank=0, allow_blank_label=False):
    rng = np.random.default_rng(seed)
    lx = np.array([3, 1, 4, 2], dtype=np.int32)
    ly = np.array([2, 3, 0, 2], dtype=np.int32)
    R = int(orc.row_offsets_i64(lx, ly)[-1])
    x = rng.standard_normal((R, V))
    lo = 0 if allow_blank_label else 1
    yp = rng.integers(lo, V, (4, 3)).astype(np.int32)
    if blank != 0 and not allow_blank_label:
        yp[yp == blank] = 0
    return x, lx, yp, ly


def _fd_dense(x, lx, y, ly, blank, mode, w):
    eps = 1e-6
    g = np.zeros_like(x)
    for r in range(x.shape[0]):
        for v in range(x.shape[1]):
            p, m = x.copy(), x.copy()
            p[r, v] += eps
            m[r, v] -= eps
            cp = orc.loss_and_grad(p, lx, y, ly, blank, mode, want_dense=False)["costs"]
            cm = orc.loss_and_grad(m, lx, y, ly, blank, mode, want_dense=False)["costs"]
            g[r, v] = ((cp - cm) * w).sum() / (2 * eps)
    return g


@pytest.mark.parametrize("mode", ["logprob", "fused"])
@pytest.mark.parametrize("blank", [0, 3])
def test_dense_gradient_matches_finite_differences(mode, blank):
    x, lx, y, ly = _tiny_batch(11, blank=blank)
    w = np.array([0.5, -1.25, 2.0, 1.0])
    out = orc.loss_and_grad(x, lx, y, ly, blank, mode, grad_out=w)
    fd = _fd_dense(x, lx, y, ly, blank, mode, w)
    np.testing.assert_allclose(out["grad"], fd, atol=5e-8)
    if mode == "fused":
        np.testing.assert_allclose(out["grad"].sum(axis=1), 0, atol=1e-12)
    else:
        # only the blank and label columns may be non-zero
        nz = np.abs(out["grad"]) > 0
        assert nz.sum(axis=1).max() <= 2


def test_fused_equals_logprob_mode_after_log_softmax_chain_rule():
    x, lx, y, ly = _tiny_batch(12)
    fused = orc.loss_and_grad(x, lx, y, ly, 0, "fused")
    lpx = orc.log_softmax(x)
    plain = orc.loss_and_grad(lpx, lx, y, ly, 0, "logprob")
    np.testing.assert_allclose(fused["costs"], plain["costs"], rtol=1e-12)
    np.testing.assert_allclose(fused["G"], plain["G"], rtol=1e-10, atol=1e-14)
    # chain rule of log_softmax: g - softmax * sum(g)
    g = plain["grad"]
    chained = g - np.exp(lpx) * g.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(fused["grad"], chained, atol=1e-12)


def test_linearity_in_grad_out_and_reductions():
    x, lx, y, ly = _tiny_batch(13)
    base = orc.loss_and_grad(x, lx, y, ly, 0, "fused")
    w = np.array([2.0, 0.0, -1.0, 0.25])
    sc = orc.loss_and_grad(x, lx, y, ly, 0, "fused", grad_out=w)
    off = base["row_off"]
    for n in range(4):
        np.testing.assert_allclose(sc["grad"][off[n]:off[n + 1]], base["grad"][off[n]:off[n + 1]] * w[n])
    c = base["costs"]
    assert orc.reduce_costs(c, "mean") == pytest.approx(c.sum() / 4)
    assert orc.reduce_costs(c, "sum") == pytest.approx(c.sum())
    assert orc.reduce_costs(c, None) is c and orc.reduce_costs(c, "none") is c
    with pytest.raises(ValueError):
        orc.reduce_costs(c, "avg")


def test_label_equal_to_blank_follows_reference_overwrite_in_logprob_mode():
    x, lx, y, ly = _tiny_batch(14, allow_blank_label=True)
    y[0, 0] = 0  # label == blank at u=0 of sequence 0
    out = orc.loss_and_grad(x, lx, y, ly, 0, "logprob")
    G, g = out["G"], out["grad"]
    # rows of sequence 0 with u == 0: t*(U+1)
    for t in range(3):
        r = t * 3
        assert g[r, 0] == G[r, 1]  # label value overwrote the blank value
    fused = orc.loss_and_grad(x, lx, y, ly, 0, "fused")
    np.testing.assert_allclose(fused["grad"].sum(axis=1), 0, atol=1e-12)


def test_configs_are_seeded_and_in_range():
    for idx in range(1, 6):
        c1 = wl.make_config(idx, scale=0.2 if idx != 1 else 1.0)
        c2 = wl.make_config(idx, scale=0.2 if idx != 1 else 1.0)
        assert np.array_equal(c1["lx"], c2["lx"]) and np.array_equal(c1["y_cat"], c2["y_cat"])
        assert c1["lx"].dtype == np.int32 and c1["ly"].dtype == np.int32
        assert c1["lx"].min() >= 1 and c1["ly"].min() >= 0
        if len(c1["y_cat"]):
            assert c1["y_cat"].min() >= 1 and c1["y_cat"].max() < c1["V"]
        assert c1["R"] == int((c1["lx"].astype(np.int64) * (c1["ly"] + 1)).sum())
    c4 = wl.make_config(4)
    assert c4["ly"].min() == 0 and c4["lx"].min() == 1 and c4["N"] == 64
    c2 = wl.make_config(2)
    assert c2["N"] == 32 and c2["V"] == 1024 and 100 <= c2["lx"].min() and c2["lx"].max() <= 250


# ----------------------------------------------------------------------------- joiner front
@pytest.mark.parametrize("act", [None, "tanh", "relu"])
def test_join_rows_equal_packed_broadcast_sum(act):
    rng = np.random.default_rng(11)
    lx, ly = np.array([3, 1, 5]), np.array([2, 0, 4])
    f = rng.normal(size=(3, 5, 6))
    g = rng.normal(size=(3, 5, 6))
    z = f[:, :, None, :] + g[:, None, :, :]
    full = {None: z, "tanh": np.tanh(z), "relu": np.maximum(z, 0)}[act]
    np.testing.assert_array_equal(orc.join_rows(f, g, lx, ly, act), orc.compact_from_padded(full, lx, ly))


@pytest.mark.parametrize("act", [None, "tanh", "relu"])
def test_join_rows_backward_matches_finite_differences(act):
    rng = np.random.default_rng(12)
    lx, ly = np.array([2, 3]), np.array([1, 2])
    f = rng.normal(size=(2, 4, 3))   # one padded frame / state in each array
    g = rng.normal(size=(2, 4, 3))
    R = int((lx * (ly + 1)).sum())
    dh = rng.normal(size=(R, 3))
    df, dg = orc.join_rows_backward(dh, f, g, lx, ly, act)
    fn = lambda a, b: float((dh * orc.join_rows(a, b, lx, ly, act)).sum())
    eps = 1e-6
    for arr, grad, which in ((f, df, 0), (g, dg, 1)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            p, m = arr.copy(), arr.copy()
            p[idx] += eps
            m[idx] -= eps
            num[idx] = ((fn(p, g) - fn(m, g)) if which == 0 else (fn(f, p) - fn(f, m))) / (2 * eps)
        np.testing.assert_allclose(grad, num, atol=1e-7)
    assert np.all(df[0, 2:] == 0) and np.all(dg[0, 2:] == 0)   # padding gets no gradient


def test_row_lse_matches_scipy_for_every_storage_type():
    from scipy.special import logsumexp
    rng = np.random.default_rng(3)
    for dt in (np.float16, np.float32, np.float64):
        x = (rng.standard_normal((5000, 37)) * 6).astype(dt)
        x[17] = 30000 if dt == np.float16 else 1e4   # exp would overflow without the row maximum
        np.testing.assert_allclose(orc.row_lse(x, chunk=999), logsumexp(x.astype(np.float64), axis=-1), rtol=1e-14)


def test_joint_layer_restatement_against_finite_differences_and_torch():
    """joint_logits / joint_backward (no reference counterpart): the matrix product against torch in
    float64, the backward against central finite differences of the loss of those logits."""
    import torch
    rng = np.random.default_rng(5)
    lx, ly = np.array([3, 2], np.int32), np.array([2, 1], np.int32)
    R, H, V = int(orc.row_offsets_i64(lx, ly)[-1]), 5, 7
    h, w, b = rng.standard_normal((R, H)), rng.standard_normal((V, H)), rng.standard_normal(V)
    y = np.array([[1, 3], [2, 0]], np.int32)
    z = orc.joint_logits(h, w, b)
    zt = torch.from_numpy(h) @ torch.from_numpy(w).T + torch.from_numpy(b)
    np.testing.assert_allclose(z, zt.numpy(), rtol=1e-13, atol=1e-13)
    ref = orc.loss_and_grad(z, lx, y, ly, 0, "fused")
    dh, dw, db = orc.joint_backward(ref["grad"], h, w)

    def total(hh, ww, bb):
        return orc.loss_and_grad(orc.joint_logits(hh, ww, bb), lx, y, ly, 0, "fused", want_dense=False)["costs"].sum()

    eps = 1e-6
    for arr, grad in ((h, dh), (w, dw), (b, db)):
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            keep = arr[idx]
            arr[idx] = keep + eps
            up = total(h, w, b)
            arr[idx] = keep - eps
            dn = total(h, w, b)
            arr[idx] = keep
            assert abs((up - dn) / (2 * eps) - grad[idx]) < 1e-6, (idx, (up - dn) / (2 * eps), grad[idx])


# ----------------------------------------------------------------------------- the C restatement
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("labels", ["2d", "1d"])
def test_c_restatement_agrees_with_the_numpy_oracle(fused, labels):
    """oracle/rnnt_oracle_c.c (the CPU baseline of the benchmark) against the NumPy oracle, which the
    tests above pin: random ragged batches with U = 0, T = 1, labels that equal the blank, weights of
    both signs; costs and sparse gradients to rounding of float64, dense gradients to the float32
    they are stored in."""
    from oracle import build_c
    lib = build_c.load()
    rng = np.random.default_rng(5 + fused)
    for trial in range(6):
        N = int(rng.integers(1, 7))
        lx = rng.integers(1, 14, N).astype(np.int32)
        ly = rng.integers(0, 9, N).astype(np.int32)
        if trial == 0:
            lx[0], ly[0] = 1, 0
        V = int(rng.integers(2, 20))
        blank = int(rng.integers(0, V))
        R = int((lx.astype(np.int64) * (ly + 1)).sum())
        x = (rng.standard_normal((R, V)) * 2).astype(np.float32)
        if not fused:
            x = orc.log_softmax(x).astype(np.float32)
        yp = rng.integers(0, V, (N, max(int(ly.max()), 1))).astype(np.int32)  # may equal the blank
        y = yp if labels == "2d" else np.concatenate([yp[n, : ly[n]] for n in range(N)]).astype(np.int32)
        go = rng.uniform(-1.5, 1.5, N)
        ref = orc.loss_and_grad(x.astype(np.float64), lx, y, ly, blank, "fused" if fused else "logprob", grad_out=go)
        got = build_c.loss_and_grad(lib, x, lx, y, ly, blank, fused, go)
        np.testing.assert_allclose(got["costs"], ref["costs"], rtol=1e-12)
        np.testing.assert_allclose(got["G"], ref["G"], rtol=0, atol=1e-12)
        np.testing.assert_allclose(got["grad"], ref["grad"], rtol=2e-7, atol=1e-9)
    assert lib.rnnt_oracle_c_threads() >= 1


def test_c_restatement_refuses_lengths_that_do_not_add_up():
    from oracle import build_c
    lib = build_c.load()
    x = np.zeros((5, 3), dtype=np.float32)
    with pytest.raises(RuntimeError):
        build_c.loss_and_grad(lib, x, np.array([2], np.int32), np.zeros((1, 1), np.int32), np.array([1], np.int32))
