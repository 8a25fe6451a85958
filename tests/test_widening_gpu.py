"""GPU parity of what sits either side of the loss path: alpha / beta export, the padded -> compact
pack op with its backward, the 4-D input branch of transducer_loss, and the warp_rnnt-style front
end.  All through the C ABI, against the float64 oracle on the same seeded inputs.

Pack / unpack move bytes: bit-exact.  Lattice values: natural logs, absolute tolerance growing
with the number of recursion steps (the device carries fp32-rounded log-probs).  FastEmit has no
counterpart inside the reference repository (it belongs to the external warp_rnnt): it is checked
against its definition, a (1 + lambda) weight on the label gradient, and is otherwise
"parity unpinned".
"""
import numpy as np
import pytest
import torch

from oracle import rnnt_oracle as orc
from test_parity_gpu import GRAD_ATOL, LOSS_RTOL, TORCH_DT, make_batch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _pkg():
    import compactwarprnntloss_amd as pkg
    return pkg


def _lp_of(b, n, fused):
    """(T, U+1, 2) float64 log-probs of sequence n, as the oracle's lattice routines take them."""
    x = orc.log_softmax(b["x_ref"]) if fused else b["x_ref"]
    g = orc.gather(x, b["lx"], b["yp"], b["ly"], b["blank"])
    off = orc.row_offsets_i64(b["lx"], b["ly"])
    T, U = int(b["lx"][n]), int(b["ly"][n])
    return g[off[n]:off[n + 1]].reshape(T, U + 1, 2)


# ----------------------------------------------------------------------------- alpha / beta export
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("lx,ly,sigma", [
    ([9, 5, 12, 1], [3, 0, 7, 4], 1.0),          # small, ragged, U=0 and T=1
    ([40, 150], [70, 130], 1.0),                 # one and two strips of 128 labels
    ([30, 7, 20], [20, 600, 300], 1.0),          # five and three strips, walked concurrently
    ([6, 9], [1100, 40], 1.0),                   # nine strips, walked concurrently by sixteen waves
    ([3, 5], [2100, 10], 1.0),                   # seventeen strips: the sequential log-domain walk
    ([60, 33], [25, 64], 40.0),                  # steep logits: the per-sequence log-domain walk
])
def test_alpha_beta_export_matches_oracle(fused, lx, ly, sigma):
    pkg = _pkg()
    b = make_batch(lx, ly, 24, seed=5, sigma=sigma, normalised=not fused)
    xs = b["x"].to(DEV)
    lxd, lyd = torch.from_numpy(b["lx"]).to(DEV), torch.from_numpy(b["ly"]).to(DEV)
    ys = torch.from_numpy(b["yp"]).to(DEV)
    costs, st = pkg.rnnt_forward(xs, lxd, ys, lyd, b["blank"], fused)
    Tp, Up = int(max(lx)) + 2, int(max(ly)) + 3     # padded widths need not be tight
    alphas, betas = pkg.lattice_state(st, lxd, lyd, Tp, Up)
    alphas, betas = alphas.cpu().numpy(), betas.cpu().numpy()
    assert int(st.status[0].item()) & ~8 == 0
    for n in range(b["N"]):
        T, U = int(lx[n]), int(ly[n])
        lp = _lp_of(b, n, fused)
        a_ref, b_ref = orc.alphas(lp), orc.betas(lp)
        tol = 1e-4 + 2e-6 * (T + U) * max(1.0, sigma)
        np.testing.assert_allclose(alphas[n, :T, :U + 1], a_ref, rtol=1e-6, atol=tol)
        np.testing.assert_allclose(betas[n, :T, :U + 1], b_ref, rtol=1e-6, atol=tol)
        # zero outside the sequence's own lattice, as the reference's zero-initialised tensors
        assert not alphas[n, T:].any() and not alphas[n, :, U + 1:].any()
        assert not betas[n, T:].any() and not betas[n, :, U + 1:].any()
        # the identity the reference checks on the device: alpha-terminal + blank == beta[0,0]
        assert abs(alphas[n, T - 1, U] + lp[T - 1, U, 0] - betas[n, 0, 0]) < 10 * tol


def test_beta_export_after_loss_only_call():
    pkg = _pkg()
    b = make_batch([20, 33], [10, 70], 16, seed=8)
    xs = b["x"].to(DEV)
    lxd, lyd = torch.from_numpy(b["lx"]).to(DEV), torch.from_numpy(b["ly"]).to(DEV)
    ys = torch.from_numpy(b["yp"]).to(DEV)
    costs, st = pkg.rnnt_forward(xs, lxd, ys, lyd, 0, True, with_grad=False)
    _, betas = pkg.lattice_state(st, lxd, lyd, 33, 71, with_alpha=False)
    betas = betas.cpu().numpy()
    for n in range(2):
        T, U = int(b["lx"][n]), int(b["ly"][n])
        np.testing.assert_allclose(betas[n, :T, :U + 1], orc.betas(_lp_of(b, n, True)), rtol=1e-6, atol=3e-4)
        np.testing.assert_allclose(-betas[n, 0, 0], costs[n].item(), rtol=1e-6)


# ----------------------------------------------------------------------------- pack / unpack
def _padded(lx, ly, V, dtype, seed, t_extra=0, u_extra=0):
    rng = np.random.default_rng(seed)
    N, T, Up = len(lx), int(max(lx)) + t_extra, int(max(ly)) + 1 + u_extra
    x = rng.standard_normal((N, T, Up, V)).astype(np.float32)
    return torch.from_numpy(x).to(TORCH_DT[dtype])


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("V", [1, 7, 64, 260])    # rows of 16-byte multiples and not
def test_pack_is_bit_exact_and_unpack_is_its_transpose(dtype, V):
    pkg = _pkg()
    lx = np.array([5, 1, 9, 3], np.int32)
    ly = np.array([2, 4, 0, 4], np.int32)
    xp = _padded(lx, ly, V, dtype, seed=V, t_extra=1, u_extra=2)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    xd = xp.to(DEV)
    xc = pkg.pack_padded(xd, lxd, lyd)
    raw = xp.view(torch.int16).numpy() if dtype == "bf16" else xp.numpy()   # numpy has no bfloat16
    ref = orc.compact_from_padded(raw, lx, ly)
    got = xc.cpu()
    got = got.view(torch.int16).numpy() if dtype == "bf16" else got.numpy()
    assert got.shape == ref.shape and np.array_equal(got.view(np.uint8), ref.view(np.uint8))
    # total_rows given by the caller: no read-back, same result
    xc2 = pkg.pack_padded(xd, lxd, lyd, total_rows=int((lx * (ly + 1)).sum()))
    assert torch.equal(xc2.view(torch.uint8), xc.view(torch.uint8))
    # backward = scatter into zeros
    xg = xd.clone().requires_grad_(True)
    w = torch.randn(xc.shape, device=DEV).to(xc.dtype)
    (pkg.pack_padded(xg, lxd, lyd).float() * w.float()).sum().backward()
    want = torch.zeros_like(xp, dtype=torch.float32)
    wc = w.float().cpu()
    off = orc.row_offsets_i64(lx, ly)
    for n in range(len(lx)):
        want[n, :lx[n], :ly[n] + 1] = wc[off[n]:off[n + 1]].view(int(lx[n]), int(ly[n]) + 1, V)
    assert torch.equal(xg.grad.float().cpu(), want)


def test_pack_flags_a_sequence_that_does_not_fit_the_padded_tensor():
    pkg = _pkg()
    lib = pkg._lib.load()
    lx = torch.tensor([4, 6], dtype=torch.int32, device=DEV)
    ly = torch.tensor([2, 1], dtype=torch.int32, device=DEV)
    R = 4 * 3 + 6 * 2
    row_off, status = pkg.loss._offsets(lx, ly, R)
    xp = torch.ones((2, 5, 3, 8), device=DEV)          # T_pad = 5 < 6
    out = torch.full((R, 8), -7.0, device=DEV)
    rc = lib.cwr_pack(xp.data_ptr(), 0, 2, 5, 3, 8, lx.data_ptr(), ly.data_ptr(), row_off.data_ptr(), R,
                      out.data_ptr(), status.data_ptr(), None)
    torch.cuda.synchronize()
    assert rc == 0
    assert int(status[0].item()) & 2
    # frame 5 of sequence 1 is missing from the padded tensor: its rows are zeroed, never left as they were
    assert torch.all(out[: 12 + 10] == 1.0) and torch.all(out[12 + 10:] == 0.0)
    # rows that belong to no sequence (more rows than the lengths add up to) are zeroed as well
    row_off2, status2 = pkg.loss._offsets(lx, ly, R + 3)
    xp2 = torch.ones((2, 6, 3, 8), device=DEV)
    out2 = torch.full((R + 3, 8), -7.0, device=DEV)
    rc = lib.cwr_pack(xp2.data_ptr(), 0, 2, 6, 3, 8, lx.data_ptr(), ly.data_ptr(), row_off2.data_ptr(), R + 3,
                      out2.data_ptr(), status2.data_ptr(), None)
    torch.cuda.synchronize()
    assert rc == 0 and int(status2[0].item()) & 1
    assert torch.all(out2[:R] == 1.0) and torch.all(out2[R:] == 0.0)
    with pytest.raises(RuntimeError):
        pkg.pack_padded(xp, lx, ly, total_rows=R, validate=True)
    # the joiner front end behaves the same way
    f = torch.ones((2, 5, 16), device=DEV)
    g = torch.ones((2, 3, 16), device=DEV)
    h = pkg.compact_join(f, g, lx, ly, None, total_rows=R)
    assert torch.all(h[: 12 + 10] == 2.0) and torch.all(h[12 + 10:] == 0.0)
    with pytest.raises(RuntimeError):
        pkg.compact_join(f, g, lx, ly, "tanh", total_rows=R, validate=True)


@pytest.mark.parametrize("fused", [True, False])
def test_four_dim_input_equals_compact_input(fused):
    import cwarp_rnnt
    lx = np.array([11, 6, 14], np.int32)
    ly = np.array([4, 7, 2], np.int32)
    b = make_batch(lx, ly, 20, seed=3, normalised=not fused)
    N, T, Up, V = 3, 14, 8, 20
    xp = torch.zeros((N, T, Up, V))
    off = orc.row_offsets_i64(lx, ly)
    for n in range(N):
        xp[n, :lx[n], :ly[n] + 1] = b["x"][off[n]:off[n + 1]].view(int(lx[n]), int(ly[n]) + 1, V)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    ys = torch.from_numpy(b["yp"]).to(DEV)
    xc = b["x"].to(DEV).requires_grad_(True)
    x4 = xp.to(DEV).requires_grad_(True)
    l2 = cwarp_rnnt.transducer_loss(xc, lxd, ys, lyd, 0, "sum", fused_log_softmax=fused)
    with pytest.warns(UserWarning):
        l4 = cwarp_rnnt.transducer_loss(x4, lxd, ys, lyd, 0, "sum", fused_log_softmax=fused)
    l2.backward()
    l4.backward()
    assert torch.equal(l2, l4)
    g4 = x4.grad.cpu()
    for n in range(N):
        assert torch.equal(g4[n, :lx[n], :ly[n] + 1].reshape(-1, V), xc.grad[off[n]:off[n + 1]].cpu())
        assert not g4[n, lx[n]:].any() and not g4[n, :, ly[n] + 1:].any()
    ref = orc.loss_and_grad(b["x_ref"], lx, b["yp"], ly, 0, "fused" if fused else "logprob")
    np.testing.assert_allclose(l4.item(), ref["costs"].sum(), rtol=LOSS_RTOL)


# ----------------------------------------------------------------------------- warp_rnnt-style front end
@pytest.mark.parametrize("reduction", [None, "mean", "sum"])
@pytest.mark.parametrize("average_frames", [False, True])
@pytest.mark.parametrize("compact", [False, True])
def test_rnnt_loss_front_end(reduction, average_frames, compact):
    pkg = _pkg()
    lx = np.array([10, 7, 13, 4], np.int32)
    ly = np.array([3, 5, 0, 4], np.int32)
    b = make_batch(lx, ly, 18, seed=21, normalised=True)
    off = orc.row_offsets_i64(lx, ly)
    lxd, lyd = torch.from_numpy(lx).to(DEV).long(), torch.from_numpy(ly).to(DEV).long()   # int64 as warp_rnnt users pass
    if compact:
        x = b["x"].to(DEV).requires_grad_(True)
        labels = torch.from_numpy(b["yc"]).to(DEV)
    else:
        xp = torch.zeros((4, 13, 6, 18))
        for n in range(4):
            xp[n, :lx[n], :ly[n] + 1] = b["x"][off[n]:off[n + 1]].view(int(lx[n]), int(ly[n]) + 1, 18)
        x = xp.to(DEV).requires_grad_(True)
        labels = torch.from_numpy(b["yp"]).to(DEV).long()
    out = pkg.rnnt_loss(x, labels, lxd, lyd, average_frames=average_frames, reduction=reduction, blank=0,
                        compact=compact)
    w = np.ones(4)
    if average_frames:
        w = w / lx
    if reduction == "mean":
        w = w / 4
    ref = orc.loss_and_grad(b["x_ref"], lx, b["yp"], ly, 0, "logprob", grad_out=w)
    per_seq = ref["costs"] / (lx if average_frames else 1)
    want = {None: per_seq, "mean": per_seq.mean(), "sum": per_seq.sum()}[reduction]
    np.testing.assert_allclose(out.detach().cpu().numpy(), want, rtol=LOSS_RTOL)
    out.sum().backward()
    g = x.grad.cpu().double().numpy()
    if not compact:
        g = orc.compact_from_padded(g, lx, ly)
    np.testing.assert_allclose(g, ref["grad"], rtol=0, atol=GRAD_ATOL)


def test_rnnt_loss_fastemit_reweights_label_gradient_only():
    pkg = _pkg()
    lx = np.array([9, 12], np.int32)
    ly = np.array([4, 6], np.int32)
    b = make_batch(lx, ly, 15, seed=4, normalised=True)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    labels = torch.from_numpy(b["yc"]).to(DEV)
    lam = 0.25
    grads, costs = [], []
    for lm in (0.0, lam):
        x = b["x"].to(DEV).requires_grad_(True)
        c = pkg.rnnt_loss(x, labels, lxd, lyd, reduction="sum", compact=True, fastemit_lambda=lm)
        c.backward()
        grads.append(x.grad.cpu().double().numpy())
        costs.append(c.item())
    assert costs[0] == costs[1]                     # the loss value is not changed
    ref = orc.loss_and_grad(b["x_ref"], lx, b["yp"], ly, 0, "logprob")
    G = ref["G"].copy()
    G[:, 1] *= 1.0 + lam
    off = orc.row_offsets_i64(lx, ly)
    want = np.zeros_like(ref["grad"])
    for n in range(2):
        T, U = int(lx[n]), int(ly[n])
        rows = off[n] + np.arange(T * (U + 1))
        u = np.arange(T * (U + 1)) % (U + 1)
        want[rows, 0] = G[rows, 0]
        m = u < U
        want[rows[m], b["yp"][n][u[m]]] = G[rows[m], 1]
    np.testing.assert_allclose(grads[1], want, rtol=0, atol=GRAD_ATOL)
    np.testing.assert_allclose(grads[0], ref["grad"], rtol=0, atol=GRAD_ATOL)
