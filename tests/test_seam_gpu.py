"""The reference's extension-module seam, executed: an autograd node written against
`_cwarp_rnnt_forward`, `_cwarp_rnnt_loss` and `_cwarp_rnnt_backward` (cwarp_cuda.cpp:138-153, the
three calls of cwarp_rnnt/__init__.py:14,20,27) runs on `cwarp_rnnt._C` and is compared with the
float64 oracle: costs, the (R,2) gradient record, the (R,V) gradient, and the padded alphas / betas
the forward call returns."""
import numpy as np
import pytest
import torch

from oracle import rnnt_oracle as orc
from test_parity_gpu import GRAD_ATOL, LOSS_RTOL, make_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _SeamLoss(torch.autograd.Function):
    """What a maintainer of the reference's Python layer keeps: one node, three native calls."""

    @staticmethod
    def forward(ctx, log_probs, frames, labels, label_counts, blank, keep):
        import cwarp_rnnt._C as core
        if not log_probs.requires_grad:
            return core._cwarp_rnnt_loss(log_probs, frames, labels, label_counts, blank)
        costs, grads, alphas, betas = core._cwarp_rnnt_forward(log_probs, frames, labels, label_counts, blank)
        keep.update(grads=grads, alphas=alphas, betas=betas)
        ctx.save_for_backward(grads, labels, frames, label_counts)
        ctx.extra = (blank, log_probs.size(-1))
        return costs

    @staticmethod
    def backward(ctx, grad_costs):
        import cwarp_rnnt._C as core
        grads, labels, frames, label_counts = ctx.saved_tensors
        blank, vocab = ctx.extra
        gx = core._cwarp_rnnt_backward(grads, grad_costs.contiguous(), labels, frames, label_counts, blank, vocab)
        return gx, None, None, None, None, None


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("lx,ly", [([9, 5, 12, 1], [3, 0, 7, 4]), ([40, 150, 33], [70, 130, 2])])
def test_reference_seam_runs_and_matches_the_oracle(dtype, lx, ly):
    b = make_batch(lx, ly, 24, seed=21, dtype=dtype, normalised=True)
    tdt = torch.float32 if dtype == "f32" else torch.float64
    x = b["x"].to(DEV).requires_grad_(True)
    lxd, lyd = torch.from_numpy(b["lx"]).to(DEV), torch.from_numpy(b["ly"]).to(DEV)
    ys = torch.from_numpy(b["yp"]).to(DEV)
    N, Tmax, Umax = b["N"], int(max(lx)), int(max(ly))
    w = np.random.default_rng(3).uniform(-1.5, 1.5, N)
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "logprob", grad_out=w)

    keep = {}
    costs = _SeamLoss.apply(x, lxd, ys, lyd, 0, keep)
    assert costs.dtype == tdt and costs.shape == (N,)
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    # (costs, grads, alphas, betas) as cwarp_cuda_rnnt_kernel.cu:383-384,496 returns them
    assert keep["grads"].dtype == tdt and keep["grads"].shape == (b["R"], 2)
    np.testing.assert_allclose(keep["grads"].cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
    for name, table in (("alphas", ref["alphas"]), ("betas", ref["betas"])):
        got = keep[name]
        assert got.dtype == tdt and got.shape == (N, Tmax, Umax + 1)
        got = got.cpu().numpy()
        for n in range(N):
            T, U = int(lx[n]), int(ly[n])
            tol = 1e-4 + 2e-6 * (T + U)
            np.testing.assert_allclose(got[n, :T, :U + 1], table[n], rtol=0, atol=tol * max(1.0, np.abs(table[n]).max() * 1e-2))
            assert not got[n, T:].any() and not got[n, :, U + 1:].any()   # zero outside the sequence's lattice

    wt = torch.from_numpy(w).to(DEV).to(tdt)
    (costs * wt).sum().backward(retain_graph=True)
    g1 = x.grad.clone()
    np.testing.assert_allclose(g1.cpu().numpy(), ref["grad"], rtol=0, atol=GRAD_ATOL)
    # the saved record is not rescaled in place: a second backward gives the same gradient again
    x.grad = None
    (costs * wt).sum().backward()
    assert torch.equal(x.grad, g1)

    # no-grad dispatch: the beta-only call
    with torch.no_grad():
        c2 = _SeamLoss.apply(x.detach(), lxd, ys, lyd, 0, {})
    np.testing.assert_allclose(c2.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)


def test_reference_seam_without_the_lattice_never_synchronises_for_it():
    import cwarp_rnnt._C as core
    b = make_batch([6, 3], [2, 1], 8, seed=1, normalised=True)
    x = b["x"].to(DEV)
    lxd, lyd = torch.from_numpy(b["lx"]).to(DEV), torch.from_numpy(b["ly"]).to(DEV)
    ys = torch.from_numpy(b["yp"]).to(DEV)
    try:
        core.RETURN_LATTICE = False
        costs, grads, alphas, betas = core._cwarp_rnnt_forward(x, lxd, ys, lyd, 0)
    finally:
        core.RETURN_LATTICE = True
    assert alphas is None and betas is None
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "logprob", want_dense=False)
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
