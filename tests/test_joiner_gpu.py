"""GPU parity of the compact joiner front (cwr_join / cwr_join_backward) against the float64 oracle
on the same seeded inputs, and against the padded route a caller of the reference would take
(broadcast sum over the padded (N,T,U+1,H) array, then the pack op).

Without an activation and with relu the forward pass only adds and selects: bit-exact against the
same arithmetic done by torch in the storage type.  tanh is evaluated in fp32 with a hardware
exponential: absolute tolerance 5e-7 in fp32.  The backward sums run in fp32 (fp64 for fp64
storage) over up to T or U+1 terms: tolerance 2e-6 per unit of gradient times the term count, and
one rounding of the storage type for 16-bit storage.  The reference repository has no joiner, so
there is no reference fixture for this op.
"""
import numpy as np
import pytest
import torch

from compactwarprnntloss_amd import workloads as wl
from oracle import rnnt_oracle as orc
from test_parity_gpu import TORCH_DT

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROUND = {"f32": 6e-8, "f16": 5e-4, "bf16": 4e-3, "f64": 1e-15}


def _pkg():
    import compactwarprnntloss_amd as pkg
    return pkg


def _inputs(lx, ly, H, dtype, seed, t_extra=0, u_extra=0):
    rng = np.random.default_rng(seed)
    lx, ly = np.asarray(lx, dtype=np.int32), np.asarray(ly, dtype=np.int32)
    N, Tp, Up = len(lx), int(lx.max()) + t_extra, int(ly.max()) + 1 + u_extra
    f = torch.from_numpy(rng.normal(size=(N, Tp, H))).to(TORCH_DT[dtype])
    g = torch.from_numpy(rng.normal(size=(N, Up, H))).to(TORCH_DT[dtype])
    return lx, ly, f, g


CASES = [
    ([5, 3, 7], [2, 4, 0], 32),            # ragged, one sequence without labels
    ([1, 9], [6, 1], 10),                  # rows off the 16-byte grid: element-wise path
    ([20, 11, 1, 8], [7, 3, 9, 0], 512),   # two column blocks per row in fp32
    ([6, 4], [3, 5], 1100),                # more than one block of 256 packs, ragged tail
]


@pytest.mark.parametrize("act", [None, "tanh", "relu"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("lx,ly,H", CASES)
def test_join_forward_and_backward_match_oracle(lx, ly, H, dtype, act):
    pkg = _pkg()
    lx, ly, f, g = _inputs(lx, ly, H, dtype, seed=H + len(lx), t_extra=2, u_extra=1)
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    h = pkg.compact_join(fd, gd, lxd, lyd, act)
    f64, g64 = f.double().numpy(), g.double().numpy()
    ref = orc.join_rows(f64, g64, lx, ly, act)
    assert h.shape == ref.shape and h.dtype == f.dtype
    got = h.detach().double().cpu().numpy()
    tol = ROUND[dtype] * 4 + (5e-7 if act == "tanh" and dtype == "f32" else 0)
    np.testing.assert_allclose(got, ref, rtol=ROUND[dtype] * 2, atol=tol)

    rng = np.random.default_rng(3)
    dh = torch.from_numpy(rng.normal(size=ref.shape)).to(TORCH_DT[dtype])
    h.backward(dh.to(DEV))
    # the device takes act' from its own stored (rounded) output: hand the oracle the same dh
    df_ref, dg_ref = orc.join_rows_backward(dh.double().numpy(), f64, g64, lx, ly, act)
    terms = max(int(lx.max()), int(ly.max()) + 1)
    atol = (2e-6 if dtype != "f64" else 1e-13) * terms + ROUND[dtype] * 8 * np.sqrt(terms) * (3 if act == "tanh" else 1)
    np.testing.assert_allclose(fd.grad.double().cpu().numpy(), df_ref, rtol=ROUND[dtype] * 4, atol=atol)
    np.testing.assert_allclose(gd.grad.double().cpu().numpy(), dg_ref, rtol=ROUND[dtype] * 4, atol=atol)
    # padding receives exact zeros
    for n in range(len(lx)):
        assert torch.all(fd.grad[n, lx[n]:] == 0) and torch.all(gd.grad[n, ly[n] + 1:] == 0)


@pytest.mark.parametrize("act", [None, "relu"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_join_is_bit_exact_against_the_padded_route(dtype, act):
    pkg = _pkg()
    lx, ly, f, g = _inputs([13, 2, 30], [4, 11, 6], 256, dtype, seed=9)
    fd, gd = f.to(DEV), g.to(DEV)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    z = (fd.float()[:, :, None, :] + gd.float()[:, None, :, :])
    if act == "relu":
        z = torch.relu(z)
    padded = pkg.pack_padded(z.to(fd.dtype).contiguous(), lxd, lyd)
    assert torch.equal(pkg.compact_join(fd, gd, lxd, lyd, act), padded)


def test_joiner_module_feeds_the_loss_like_the_padded_route():
    pkg = _pkg()
    torch.manual_seed(0)
    lx, ly = np.array([9, 4, 12], dtype=np.int32), np.array([3, 5, 0], dtype=np.int32)
    N, E, P, J, V = 3, 24, 16, 64, 40
    enc = torch.randn(N, int(lx.max()), E, device=DEV)
    pred = torch.randn(N, int(ly.max()) + 1, P, device=DEV)
    y = torch.randint(1, V, (N, int(ly.max())), dtype=torch.int32, device=DEV)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    joiner = pkg.CompactJoiner(E, P, J, V).to(DEV)

    loss = pkg.transducer_loss(joiner(enc, pred, lxd, lyd), lxd, y, lyd, 0, "mean", fused_log_softmax=True)
    loss.backward()
    got = [p.grad.clone() for p in joiner.parameters()]
    joiner.zero_grad()

    z = torch.tanh(joiner.enc(enc)[:, :, None, :] + joiner.pred(pred)[:, None, :, :])
    logits = pkg.pack_padded(joiner.out(z).contiguous(), lxd, lyd)
    ref = pkg.transducer_loss(logits, lxd, y, lyd, 0, "mean", fused_log_softmax=True)
    ref.backward()
    torch.testing.assert_close(loss, ref, rtol=1e-5, atol=1e-5)
    for a, p in zip(got, joiner.parameters()):
        torch.testing.assert_close(a, p.grad, rtol=1e-4, atol=2e-5)


def test_join_full_size_properties():
    """Benchmark-sized call (N=32, T~U[100,250], U~U[20,80], H=512): the compact rows equal the
    broadcast sum at sampled cells, and with unit dh the backward returns the cell counts."""
    pkg = _pkg()
    cfg = wl.make_config(2)
    lx, ly = cfg["lx"].astype(np.int32), cfg["ly"].astype(np.int32)
    N, H = len(lx), 512
    f = torch.randn(N, int(lx.max()), H, device=DEV).requires_grad_(True)
    g = torch.randn(N, int(ly.max()) + 1, H, device=DEV).requires_grad_(True)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    h = pkg.compact_join(f, g, lxd, lyd, None, total_rows=cfg["R"])
    off = orc.row_offsets_i64(lx, ly)
    rng = np.random.default_rng(0)
    for _ in range(200):
        n = int(rng.integers(N)); t = int(rng.integers(lx[n])); u = int(rng.integers(ly[n] + 1))
        r = int(off[n]) + t * (int(ly[n]) + 1) + u
        assert torch.equal(h[r], f[n, t] + g[n, u])
    h.backward(torch.ones_like(h))
    for n in (0, N // 2, N - 1):
        assert torch.all(f.grad[n, :lx[n]] == float(ly[n] + 1)) and torch.all(f.grad[n, lx[n]:] == 0)
        assert torch.all(g.grad[n, :ly[n] + 1] == float(lx[n])) and torch.all(g.grad[n, ly[n] + 1:] == 0)


def test_join_rejects_bad_arguments():
    pkg = _pkg()
    f = torch.zeros(2, 3, 8, device=DEV)
    g = torch.zeros(2, 2, 8, device=DEV)
    l = torch.ones(2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError):
        pkg.compact_join(f, g, l, l, "gelu")
    with pytest.raises(RuntimeError):
        pkg.compact_join(f, g[:, :, :4], l, l)
    with pytest.raises(RuntimeError):
        pkg.compact_join(f, g.half(), l, l)
    with pytest.raises(RuntimeError):
        pkg.compact_join(f, g, l.long(), l)


@pytest.mark.parametrize("seed", range(8))
def test_join_and_pack_random_batches(seed):
    """Random batch shapes (1 to 100 sequences, empty label sequences, rows on and off the 16-byte
    grid, padded widths wider than needed): compact_join against the oracle, and pack_padded of the
    padded broadcast sum bit-exact against compact_join."""
    pkg = _pkg()
    rng = np.random.default_rng(100 + seed)
    N = int(rng.integers(1, 101))
    lx = rng.integers(1, 14, N).astype(np.int32)
    ly = rng.integers(0, 9, N).astype(np.int32)
    H = int(rng.choice([4, 7, 24, 64, 100, 256, 260]))
    dtype = str(rng.choice(["f32", "f16", "bf16", "f64"]))
    lx_, ly_, f, g = _inputs(lx, ly, H, dtype, seed=seed, t_extra=int(rng.integers(0, 3)), u_extra=int(rng.integers(0, 3)))
    fd, gd = f.to(DEV), g.to(DEV)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    h = pkg.compact_join(fd, gd, lxd, lyd, None)
    ref = orc.join_rows(f.double().numpy(), g.double().numpy(), lx, ly, None)
    np.testing.assert_allclose(h.double().cpu().numpy(), ref, rtol=ROUND[dtype] * 2, atol=ROUND[dtype] * 4)
    acc = torch.float64 if dtype == "f64" else torch.float32
    z = (fd.to(acc)[:, :, None, :] + gd.to(acc)[:, None, :, :]).to(fd.dtype).contiguous()
    assert torch.equal(pkg.pack_padded(z, lxd, lyd), h)


def _join_fixtures():
    import os
    gdir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    return sorted(os.path.join(gdir, f) for f in os.listdir(gdir) if f.startswith("join_") and f.endswith(".npz"))


@pytest.mark.parametrize("path", _join_fixtures(), ids=lambda p: p.split("/")[-1][:-4])
def test_join_against_golden_fixtures(path):
    pkg = _pkg()
    z = np.load(path)
    act = str(z["act"])
    f = torch.from_numpy(z["f"]).to(DEV).requires_grad_(True)
    g = torch.from_numpy(z["g"]).to(DEV).requires_grad_(True)
    lx, ly = torch.from_numpy(z["lx"]).to(DEV), torch.from_numpy(z["ly"]).to(DEV)
    h = pkg.compact_join(f, g, lx, ly, None if act == "none" else act)
    np.testing.assert_allclose(h.detach().cpu().numpy(), z["h"], rtol=3e-7, atol=6e-7)
    h.backward(torch.from_numpy(z["dh"]).to(DEV))
    np.testing.assert_allclose(f.grad.cpu().numpy(), z["df"], rtol=1e-6, atol=2e-5)
    np.testing.assert_allclose(g.grad.cpu().numpy(), z["dg"], rtol=1e-6, atol=2e-5)


def test_joiner_and_loss_train_a_tiny_model():
    """End to end: a few Adam steps on random encoder / predictor features must drive the loss
    down (joiner front, library GEMMs, fused loss and all three backward passes together)."""
    pkg = _pkg()
    torch.manual_seed(1)
    lx, ly = np.array([14, 9, 20, 6], dtype=np.int32), np.array([4, 6, 3, 0], dtype=np.int32)
    N, E, P, J, V = 4, 16, 12, 32, 11
    enc = torch.randn(N, int(lx.max()), E, device=DEV)
    pred = torch.randn(N, int(ly.max()) + 1, P, device=DEV)
    y = torch.randint(1, V, (N, int(ly.max())), dtype=torch.int32, device=DEV)
    lxd, lyd = torch.from_numpy(lx).to(DEV), torch.from_numpy(ly).to(DEV)
    R = int((lx.astype(np.int64) * (ly + 1)).sum())
    joiner = pkg.CompactJoiner(E, P, J, V).to(DEV)
    opt = torch.optim.Adam(joiner.parameters(), lr=3e-2)
    losses = []
    for _ in range(40):
        opt.zero_grad()
        loss = pkg.transducer_loss(joiner(enc, pred, lxd, lyd, total_rows=R), lxd, y, lyd, 0, "mean",
                                   fused_log_softmax=True)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(np.isfinite(losses))
    assert losses[-1] < 0.5 * losses[0], losses[::8]
