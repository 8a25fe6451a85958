"""The fused output layer (cwr_joint_forward / cwr_joint_backward): logits = h @ W^T + bias are
multiplied on the matrix cores and reduced tile by tile, never stored.  Parity against the float64
oracle evaluated on the same 16-bit operands: `joint_logits` (a float64 matrix product) followed by
the fused-mode loss.  Tolerances: loss 1e-5 relative (fp32 accumulation of 16-bit products),
per-row quantities 1e-4 absolute."""
import numpy as np
import pytest
import torch

from oracle import rnnt_oracle as orc
from test_parity_gpu import GRAD_ATOL, LOSS_RTOL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TDT = {"bf16": torch.bfloat16, "f16": torch.float16}


def make_joint(lx, ly, H, V, seed, dtype, scale=1.0, bias=True):
    rng = np.random.default_rng(seed)
    lx, ly = np.asarray(lx, np.int32), np.asarray(ly, np.int32)
    N = len(lx)
    R = int(orc.row_offsets_i64(lx, ly)[-1])
    h = torch.from_numpy(rng.standard_normal((R, H)).astype(np.float32)).to(TDT[dtype])
    w = torch.from_numpy((rng.standard_normal((V, H)) * scale / np.sqrt(H)).astype(np.float32)).to(TDT[dtype])
    b = torch.from_numpy(rng.standard_normal(V).astype(np.float32)) if bias else None
    yp = np.zeros((N, max(int(ly.max()), 1)), np.int32)
    for n in range(N):
        yp[n, : ly[n]] = rng.integers(1, V, int(ly[n]))
    yp = yp[:, : int(ly.max())]
    return dict(lx=lx, ly=ly, yp=yp, h=h, w=w, b=b, N=N, R=R, H=H, V=V)


def reference(j, grad_out=None, want_dense=False):
    z = orc.joint_logits(j["h"].double().numpy(), j["w"].double().numpy(), None if j["b"] is None else j["b"].numpy())
    return z, orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], 0, "fused", grad_out=grad_out, want_dense=want_dense)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("lx,ly,H,V,bias", [
    ([9, 5, 12, 1], [3, 0, 7, 4], 64, 128, True),        # one vocabulary tile, one workgroup, tail rows
    ([40, 33, 17], [12, 20, 5], 96, 300, True),           # a ragged last vocabulary tile, several workgroups
    ([50, 21], [30, 70], 256, 1024, False),               # eight tiles, two strips, no bias
    ([30, 14], [9, 3], 32, 40, True),                     # fewer entries than half a tile: a wave with no valid entry
    ([61, 40], [33, 70], 512, 1000, True),                # the largest resident shape at two waves per SIMD
    ([25, 31], [20, 9], 768, 257, False),                 # one wave per SIMD, a single odd entry in the last tile
    ([33, 12], [8, 40], 128, 300, True),                  # two K-slices per vocabulary tile
    ([33, 12], [8, 40], 192, 257, False),                 # an odd number of K-slices per tile (3)
    ([20, 41], [30, 6], 320, 1024, True),                 # ... 5
    ([27, 9], [11, 25], 448, 130, True),                  # ... 7
    ([27, 9], [11, 25], 576, 515, False),                 # ... 9
    ([18, 22], [14, 9], 896, 300, True),                  # one wave per SIMD, 14 slices
    ([18, 22], [14, 9], 704, 130, False),                 # one wave per SIMD, odd numbers of slices
    ([11, 15], [9, 14], 832, 257, True),
    ([11, 15], [9, 14], 960, 64, True),
])
def test_joint_forward_matches_oracle(dtype, lx, ly, H, V, bias):
    import compactwarprnntloss_amd as pkg
    j = make_joint(lx, ly, H, V, seed=3, dtype=dtype, scale=3.0, bias=bias)
    z, ref = reference(j)
    costs, st = pkg.joint_forward(j["h"].to(DEV), j["w"].to(DEV), None if j["b"] is None else j["b"].to(DEV),
                                  torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["yp"]).to(DEV),
                                  torch.from_numpy(j["ly"]).to(DEV), 0)
    torch.cuda.synchronize()
    assert int(st.status[0].item()) == 0
    np.testing.assert_allclose(st.lse.cpu().numpy(), ref["lse"], rtol=2e-6, atol=2e-5)
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
    # the per-row record the backward pass reads
    off = orc.row_offsets_i64(j["lx"], j["ly"])
    ri = st.rowinfo.cpu().numpy()
    for n in range(j["N"]):
        T, U = int(j["lx"][n]), int(j["ly"][n])
        want_lab = np.tile(np.concatenate([j["yp"][n, :U], [-1]]), T)
        assert np.array_equal(ri[off[n]:off[n + 1], 0], want_lab)
        assert np.all(ri[off[n]:off[n + 1], 1] == n)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("lx,ly,H,V,bias,blank", [
    ([9, 5, 12, 1], [3, 0, 7, 4], 64, 128, True, 0),
    ([40, 33, 17], [12, 20, 5], 96, 300, True, 299),      # ragged last tile; the blank in it (streaming kernel)
    ([50, 21], [30, 70], 256, 1024, False, 77),           # resident kernel, two data blocks per wave
    ([50, 21], [30, 20], 512, 515, True, 130),            # resident kernel; V not a multiple of 4: element stores
    ([30, 14], [9, 3], 32, 40, True, 5),
    ([33, 12], [8, 40], 192, 257, True, 3),               # an odd number of K-slices per tile
    ([27, 9], [11, 25], 448, 130, False, 129),            # ... in the four-wave shape
    ([18, 22], [14, 9], 896, 300, True, 0),
])
def test_joint_backward_dlogits_match_oracle(dtype, lx, ly, H, V, bias, blank):
    """cwr_joint_backward through the C ABI, a block of rows at a time (blocks that end inside a
    kernel's group of rows), against the oracle's dense fused gradient of the float64 logits.
    Tolerance: the one rounding of the result to the 16-bit type (2^-8 / 2^-11 relative) plus the
    fp32 evaluation of softmax (1e-5 of the row's largest entry)."""
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd import _lib
    from compactwarprnntloss_amd.loss import _DTYPES, _stream_ptr
    j = make_joint(lx, ly, H, V, seed=4, dtype=dtype, scale=3.0, bias=bias)
    N, R = j["N"], j["R"]
    go = np.random.default_rng(2).uniform(0.5, 1.5, N)
    z = orc.joint_logits(j["h"].double().numpy(), j["w"].double().numpy(), None if j["b"] is None else j["b"].numpy())
    ref = orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], blank, "fused", grad_out=go, want_dense=True)
    h, W = j["h"].to(DEV), j["w"].to(DEV)
    b = None if j["b"] is None else j["b"].to(DEV)
    costs, st = pkg.joint_forward(h, W, b, torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["yp"]).to(DEV),
                                  torch.from_numpy(j["ly"]).to(DEV), blank)
    gc = torch.from_numpy(go).float().to(DEV)
    dz = torch.full((R, V), float("nan"), dtype=TDT[dtype], device=DEV)
    lib = _lib.load()
    block = 173
    for r0 in range(0, R, block):
        n = min(block, R - r0)
        rc = lib.cwr_joint_backward(h[r0:].data_ptr(), W.data_ptr(), b.data_ptr() if b is not None else None,
                                    _DTYPES[TDT[dtype]], n, H, V, N, blank, st.rowinfo[r0:].data_ptr(),
                                    st.grads[r0:].data_ptr(), st.lse[r0:].data_ptr(), gc.data_ptr(), 1, 1.0,
                                    dz[r0:].data_ptr(), _stream_ptr(torch.device(DEV)))
        assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    got = dz.double().cpu().numpy()
    eps = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    tol = eps * np.abs(ref["grad"]) + 2e-5 * np.abs(ref["grad"]).max(axis=1, keepdims=True) + 1e-7
    assert np.all(np.isfinite(got))
    bad = np.abs(got - ref["grad"]) > tol
    assert not bad.any(), (np.argwhere(bad)[:5], got[bad][:5], ref["grad"][bad][:5])


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_fused_joint_loss_gradients_match_oracle(dtype, reduction):
    """loss -> (dh, dW, dbias) through the autograd node, against the oracle's chain rule
    (dense fused gradient of the float64 logits, then joint_backward).  'mean' and 'sum' are the
    node's own reductions (a scalar gradient comes back and the node spreads it, with 1/N for the
    mean); 'none' weights the per-sequence costs by hand.  The backward pass forms the logits a block
    of rows at a time; a small block size makes the test cross several blocks.  Tolerance of the
    gradients: one rounding of d logits to the 16-bit type before the products."""
    import compactwarprnntloss_amd as pkg
    j = make_joint([40, 33, 17], [12, 20, 5], 96, 300 if dtype == "bf16" else 256, seed=9, dtype=dtype, scale=3.0)
    N = j["N"]
    w = np.random.default_rng(1).uniform(0.5, 1.5, N)
    c = 0.7
    go = {"mean": np.full(N, c / N), "sum": np.full(N, c), "none": w}[reduction]
    z, ref = reference(j, grad_out=go, want_dense=True)
    dh_ref, dw_ref, db_ref = orc.joint_backward(ref["grad"], j["h"].double().numpy(), j["w"].double().numpy())
    h = j["h"].to(DEV).requires_grad_(True)
    W = j["w"].to(DEV).requires_grad_(True)
    b = j["b"].to(DEV).requires_grad_(True)
    lx, ly = torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["ly"]).to(DEV)
    y = torch.from_numpy(j["yp"]).to(DEV)
    wt = torch.from_numpy(w).to(DEV).float()
    if reduction == "none":
        loss = (pkg.fused_joint_loss(h, W, b, lx, y, ly, 0, "none", chunk_rows=257) * wt).sum()
    else:
        loss = pkg.fused_joint_loss(h, W, b, lx, y, ly, 0, reduction, chunk_rows=257) * c
        _, ref0 = reference(j)
        want = ref0["costs"].mean() if reduction == "mean" else ref0["costs"].sum()
        assert abs(loss.item() / c - want) <= LOSS_RTOL * want
    loss.backward()
    torch.cuda.synchronize()
    rel = 1e-2 if dtype == "bf16" else 2e-3
    for got, want, name in ((h.grad, dh_ref, "dh"), (W.grad, dw_ref, "dW"), (b.grad, db_ref, "dbias")):
        got = got.double().cpu().numpy()
        scale = np.abs(want).max()
        np.testing.assert_allclose(got, want, rtol=rel, atol=rel * scale, err_msg=name)
    # and the value itself, with the reduction done by the node
    with torch.no_grad():
        lm = pkg.fused_joint_loss(h, W, b, lx, y, ly, 0, "mean")
    _, ref1 = reference(j)
    assert abs(float(lm) - ref1["costs"].mean()) <= LOSS_RTOL * ref1["costs"].mean()


def test_joint_forward_with_more_sequences_than_lanes():
    """More than 64 sequences: the kernels place their rows by a search through the offsets instead
    of through per-lane sequence tables."""
    import compactwarprnntloss_amd as pkg
    rng = np.random.default_rng(11)
    N = 75
    lx = rng.integers(1, 6, N)
    ly = rng.integers(0, 4, N)
    j = make_joint(lx, ly, 64, 130, seed=5, dtype="bf16", scale=2.0)
    z, ref = reference(j)
    costs, st = pkg.joint_forward(j["h"].to(DEV), j["w"].to(DEV), j["b"].to(DEV), torch.from_numpy(j["lx"]).to(DEV),
                                  torch.from_numpy(j["yp"]).to(DEV), torch.from_numpy(j["ly"]).to(DEV), 0)
    torch.cuda.synchronize()
    assert int(st.status[0].item()) == 0
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)


def test_joint_forward_keeps_the_absolute_accuracy_of_small_costs():
    """Logits of large magnitude over small vocabularies: most rows are one-hot, row maxima are ~30
    and a cost can be a few thousandths of a nat.  The running log-sum-exp of the tiles must not
    inherit the rounding of maximum * log2(e) (half an ulp of ~40 per tile, 1e-6 nat)."""
    import compactwarprnntloss_amd as pkg
    rng = np.random.default_rng(77)
    for case in range(36):
        N = 16
        lx = rng.integers(1, 6, N)
        ly = rng.integers(0, 3, N)
        V = [5, 40, 300][case % 3]                      # one tile, one tile, three tiles
        H = [96, 64, 256][(case // 3) % 3]              # the streaming kernel and two resident shapes
        j = make_joint(lx, ly, H, V, seed=int(rng.integers(1 << 30)), dtype=["f16", "bf16"][case % 2],
                       scale=8.0, bias=bool(case & 4))
        z, ref = reference(j)
        costs, st = pkg.joint_forward(j["h"].to(DEV), j["w"].to(DEV), None if j["b"] is None else j["b"].to(DEV),
                                      torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["yp"]).to(DEV),
                                      torch.from_numpy(j["ly"]).to(DEV), 0)
        torch.cuda.synchronize()
        assert int(st.status[0].item()) == 0
        np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL, atol=3e-7,
                                   err_msg=f"case {case}: V={V} H={H}")


@pytest.mark.parametrize("seed", range(4))
def test_joint_random_shapes_against_oracle(seed):
    """Fifteen random cases per seed: batch sizes on both sides of 64 sequences, joint sizes with and
    without a resident kernel, vocabularies on and off the tile and store grids, both 16-bit types,
    any blank, with and without bias, three logit scales, several block sizes of the backward pass:
    costs, per-row gradients and the dense logit gradient against the oracle."""
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd import _lib
    from compactwarprnntloss_amd.loss import _DTYPES, _stream_ptr
    lib = _lib.load()
    rng = np.random.default_rng(31000 + seed)
    for case in range(15):
        N = int(rng.integers(65, 80)) if rng.random() < 0.15 else int(rng.integers(1, 6))
        lx = rng.integers(1, 40 if N < 10 else 6, N)
        ly = rng.integers(0, 80 if (N < 10 and rng.random() < 0.3) else 12, N)
        H = int(rng.choice([32, 64, 96] + list(range(128, 1025, 64))))
        V = int(rng.choice([5, 40, 128, 130, 256, 300, 515, 1024]))
        dtype = str(rng.choice(["bf16", "f16"]))
        blank = int(rng.integers(0, V))
        scale = float(rng.choice([1.0, 3.0, 6.0]))
        j = make_joint(lx, ly, H, V, seed=1000 * seed + case, dtype=dtype, scale=scale, bias=bool(rng.integers(0, 2)))
        go = rng.uniform(0.5, 1.5, N)
        what = f"seed {seed} case {case}: N={N} H={H} V={V} {dtype} blank={blank} scale={scale} R={j['R']}"
        z = orc.joint_logits(j["h"].double().numpy(), j["w"].double().numpy(),
                             None if j["b"] is None else j["b"].numpy())
        ref = orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], blank, "fused", grad_out=go, want_dense=True)
        h, W = j["h"].to(DEV), j["w"].to(DEV)
        b = None if j["b"] is None else j["b"].to(DEV)
        costs, st = pkg.joint_forward(h, W, b, torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["yp"]).to(DEV),
                                      torch.from_numpy(j["ly"]).to(DEV), blank)
        torch.cuda.synchronize()
        assert int(st.status[0].item()) == 0, what
        # a cost of a few thousandths of a nat carries the fp32 rounding of sums next to 1: 1e-7 absolute
        np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL, atol=3e-7, err_msg=what)
        np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL, err_msg=what)
        R = j["R"]
        gc = torch.from_numpy(go).float().to(DEV)
        dz = torch.full((R, V), float("nan"), dtype=TDT[dtype], device=DEV)
        block = int(rng.choice([R, 173, 1000]))
        for r0 in range(0, R, block):
            rc = lib.cwr_joint_backward(h[r0:].data_ptr(), W.data_ptr(), b.data_ptr() if b is not None else None,
                                        _DTYPES[TDT[dtype]], min(block, R - r0), H, V, N, blank,
                                        st.rowinfo[r0:].data_ptr(), st.grads[r0:].data_ptr(), st.lse[r0:].data_ptr(),
                                        gc.data_ptr(), 1, 1.0, dz[r0:].data_ptr(), _stream_ptr(torch.device(DEV)))
            assert rc == 0, (what, _lib.strerror(rc))
        torch.cuda.synchronize()
        got = dz.double().cpu().numpy()
        eps = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
        # entries that are the difference of two terms (softmax * gamma against G) carry the fp32 rounding of both
        tol = eps * np.abs(ref["grad"]) + 2e-5 * np.abs(ref["grad"]).max(axis=1, keepdims=True) + 5e-6
        assert np.all(np.isfinite(got)), what
        bad = np.abs(got - ref["grad"]) > tol
        assert not bad.any(), (what, np.argwhere(bad)[:5], got[bad][:5], ref["grad"][bad][:5])


@pytest.mark.parametrize("H", [64, 256])
def test_joint_bias_of_minus_inf_masks_a_vocabulary_entry(H):
    """An entry switched off through its bias (-inf, no label uses it) drops out of every row's
    log-sum-exp and gets a zero gradient; everything else matches the oracle on logits that hold
    -inf in that column.  Both the streaming (H=64) and a resident (H=256) kernel."""
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd import _lib
    from compactwarprnntloss_amd.loss import _DTYPES, _stream_ptr
    V, off = 40, 15
    j = make_joint([12, 7, 20], [4, 3, 9], H, V, seed=21, dtype="bf16", scale=2.0)
    j["yp"][j["yp"] == off] = off - 1
    j["b"][off] = -float("inf")
    N, R = j["N"], j["R"]
    with np.errstate(all="ignore"):
        z = orc.joint_logits(j["h"].double().numpy(), j["w"].double().numpy(), j["b"].numpy())
        ref = orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], 0, "fused", want_dense=True)
    h, W, b = j["h"].to(DEV), j["w"].to(DEV), j["b"].to(DEV)
    costs, st = pkg.joint_forward(h, W, b, torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["yp"]).to(DEV),
                                  torch.from_numpy(j["ly"]).to(DEV), 0)
    gc = torch.ones(N, device=DEV)
    dz = torch.full((R, V), float("nan"), dtype=torch.bfloat16, device=DEV)
    rc = _lib.load().cwr_joint_backward(h.data_ptr(), W.data_ptr(), b.data_ptr(), _DTYPES[torch.bfloat16], R, H, V, N,
                                        0, st.rowinfo.data_ptr(), st.grads.data_ptr(), st.lse.data_ptr(),
                                        gc.data_ptr(), 1, 1.0, dz.data_ptr(), _stream_ptr(torch.device(DEV)))
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    assert int(st.status[0].item()) == 0
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
    got = dz.double().cpu().numpy()
    assert np.all(np.isfinite(got)) and np.all(got[:, off] == 0)
    tol = 2.0 ** -8 * np.abs(ref["grad"]) + 2e-5 * np.abs(ref["grad"]).max(axis=1, keepdims=True) + 1e-7
    assert np.all(np.abs(got - ref["grad"]) <= tol)


def test_joint_full_size_config2_against_oracle():
    """The fused output layer at the benchmark's own size (config 2's lengths, N=32, R=311449,
    V=1024; H=512, bf16), sequence by sequence so that the float64 logits stay small: every cost
    and every entry of the per-row gradients from cwr_joint_forward, and the logit gradient of
    cwr_joint_backward (one call over all rows) on a few hundred sampled rows per sequence."""
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd import _lib, workloads as wl
    from compactwarprnntloss_amd.loss import _DTYPES, _stream_ptr
    cfg = wl.make_config(2)
    N, R, V, H = cfg["N"], cfg["R"], cfg["V"], 512
    g = torch.Generator(device="cpu").manual_seed(77)
    h = torch.randn((R, H), generator=g).to(torch.bfloat16)
    W = (torch.randn((V, H), generator=g) * (2.0 / H ** 0.5)).to(torch.bfloat16)   # logits ~ N(0, 2), as the config's
    b = torch.randn(V, generator=g)
    hd, Wd, bd = h.to(DEV), W.to(DEV), b.to(DEV)
    lx, ly = torch.from_numpy(cfg["lx"]).to(DEV), torch.from_numpy(cfg["ly"]).to(DEV)
    ys = torch.from_numpy(cfg["y_padded"]).to(DEV)
    costs, st = pkg.joint_forward(hd, Wd, bd, lx, ys, ly, 0, max_u=ys.size(1))
    rng = np.random.default_rng(5)
    go = rng.uniform(0.5, 1.5, N) / N
    gc = torch.from_numpy(go).float().to(DEV)
    dz = torch.empty((R, V), dtype=torch.bfloat16, device=DEV)
    rc = _lib.load().cwr_joint_backward(hd.data_ptr(), Wd.data_ptr(), bd.data_ptr(), _DTYPES[torch.bfloat16], R, H, V,
                                        N, 0, st.rowinfo.data_ptr(), st.grads.data_ptr(), st.lse.data_ptr(),
                                        gc.data_ptr(), 1, 1.0, dz.data_ptr(), _stream_ptr(torch.device(DEV)))
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    assert int(st.status[0].item()) == 0
    costs = costs.cpu().numpy().astype(np.float64)
    G_dev = st.grads.cpu().numpy().astype(np.float64)
    off = orc.row_offsets_i64(cfg["lx"], cfg["ly"])
    W64, b64 = W.double().numpy(), b.numpy()
    for n in range(N):
        a, e = int(off[n]), int(off[n + 1])
        U = int(cfg["ly"][n])
        z = orc.joint_logits(h[a:e].double().numpy(), W64, b64)
        ref = orc.loss_and_grad(z, cfg["lx"][n:n + 1], cfg["y_padded"][n:n + 1], cfg["ly"][n:n + 1], 0, "fused",
                                want_dense=False)
        assert abs(costs[n] - ref["costs"][0]) <= LOSS_RTOL * abs(ref["costs"][0]), (n, costs[n], ref["costs"][0])
        np.testing.assert_allclose(G_dev[a:e], ref["G"], rtol=0, atol=GRAD_ATOL, err_msg=f"sequence {n}")
        gamma = -(ref["G"][:, 0] + ref["G"][:, 1])
        rows = np.unique(np.concatenate([np.arange(U + 1), np.arange(e - a - U - 1, e - a),
                                         rng.integers(0, e - a, 200)]))
        want = np.exp(z[rows] - ref["lse"][rows, None]) * gamma[rows, None]
        want[:, 0] += ref["G"][rows, 0]
        u_of = rows % (U + 1)
        has = u_of < U
        lab = cfg["y_padded"][n, np.minimum(u_of, max(U - 1, 0))]
        want[np.nonzero(has)[0], lab[has]] += ref["G"][rows[has], 1]
        want *= go[n]
        got = dz[torch.from_numpy(a + rows).to(DEV)].double().cpu().numpy()
        tol = 2.0 ** -8 * np.abs(want) + 2e-5 * np.abs(want).max(axis=1, keepdims=True) + 1e-7
        bad = np.abs(got - want) > tol
        assert not bad.any(), (n, np.argwhere(bad)[:5], got[bad][:5], want[bad][:5])


def test_joiner_module_loss_agrees_with_the_stored_logits_route():
    """CompactJoiner.loss (output layer fused into the loss) against the same module's logits handed
    to transducer_loss, in bf16: the stored route rounds the logits to bf16 before the loss, the fused
    one does not, so the two agree to bf16 accuracy of the logits, not better."""
    import compactwarprnntloss_amd as pkg
    torch.manual_seed(3)
    N, E, P, J, V = 3, 24, 16, 64, 96
    lx = torch.tensor([9, 14, 6], dtype=torch.int32, device=DEV)
    ly = torch.tensor([4, 7, 2], dtype=torch.int32, device=DEV)
    enc = torch.randn(N, 14, E, device=DEV, dtype=torch.bfloat16)
    pred = torch.randn(N, 8, P, device=DEV, dtype=torch.bfloat16)
    y = torch.randint(1, V, (N, 7), dtype=torch.int32, device=DEV)
    joiner = pkg.CompactJoiner(E, P, J, V).to(DEV).to(torch.bfloat16)
    fused = joiner.loss(enc, pred, lx, y, ly, 0, "mean")
    fused.backward()
    got = [p.grad.float().clone() for p in joiner.parameters()]
    joiner.zero_grad()
    stored = pkg.transducer_loss(joiner(enc, pred, lx, ly), lx, y, ly, 0, "mean", fused_log_softmax=True)
    stored.backward()
    assert abs(float(fused.detach()) - float(stored.detach())) <= 2e-2 * abs(float(stored.detach()))
    for a, p in zip(got, joiner.parameters()):
        b = p.grad.float()
        assert torch.isfinite(a).all()
        cos = torch.nn.functional.cosine_similarity(a.flatten(), b.flatten(), dim=0)
        assert float(cos) > 0.99, float(cos)


# ----------------------------------------------------------------------------- the joiner's whole chain in one kernel
def make_fg(lx, ly, H, seed, dtype, T_extra=2, U_extra=1):
    rng = np.random.default_rng(seed)
    N = len(lx)
    T, Up = int(max(lx)) + T_extra, int(max(ly)) + 1 + U_extra  # padded beyond the longest sequence
    f = torch.from_numpy(rng.standard_normal((N, T, H)).astype(np.float32)).to(TDT[dtype])
    g = torch.from_numpy(rng.standard_normal((N, Up, H)).astype(np.float32)).to(TDT[dtype])
    return f, g


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("act", [None, "tanh", "relu"])
@pytest.mark.parametrize("lx,ly,H,V", [([9, 5, 12, 1], [3, 0, 7, 4], 256, 128), ([40, 33, 17], [12, 20, 5], 512, 300),
                                       ([25, 31], [20, 9], 768, 257), ([14, 6], [5, 130], 384, 64),
                                       ([12, 9], [7, 20], 128, 130), ([12, 9], [7, 20], 192, 64),
                                       ([21, 8], [6, 33], 320, 300), ([21, 8], [6, 33], 448, 64),
                                       ([16, 10], [12, 5], 576, 257), ([16, 10], [12, 5], 896, 130)])
def test_joiner_chain_forward_matches_oracle(dtype, act, lx, ly, H, V):
    """cwr_joint_forward_fg: rows act(f[n,t] + g[n,u]) formed in the kernel.  Oracle: join_rows in
    float64, rounded once to the 16-bit type (the kernel's one rounding), joint_logits, fused-mode
    loss.  The rows the kernel leaves behind on request are bit-identical to compact_join's, and the
    results do not depend on whether it leaves them."""
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd.joiner import _ACTS
    j = make_joint(lx, ly, H, V, seed=21, dtype=dtype, scale=3.0)
    f, g = make_fg(lx, ly, H, 22, dtype)
    h64 = orc.join_rows(f.double().numpy(), g.double().numpy(), j["lx"], j["ly"], act)
    h16 = torch.from_numpy(h64).to(TDT[dtype])
    z = orc.joint_logits(h16.double().numpy(), j["w"].double().numpy(), j["b"].numpy())
    ref = orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], 0, "fused", want_dense=False)
    lxd, lyd = torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["ly"]).to(DEV)
    yd = torch.from_numpy(j["yp"]).to(DEV)
    fd, gd, wd, bd = f.to(DEV), g.to(DEV), j["w"].to(DEV), j["b"].to(DEV)
    outs = []
    for keep in (False, True):
        costs, st, h = pkg.loss.joint_forward_fg(fd, gd, _ACTS[act], wd, bd, lxd, yd, lyd, 0, j["R"], keep_rows=keep)
        torch.cuda.synchronize()
        assert int(st.status[0].item()) == 0
        # a row's rounding to 16 bits may differ from the oracle's by one ulp of the type where the
        # float32 sum sits on a rounding boundary: the tolerances of the stored-rows route apply
        np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=2e-4 if dtype == "bf16" else 3e-5)
        outs.append((costs.cpu().numpy(), st.lse.cpu().numpy(), st.grads.cpu().numpy()))
        if keep:
            hj = pkg.compact_join(fd, gd, lxd, lyd, act, total_rows=j["R"])
            assert torch.equal(h, hj)
            # and from those very rows the stored-rows entry point gives the same bits
            c2, st2 = pkg.joint_forward(hj, wd, bd, lxd, yd, lyd, 0)
            assert torch.equal(c2, costs) and torch.equal(st2.lse, st.lse) and torch.equal(st2.grads, st.grads)
            z2 = orc.joint_logits(hj.double().cpu().numpy(), j["w"].double().numpy(), j["b"].numpy())
            ref2 = orc.loss_and_grad(z2, j["lx"], j["yp"], j["ly"], 0, "fused", want_dense=False)
            np.testing.assert_allclose(costs.cpu().numpy(), ref2["costs"], rtol=LOSS_RTOL)
            np.testing.assert_allclose(st.grads.cpu().numpy(), ref2["G"], rtol=0, atol=GRAD_ATOL)
            np.testing.assert_allclose(st.lse.cpu().numpy(), ref2["lse"], rtol=2e-6, atol=2e-5)
    for a, b in zip(outs[0], outs[1]):
        assert np.array_equal(a, b)


def test_joiner_chain_flags_cells_outside_its_inputs_and_refuses_other_joint_sizes():
    import compactwarprnntloss_amd as pkg
    from compactwarprnntloss_amd import _lib
    j = make_joint([6, 4], [3, 2], 256, 64, seed=5, dtype="bf16")
    f, g = make_fg([6, 4], [3, 2], 256, 6, "bf16", T_extra=-1, U_extra=0)  # one frame short of the longest sequence
    lxd, lyd = torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["ly"]).to(DEV)
    yd = torch.from_numpy(j["yp"]).to(DEV)
    costs, st, _ = pkg.loss.joint_forward_fg(f.to(DEV), g.to(DEV), 1, j["w"].to(DEV), None, lxd, yd, lyd, 0, j["R"])
    torch.cuda.synchronize()
    assert int(st.status[0].item()) & _lib.FLAG_BAD_LENGTH
    assert torch.isfinite(costs).all()
    f2, g2 = make_fg([6, 4], [3, 2], 96, 7, "bf16")
    with pytest.raises(RuntimeError):
        pkg.loss.joint_forward_fg(f2.to(DEV), g2.to(DEV), 1, j["w"][:, :96].contiguous().to(DEV), None, lxd, yd, lyd, 0, j["R"])
    lib = _lib.load()
    A = 1 << 20
    assert lib.cwr_joint_forward_fg(A, A, 1, 8, 5, None, A, None, _lib.BF16, 100, 96, 64, A, A, A, 3, 6, 2, 0, 3, A,
                                    1 << 20, A, A, A, A, A, A, A, None) == 4      # CWR_ERR_SHAPE: not a resident size
    assert lib.cwr_joint_forward_fg(A, A, 7, 8, 5, None, A, None, _lib.BF16, 100, 256, 64, A, A, A, 3, 6, 2, 0, 3, A,
                                    1 << 20, A, A, A, A, A, A, A, None) == 3      # CWR_ERR_MODE: activation
    assert lib.cwr_joint_forward_fg(None, A, 1, 8, 5, None, A, None, _lib.BF16, 100, 256, 64, A, A, A, 3, 6, 2, 0, 3,
                                    A, 1 << 20, A, A, A, A, A, A, A, None) == 1   # CWR_ERR_NULL


@pytest.mark.parametrize("act", [None, "tanh", "relu"])
@pytest.mark.parametrize("reduction", ["mean", "none"])
def test_fused_joiner_loss_gradients(act, reduction):
    """fused_joiner_loss -> (df, dg, dW, dbias): identical to compact_join + fused_joint_loss (the same
    kernels behind both, the rows bit-identical), and within the 16-bit tolerances of the oracle's
    chain rule (dense fused gradient of the float64 logits, joint_backward, join_rows_backward)."""
    import compactwarprnntloss_amd as pkg
    lx, ly, H, V = [40, 33, 17], [12, 20, 5], 256, 300
    j = make_joint(lx, ly, H, V, seed=31, dtype="bf16", scale=3.0)
    f, g = make_fg(lx, ly, H, 32, "bf16")
    N = j["N"]
    w8 = np.random.default_rng(2).uniform(0.5, 1.5, N)
    go = np.full(N, 1.0 / N) if reduction == "mean" else w8
    lxd, lyd = torch.from_numpy(j["lx"]).to(DEV), torch.from_numpy(j["ly"]).to(DEV)
    yd = torch.from_numpy(j["yp"]).to(DEV)
    wt = torch.from_numpy(w8).to(DEV).float()

    def run(chain):
        fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
        W, b = j["w"].to(DEV).requires_grad_(True), j["b"].to(DEV).requires_grad_(True)
        red = "mean" if reduction == "mean" else "none"
        if chain:
            out = pkg.fused_joiner_loss(fd, gd, W, b, lxd, yd, lyd, 0, red, act, total_rows=j["R"], chunk_rows=257,
                                        one_kernel=True)
        else:
            h = pkg.compact_join(fd, gd, lxd, lyd, act, total_rows=j["R"])
            out = pkg.fused_joint_loss(h, W, b, lxd, yd, lyd, 0, red, chunk_rows=257)
        loss = out if reduction == "mean" else (out * wt).sum()
        loss.backward()
        torch.cuda.synchronize()
        return [t.grad for t in (fd, gd, W, b)], loss.detach()

    got, loss = run(True)
    two, loss2 = run(False)
    assert torch.equal(loss, loss2)
    for a, b_, name in zip(got, two, ("df", "dg", "dW", "dbias")):
        assert torch.equal(a, b_), name
    # oracle
    f64, g64 = f.double().numpy(), g.double().numpy()
    h16 = pkg.compact_join(f.to(DEV), g.to(DEV), lxd, lyd, act, total_rows=j["R"]).double().cpu().numpy()
    z = orc.joint_logits(h16, j["w"].double().numpy(), j["b"].numpy())
    ref = orc.loss_and_grad(z, j["lx"], j["yp"], j["ly"], 0, "fused", grad_out=go, want_dense=True)
    dh_ref, dw_ref, db_ref = orc.joint_backward(ref["grad"], h16, j["w"].double().numpy())
    df_ref, dg_ref = orc.join_rows_backward(dh_ref, f64, g64, j["lx"], j["ly"], act)
    for a, want, name in zip(got, (df_ref, dg_ref, dw_ref, db_ref), ("df", "dg", "dW", "dbias")):
        a = a.double().cpu().numpy()
        scale = np.abs(want).max()
        np.testing.assert_allclose(a, want, rtol=2e-2, atol=2e-2 * scale, err_msg=name)
