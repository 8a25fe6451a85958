"""GPU parity: the HIP path (through the C ABI) against the float64 oracle on the same seeded
inputs.  Gates: loss <= 1e-5 relative, gradients <= 1e-4 absolute (fp32), offsets and flags exact.
"""
import math

import numpy as np
import pytest
import torch

from compactwarprnntloss_amd import workloads as wl
from oracle import rnnt_oracle as orc

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-4

TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "f64": torch.float64}


def _pkg():
    import compactwarprnntloss_amd as pkg
    return pkg


def make_batch(lx, ly, V, seed, sigma=1.0, dtype="f32", blank=0, normalised=False):
    rng = np.random.default_rng(seed)
    lx = np.asarray(lx, dtype=np.int32)
    ly = np.asarray(ly, dtype=np.int32)
    N = len(lx)
    R = int(orc.row_offsets_i64(lx, ly)[-1])
    x = (rng.standard_normal((R, V)) * sigma).astype(np.float32)
    if normalised:
        x = orc.log_softmax(x).astype(np.float32)
    Umax = int(ly.max()) if N else 0
    yp = np.zeros((N, Umax), dtype=np.int32)
    for n in range(N):
        lab = rng.integers(0, V - 1, int(ly[n])).astype(np.int32)
        lab[lab >= blank] += 1  # any symbol but the blank
        yp[n, : ly[n]] = lab
    yc = np.concatenate([yp[n, : ly[n]] for n in range(N)]) if N else np.zeros(0, np.int32)
    tdt = TORCH_DT[dtype]
    xt = torch.from_numpy(x).to(tdt)
    x_ref = xt.to(torch.float64).numpy()  # what the device actually sees, exactly
    return dict(lx=lx, ly=ly, yp=yp, yc=yc, x=xt, x_ref=x_ref, V=V, R=R, N=N, blank=blank)


def run_device(b, fused, labels="2d", grad_out=None, with_grad=True, max_u=None):
    pkg = _pkg()
    dev = torch.device("cuda:0")
    xs = b["x"].to(dev)
    lx = torch.from_numpy(b["lx"]).to(dev)
    ly = torch.from_numpy(b["ly"]).to(dev)
    ys = torch.from_numpy(b["yp"] if labels == "2d" else b["yc"]).to(dev)
    costs, st = pkg.rnnt_forward(xs, lx, ys, ly, b["blank"], fused, max_u=max_u, with_grad=with_grad)
    out = dict(costs=costs.cpu().numpy().astype(np.float64), flags=int(st.status[0].item()),
               row_off=st.row_off.cpu().numpy(), lab_off=st.lab_off.cpu().numpy())
    if with_grad:
        out["G"] = st.grads.cpu().numpy().astype(np.float64)
        if fused:
            out["lse"] = st.lse.cpu().numpy().astype(np.float64)
        go = np.ones(b["N"]) if grad_out is None else grad_out
        g = pkg.rnnt_backward(xs, lx, ys, ly, b["blank"], st, torch.from_numpy(go).to(dev))
        out["grad"] = g.to(torch.float64).cpu().numpy()
    torch.cuda.synchronize()
    return out


def check_case(b, fused, labels="2d", dtype="f32", seed=0, with_weights=True):
    rng = np.random.default_rng(seed + 99)
    go = rng.uniform(-1.5, 1.5, b["N"]) if with_weights else None
    dev = run_device(b, fused, labels, go)
    y = b["yp"] if labels == "2d" else b["yc"]
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], y, b["ly"], b["blank"], "fused" if fused else "logprob",
                            grad_out=go)
    assert dev["flags"] == 0
    assert np.array_equal(dev["row_off"], ref["row_off"])
    assert np.array_equal(dev["lab_off"], orc.label_offsets_i64(b["ly"]))
    np.testing.assert_allclose(dev["costs"], ref["costs"], rtol=LOSS_RTOL, atol=1e-6)
    np.testing.assert_allclose(dev["G"], ref["G"], rtol=0, atol=GRAD_ATOL)
    if fused:
        np.testing.assert_allclose(dev["lse"], ref["lse"], rtol=1e-6, atol=1e-5)
    if dtype == "f32" or dtype == "f64":
        np.testing.assert_allclose(dev["grad"], ref["grad"], rtol=0, atol=GRAD_ATOL)
    else:
        rel = 1e-3 if dtype == "f16" else 8e-3  # one rounding to the storage type
        np.testing.assert_allclose(dev["grad"], ref["grad"], rtol=rel, atol=GRAD_ATOL)
    return dev, ref


# ----------------------------------------------------------------------------- offsets
def test_offsets_exact_and_flags():
    from compactwarprnntloss_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    for N in [1, 2, 63, 64, 65, 200, 1000]:
        lx = rng.integers(1, 400, N).astype(np.int32)
        ly = rng.integers(0, 120, N).astype(np.int32)
        lxd, lyd = torch.from_numpy(lx).to(dev), torch.from_numpy(ly).to(dev)
        ro = torch.empty(N + 1, dtype=torch.int64, device=dev)
        lo = torch.empty(N + 1, dtype=torch.int64, device=dev)
        st = torch.empty(4, dtype=torch.int32, device=dev)
        R = int(orc.row_offsets_i64(lx, ly)[-1])
        rc = lib.cwr_offsets(lxd.data_ptr(), lyd.data_ptr(), N, R, ro.data_ptr(), lo.data_ptr(),
                             st.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        assert np.array_equal(ro.cpu().numpy(), orc.row_offsets_i64(lx, ly))
        assert np.array_equal(lo.cpu().numpy(), orc.label_offsets_i64(ly))
        # the reference keeps the first N entries as int32
        assert np.array_equal(ro.cpu().numpy()[:N].astype(np.int32), orc.row_offsets(lx, ly))
        assert st.cpu().numpy().tolist() == [0, 0, 0, 0]
        rc = lib.cwr_offsets(lxd.data_ptr(), lyd.data_ptr(), N, R + 1, ro.data_ptr(), lo.data_ptr(),
                             st.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0 and int(st[0].item()) == _lib.FLAG_ROWS_MISMATCH


# ----------------------------------------------------------------------------- small shapes
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("labels", ["2d", "1d"])
def test_config1_tiny(fused, labels):
    cfg = wl.make_config(1)
    b = make_batch(cfg["lx"], cfg["ly"], cfg["V"], seed=1, sigma=1.0, normalised=not fused)
    check_case(b, fused, labels)


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("T,U", [(1, 0), (1, 1), (1, 7), (5, 0), (2, 1), (9, 4), (4, 9), (1, 64), (70, 62),
                                 (70, 63), (70, 64), (33, 127), (40, 128), (20, 200), (3, 300), (300, 3),
                                 (10, 511), (10, 512), (7, 600), (400, 130), (900, 70), (150, 200), (300, 255),
                                 (300, 256), (120, 383), (9, 1022), (9, 1023), (6, 1024), (5, 1100), (60, 520),
                                 (40, 1500), (4, 2046), (4, 2047), (3, 2048), (2, 2300)])
def test_edge_shapes_single_sequence(fused, T, U):
    b = make_batch([T], [U], 16, seed=T * 1000 + U, normalised=not fused)
    check_case(b, fused)


@pytest.mark.parametrize("fused", [False, True])
def test_ragged_mix_with_empty_label_and_single_frame(fused):
    lx = [7, 1, 30, 2, 65, 1, 12, 90]
    ly = [3, 5, 0, 2, 70, 0, 12, 1]
    b = make_batch(lx, ly, 40, seed=5, normalised=not fused)
    check_case(b, fused, "2d")
    check_case(b, fused, "1d")


@pytest.mark.parametrize("V", [3, 5, 32, 33, 64, 96, 100, 128, 200, 256, 257, 300, 500, 512, 1000, 1024, 2048, 4096, 4100, 4233,
                               5537, 8192, 16384, 32000, 50257])
def test_vocabulary_sizes_fused(V):
    b = make_batch([6, 3, 9], [2, 4, 1], V, seed=V, sigma=2.0)
    check_case(b, True)


@pytest.mark.parametrize("V", [3, 32, 33, 128, 1024, 1000, 257, 4233, 50257])
def test_vocabulary_sizes_logprob(V):
    b = make_batch([6, 3, 9], [2, 4, 1], V, seed=V, normalised=True)
    check_case(b, False)


@pytest.mark.parametrize("blank", [0, 5, 15])
@pytest.mark.parametrize("fused", [False, True])
def test_blank_positions(blank, fused):
    b = make_batch([6, 3, 9, 11], [2, 4, 1, 6], 16, seed=blank, blank=blank, normalised=not fused)
    check_case(b, fused)


@pytest.mark.parametrize("dtype,V", [("f16", 64), ("f16", 4096), ("bf16", 256), ("f64", 32), ("f64", 1024),
                                     ("f16", 5537), ("f16", 520), ("bf16", 4233), ("f64", 777), ("f16", 32000),
                                     ("f16", 41), ("bf16", 100), ("f64", 33), ("f16", 7), ("f16", 512), ("bf16", 1024),
                                     ("f16", 200), ("f64", 100), ("f64", 256)])
@pytest.mark.parametrize("fused", [False, True])
def test_storage_types(dtype, V, fused):
    b = make_batch([12, 5, 20], [4, 7, 2], V, seed=V, dtype=dtype, normalised=not fused)
    check_case(b, fused, dtype=dtype)


def test_nograd_cost_equals_grad_cost():
    b = make_batch([30, 11, 64, 5], [10, 11, 70, 0], 48, seed=3)
    for fused in (False, True):
        a = run_device(b, fused)
        c = run_device(b, fused, with_grad=False)
        np.testing.assert_allclose(a["costs"], c["costs"], rtol=1e-6)


def test_label_equal_to_blank_logprob_follows_reference_overwrite():
    b = make_batch([4, 3], [2, 2], 8, seed=8, normalised=True)
    b["yp"][0, 0] = 0
    b["yc"][0] = 0
    check_case(b, False)
    check_case(b, True)


# ----------------------------------------------------------------------------- benchmark shapes
@pytest.mark.parametrize("idx,scale", [(2, 0.25), (4, 0.3), (5, 0.15)])
@pytest.mark.parametrize("fused", [False, True])
def test_benchmark_configs_reduced(idx, scale, fused):
    cfg = wl.make_config(idx, scale=scale)
    b = make_batch(cfg["lx"], cfg["ly"], cfg["V"], seed=idx, sigma=cfg["sigma"], normalised=not fused)
    check_case(b, fused, "1d")


def test_config3_reduced_fp16():
    cfg = wl.make_config(3, scale=0.15)
    b = make_batch(cfg["lx"], cfg["ly"], cfg["V"], seed=3, sigma=1.0, dtype="f16")
    check_case(b, True, "2d", dtype="f16")


# ----------------------------------------------------------------------------- entry point
@pytest.mark.parametrize("reduction", ["mean", "sum", "none", None])
@pytest.mark.parametrize("fused", [False, True])
def test_transducer_loss_autograd(reduction, fused):
    import cwarp_rnnt
    b = make_batch([9, 4, 15], [3, 4, 0], 24, seed=21, normalised=not fused)
    dev = torch.device("cuda:0")
    x = b["x"].to(dev).requires_grad_(True)
    lx, ly = torch.from_numpy(b["lx"]).to(dev), torch.from_numpy(b["ly"]).to(dev)
    y = torch.from_numpy(b["yp"]).to(dev)
    loss = cwarp_rnnt.transducer_loss(x, lx, y, ly, 0, reduction, fused_log_softmax=fused, validate=True)
    w = np.array([1.0, -2.0, 0.5])
    if reduction in ("none", None):
        assert loss.shape == (3,)
        (loss * torch.from_numpy(w).to(dev, torch.float32)).sum().backward()
        go = w
    else:
        assert loss.dim() == 0
        loss.backward()
        go = np.full(3, 1.0 / 3 if reduction == "mean" else 1.0)
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "fused" if fused else "logprob", grad_out=go)
    want = orc.reduce_costs(ref["costs"], reduction)
    np.testing.assert_allclose(loss.detach().cpu().numpy(), want, rtol=LOSS_RTOL)
    np.testing.assert_allclose(x.grad.cpu().numpy(), ref["grad"], atol=GRAD_ATOL)
    # no-grad path
    with torch.no_grad():
        l2 = cwarp_rnnt.transducer_loss(x.detach(), lx, y, ly, 0, reduction, fused_log_softmax=fused)
    np.testing.assert_allclose(l2.cpu().numpy(), want, rtol=LOSS_RTOL)


def test_data_dependent_problems_are_flagged_not_faulted():
    from compactwarprnntloss_amd import _lib
    b = make_batch([5, 6], [2, 3], 12, seed=2)
    # a label outside [0,V)
    b2 = dict(b)
    b2["yp"] = b["yp"].copy()
    b2["yp"][1, 1] = 99
    for fused in (True, False):
        out = run_device(b2, fused)
        assert out["flags"] & _lib.FLAG_BAD_LABEL
        # the sequence with the bad label cannot be consumed by mistake; the other one is untouched
        assert np.isnan(out["costs"][1]) and np.isfinite(out["costs"][0])
        good = run_device(b, fused)
        assert out["costs"][0] == good["costs"][0]
    out = run_device(b2, True, with_grad=False)
    assert np.isnan(out["costs"][1]) and np.isfinite(out["costs"][0])
    b2c = dict(b2)   # concatenated labels that end too early: the last label of the batch is missing
    b2c["yc"] = b["yc"][:-1].copy()
    out = run_device(b2c, True, labels="1d", max_u=3)
    assert out["flags"] & _lib.FLAG_BAD_LABEL and np.isnan(out["costs"][1]) and np.isfinite(out["costs"][0])
    assert np.isfinite(out["G"]).all() and not out["G"][out["row_off"][1]:out["row_off"][2]].any()
    # lengths that claim more rows than x has
    b3 = dict(b)
    b3["lx"] = np.array([5, 60], dtype=np.int32)
    out = run_device(b3, True)
    assert out["flags"] & _lib.FLAG_ROWS_MISMATCH
    assert np.isnan(out["costs"][1]) and np.isfinite(out["costs"][0])
    # a non-positive frame count
    b4 = dict(b)
    b4["lx"] = np.array([0, 6], dtype=np.int32)
    out = run_device(b4, True)
    assert out["flags"] & _lib.FLAG_BAD_LENGTH
    assert np.isnan(out["costs"][0])
    import cwarp_rnnt
    dev = torch.device("cuda:0")
    with pytest.raises(RuntimeError):
        cwarp_rnnt.transducer_loss(b2["x"].to(dev), torch.from_numpy(b2["lx"]).to(dev),
                                   torch.from_numpy(b2["yp"]).to(dev), torch.from_numpy(b2["ly"]).to(dev),
                                   fused_log_softmax=True, validate=True)


def test_a_wait_that_runs_out_ends_the_walk_and_poisons_only_its_sequence():
    """The strips of a sequence wait for each other with bounded polls.  With the bound set to one
    poll from the host, the second strip of a two-strip sequence gives up at once: the kernel must
    still finish, flag CWR_FLAG_INTERNAL, give that sequence a NaN cost and leave the one-strip
    sequences of the batch exact.  With the default bound back, the same batch is exact throughout."""
    from compactwarprnntloss_amd import _lib
    lib = _lib.load()
    b = make_batch([60, 200, 45], [30, 150, 63], 24, seed=8)
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "fused", want_dense=False)
    try:
        lib.cwr_debug_wait_limit(1)
        for with_grad in (True, False):
            out = run_device(b, True, with_grad=with_grad)
            assert out["flags"] & _lib.FLAG_INTERNAL
            assert np.isnan(out["costs"][1])
            np.testing.assert_allclose(out["costs"][[0, 2]], ref["costs"][[0, 2]], rtol=LOSS_RTOL)
            if with_grad:
                # the poisoned sequence's gradients are zeros, not whatever its unfinished lattice held:
                # a caller that masks the NaN cost with a zero weight must not get NaN * 0
                a, e = out["row_off"][1], out["row_off"][2]
                assert not out["G"][a:e].any() and np.isfinite(out["grad"]).all()
                assert not out["grad"][a:e].any()
                np.testing.assert_allclose(out["G"][:a], ref["G"][:a], rtol=0, atol=GRAD_ATOL)
    finally:
        lib.cwr_debug_wait_limit(0)
    out = run_device(b, True)
    assert out["flags"] == 0
    np.testing.assert_allclose(out["costs"], ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(out["G"], ref["G"], rtol=0, atol=GRAD_ATOL)


# ----------------------------------------------------------------------------- golden fixtures
def _golden_files():
    import os
    gdir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    return sorted(os.path.join(gdir, f) for f in os.listdir(gdir) if f.endswith(".npz") and not f.startswith("join_"))


@pytest.mark.parametrize("path", _golden_files(), ids=lambda p: p.split("/")[-1][:-4])
def test_against_golden_fixtures(path):
    z = np.load(path)
    fused = str(z["mode"]) == "fused"
    b = dict(lx=z["lx"], ly=z["ly"], yp=z["y"], yc=np.concatenate([z["y"][n, : z["ly"][n]] for n in range(len(z["lx"]))]),
             x=torch.from_numpy(z["x"]), V=z["x"].shape[1], R=z["x"].shape[0], N=len(z["lx"]), blank=int(z["blank"]))
    for labels in ("2d", "1d"):
        dev = run_device(b, fused, labels, z["grad_out"])
        assert dev["flags"] == 0
        assert np.array_equal(dev["row_off"][:-1].astype(np.int32), z["row_off_i32"])
        np.testing.assert_allclose(dev["costs"], z["costs"], rtol=LOSS_RTOL)
        np.testing.assert_allclose(dev["G"], z["G"], atol=GRAD_ATOL)
        np.testing.assert_allclose(dev["grad"], z["grad"], atol=GRAD_ATOL)


# ----------------------------------------------------------------------------- number systems of the walk
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("sigma", [8.0, 25.0, 60.0])
def test_steep_logits_linear_and_log_walks(fused, sigma):
    """sigma 8 keeps the scaled linear-domain walk busy renormalising (about -50 bits per step);
    25 and 60 push log-probs below the linear walk's range, so those sequences take the log walk."""
    b = make_batch([90, 30, 150], [70, 3, 140], 200, seed=int(sigma), sigma=sigma, normalised=not fused)
    check_case(b, fused)


def test_mixed_batch_one_extreme_sequence():
    """Only the sequence with extreme log-probs is marked for the log-domain walk."""
    b = make_batch([40, 60, 35, 80], [20, 70, 5, 10], 64, seed=77, sigma=2.0)
    off = orc.row_offsets_i64(b["lx"], b["ly"])
    x = b["x"].clone()
    x[off[1]:off[2]] *= 40.0
    b["x"] = x
    b["x_ref"] = x.to(torch.float64).numpy()
    dev, ref = check_case(b, True)
    assert np.all(np.isfinite(dev["costs"]))


def test_minus_inf_logits_stay_finite_where_a_path_exists():
    """A vocabulary entry masked with -inf that no label uses must not disturb the loss."""
    b = make_batch([12, 7], [4, 3], 16, seed=5)
    x = b["x"].clone()
    x[:, 15] = -float("inf")
    b["yp"][b["yp"] == 15] = 14
    b["yc"][b["yc"] == 15] = 14
    b["x"] = x
    b["x_ref"] = x.to(torch.float64).numpy()
    dev = run_device(b, True)
    with np.errstate(all="ignore"):
        ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "fused")
    np.testing.assert_allclose(dev["costs"], ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(dev["grad"], ref["grad"], atol=GRAD_ATOL)


# ----------------------------------------------------------------------------- full benchmark sizes
def _full_config(idx):
    cfg = wl.make_config(idx)
    tdt = torch.float16 if cfg["dtype"] == "f16" else torch.float32
    g = torch.Generator(device="cpu").manual_seed(1000 + idx)
    x = (torch.randn((cfg["R"], cfg["V"]), generator=g, dtype=torch.float32) * cfg["sigma"]).to(tdt)
    return cfg, x


@pytest.mark.parametrize("idx", [2, 3, 4, 5])
def test_full_size_configs_size_independent_properties(idx):
    """At the benchmark's own sizes: what must hold whatever the size.  Every frame leaves its
    lattice row by exactly one blank and every label is emitted exactly once (so the sparse
    gradients of a sequence sum to -T and -U), a dense fused gradient row sums to zero, the
    gradient is linear in the incoming one, and the gradient and loss-only passes agree."""
    pkg = _pkg()
    cfg, x = _full_config(idx)
    dev = torch.device("cuda:0")
    xs = x.to(dev)
    lx, ly = torch.from_numpy(cfg["lx"]).to(dev), torch.from_numpy(cfg["ly"]).to(dev)
    ys = torch.from_numpy(cfg["y_padded"]).to(dev)
    N = cfg["N"]
    costs, st = pkg.rnnt_forward(xs, lx, ys, ly, 0, True)
    costs_only, _ = pkg.rnnt_forward(xs, lx, ys, ly, 0, True, with_grad=False)
    assert int(st.status[0].item()) == 0
    assert torch.isfinite(costs).all() and (costs > 0).all()
    torch.testing.assert_close(costs_only, costs, rtol=1e-6, atol=0)
    rows = (lx.long() * (ly.long() + 1))
    assert int(rows.sum().item()) == cfg["R"] and int(st.row_off[-1].item()) == cfg["R"]
    seq = torch.repeat_interleave(torch.arange(N, device=dev), rows)
    assert torch.equal(st.rowinfo[:, 1].long(), seq)
    occ = torch.zeros((N, 2), dtype=torch.float64, device=dev).index_add_(0, seq, -st.grads.double())
    torch.testing.assert_close(occ[:, 0], lx.double(), rtol=2e-5, atol=1e-3)
    torch.testing.assert_close(occ[:, 1], ly.double(), rtol=2e-5, atol=1e-3)
    w = torch.rand(N, device=dev) + 0.5
    g1 = pkg.rnnt_backward(xs, lx, ys, ly, 0, st, w)
    row_sum = g1.float().sum(dim=1).abs().max().item()
    assert row_sum < (2e-5 if idx != 3 else 2e-2)      # fp16 storage rounds each of the 4096 entries
    g2 = pkg.rnnt_backward(xs, lx, ys, ly, 0, st, w, scale=2.0)
    # a power-of-two factor commutes with rounding (up to flushed denormals, and fp16 overflow aside)
    torch.testing.assert_close(g2.float(), 2 * g1.float(), rtol=1e-6 if idx != 3 else 2e-3,
                               atol=1e-30 if idx != 3 else 2e-7)   # fp16 subnormals step by 6e-8
    del g2
    # the blank and label columns carry the whole of the sparse gradient's mass
    lab = st.rowinfo[:, 0].long()
    wrow = w[seq].double()
    pb = torch.exp(xs[:, 0].double() - st.lse.double())
    gamma = -(st.grads.double().sum(dim=1))
    torch.testing.assert_close(g1[:, 0].double(), wrow * (pb * gamma + st.grads[:, 0].double()),
                               rtol=2e-3 if idx == 3 else 1e-5, atol=1e-6)
    has = lab >= 0
    pl = torch.exp(xs[has, lab[has]].double() - st.lse[has].double())
    torch.testing.assert_close(g1[has, lab[has]].double(), wrow[has] * (pl * gamma[has] + st.grads[has, 1].double()),
                               rtol=2e-3 if idx == 3 else 1e-5, atol=1e-6)


@pytest.mark.parametrize("idx", [2, 3, 4, 5])
def test_full_size_configs_against_oracle(idx):
    """Direct parity at the benchmark's own sizes, sequence by sequence so that the float64 copy
    of the logits stays small: every cost, every entry of the sparse gradient, and the dense
    gradient on a few hundred sampled rows per sequence (rebuilt from the oracle's G and lse as
    softmax * gamma + G) and on the blank and label columns of every row.  Per-element agreement of
    forward and backward, as test/test.py:84-101 of the reference intends."""
    pkg = _pkg()
    cfg, x = _full_config(idx)
    half = cfg["dtype"] == "f16"
    dev = torch.device("cuda:0")
    xs = x.to(dev)
    lx, ly = torch.from_numpy(cfg["lx"]).to(dev), torch.from_numpy(cfg["ly"]).to(dev)
    ys = torch.from_numpy(cfg["y_padded"]).to(dev)
    N, V = cfg["N"], cfg["V"]
    costs, st = pkg.rnnt_forward(xs, lx, ys, ly, 0, True)
    rng = np.random.default_rng(idx)
    go = rng.uniform(0.5, 1.5, N) / N
    g = pkg.rnnt_backward(xs, lx, ys, ly, 0, st, torch.from_numpy(go).to(dev))
    assert int(st.status[0].item()) == 0
    costs = costs.cpu().numpy().astype(np.float64)
    G_dev = st.grads.cpu().numpy().astype(np.float64)
    off = orc.row_offsets_i64(cfg["lx"], cfg["ly"])
    assert np.array_equal(st.row_off.cpu().numpy(), off)
    rel = 1e-3 if half else 0.0  # one rounding of the stored gradient to fp16
    for n in range(N):
        a, b = int(off[n]), int(off[n + 1])
        T, U = int(cfg["lx"][n]), int(cfg["ly"][n])
        xn = x[a:b].numpy()  # storage type: the oracle widens what it uses to float64
        ref = orc.loss_and_grad(xn, cfg["lx"][n:n + 1], cfg["y_padded"][n:n + 1], cfg["ly"][n:n + 1], 0, "fused",
                                want_dense=False)
        assert abs(costs[n] - ref["costs"][0]) <= LOSS_RTOL * abs(ref["costs"][0]), (n, costs[n], ref["costs"][0])
        assert not ref["mismatch"][0]
        np.testing.assert_allclose(G_dev[a:b], ref["G"], rtol=0, atol=GRAD_ATOL, err_msg=f"sequence {n}")
        gamma = -(ref["G"][:, 0] + ref["G"][:, 1])
        # sampled rows: the first and last frames, and random ones in between
        rows = np.unique(np.concatenate([np.arange(min(U + 1, b - a)), np.arange(max(0, b - a - U - 1), b - a),
                                         rng.integers(0, b - a, 300)]))
        want = np.exp(xn[rows].astype(np.float64) - ref["lse"][rows, None]) * gamma[rows, None]
        want[:, 0] += ref["G"][rows, 0]
        u_of = rows % (U + 1)
        has = u_of < U
        lab = cfg["y_padded"][n, np.minimum(u_of, max(U - 1, 0))] if U > 0 else np.zeros(len(rows), np.int64)
        want[np.nonzero(has)[0], lab[has]] += ref["G"][rows[has], 1]
        want *= go[n]
        got = g[torch.from_numpy(a + rows).to(dev)].to(torch.float64).cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=rel, atol=GRAD_ATOL, err_msg=f"sequence {n}")
        # blank and label columns of EVERY row of the sequence
        gb = g[a:b, 0].to(torch.float64).cpu().numpy()
        wb = go[n] * (np.exp(xn[:, 0].astype(np.float64) - ref["lse"]) * gamma + ref["G"][:, 0])
        np.testing.assert_allclose(gb, wb, rtol=rel, atol=GRAD_ATOL)
        if U > 0:
            allrows = np.arange(b - a)
            uu = allrows % (U + 1)
            hh = uu < U
            ll = cfg["y_padded"][n, np.minimum(uu, U - 1)]
            gl = g[a:b][torch.from_numpy(allrows[hh]).to(dev), torch.from_numpy(ll[hh].astype(np.int64)).to(dev)]
            wl_ = go[n] * (np.exp(xn[allrows[hh], ll[hh]].astype(np.float64) - ref["lse"][hh]) * gamma[hh]
                           + ref["G"][hh, 1])
            np.testing.assert_allclose(gl.to(torch.float64).cpu().numpy(), wl_, rtol=rel, atol=GRAD_ATOL)


@pytest.mark.parametrize("fused,V", [(True, 64), (True, 128), (True, 512), (True, 1024), (False, 40)])
def test_more_than_64_sequences(fused, V):
    """Batches beyond 64 sequences leave the in-register sequence tables (gather, fill) for the
    search over the offset arrays."""
    rng = np.random.default_rng(77)
    N = 150
    lx = rng.integers(1, 12, N)
    ly = rng.integers(0, 9, N)
    b = make_batch(lx, ly, V, seed=12, normalised=not fused)
    check_case(b, fused, "1d")


@pytest.mark.parametrize("fused", [True, False])
def test_rows_beyond_two_to_the_31_elements(fused):
    """A tensor of more than 2^31 elements (the reference's int32 offsets end there,
    cwarp_cuda.cpp:72-77): the sequences at its far end must give the same costs and gradient
    rows as when they are run as a small batch of their own, and so must the first ones."""
    pkg = _pkg()
    N, T, U, V = 32, 700, 99, 1024
    R = N * T * (U + 1)
    assert R * V > 2 ** 31
    DEV = torch.device("cuda:0")
    gen = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn((R, V), device=DEV, dtype=torch.float16, generator=gen)
    if not fused:
        x = x.sub_(torch.logsumexp(x[:4096].float(), dim=1).mean().half())  # roughly normalised is enough here
    y = torch.randint(1, V, (N, U), device=DEV, dtype=torch.int32, generator=gen)
    lx = torch.full((N,), T, dtype=torch.int32, device=DEV)
    ly = torch.full((N,), U, dtype=torch.int32, device=DEV)
    costs, st = pkg.rnnt_forward(x, lx, y, ly, 0, fused)
    go = torch.ones(N, device=DEV)
    g = pkg.rnnt_backward(x, lx, y, ly, 0, st, go)
    assert int(st.status[0].item()) & ~8 == 0
    rows = T * (U + 1)
    for sl in (slice(0, 2), slice(N - 2, N)):
        xs = x[sl.start * rows: sl.stop * rows]
        c2, st2 = pkg.rnnt_forward(xs, lx[sl].contiguous(), y[sl].contiguous(), ly[sl].contiguous(), 0, fused)
        g2 = pkg.rnnt_backward(xs, lx[sl].contiguous(), y[sl].contiguous(), ly[sl].contiguous(), 0, st2, go[sl].contiguous())
        torch.testing.assert_close(costs[sl], c2, rtol=1e-6, atol=0)
        assert torch.equal(g[sl.start * rows: sl.stop * rows], g2)
    assert torch.isfinite(costs).all()
    if fused:   # rows of the dense gradient sum to zero, also at the far end
        tail = g[-4096:].float().sum(dim=1)
        assert float(tail.abs().max()) < 2e-2   # 1024 fp16-rounded entries per row


@pytest.mark.parametrize("fused,V", [(True, 16), (False, 64)])
def test_thousands_of_short_sequences(fused, V):
    """3000 sequences of a few cells each: the offsets scan in chunks of 64, one lattice workgroup
    per sequence and direction, and every per-sequence lookup far beyond the in-register tables."""
    rng = np.random.default_rng(6)
    N = 3000
    b = make_batch(rng.integers(1, 7, N), rng.integers(0, 4, N), V, seed=N, normalised=not fused)
    check_case(b, fused, "1d", seed=1)


# ----------------------------------------------------------------------------- number systems of the lattice walk
def _walk_modes(st):
    """Per-sequence walk-mode words of a forward call (workspace section 4)."""
    import ctypes as C
    lib = _pkg()._lib.load()
    off, nbytes = C.c_size_t(), C.c_size_t()
    assert lib.cwr_workspace_section(st.N, st.R, st.max_u, 4, C.byref(off), C.byref(nbytes)) == 0
    return st.workspace[off.value: off.value + 4 * st.N].view(torch.int32).cpu().numpy()


def _logprob_case(lx, ly, V, blank_nats, label_nats=None, seed=1):
    b = make_batch(lx, ly, V, seed=seed, normalised=True)
    x = b["x"].clone()
    x[:, 0] = blank_nats
    if label_nats is not None:
        x[:, 1:] = label_nats
    b["x"] = x
    b["x_ref"] = x.double().numpy()
    return b


@pytest.mark.parametrize("blank_nats", [-10.0, -30.0, -45.0, -62.0])
def test_columns_of_very_different_magnitude_stay_exact(blank_nats):
    """A blank that is improbable everywhere makes neighbouring label positions differ by that
    factor, so a diagonal of 60 cells spans thousands of bits.  The linear-domain walk carries
    one scale per column and must still be exact (a single scale per wave is not)."""
    b = _logprob_case([40, 120], [60, 50], 8, blank_nats)
    pkg = _pkg()
    dev = torch.device("cuda:0")
    xs = b["x"].to(dev)
    lx, ly = torch.from_numpy(b["lx"]).to(dev), torch.from_numpy(b["ly"]).to(dev)
    ys = torch.from_numpy(b["yp"]).to(dev)
    costs, st = pkg.rnnt_forward(xs, lx, ys, ly, 0, False)
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "logprob")
    assert int(st.status[0].item()) == 0
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
    assert not _walk_modes(st).any()        # all of it in the linear domain


def test_walk_leaves_the_linear_domain_when_its_range_check_fails():
    """Labels of probability 2^-95 next to blanks of probability ~1 put every label position 95
    bits below the one that feeds it; a column then sits more than 600 bits below the largest
    magnitude that can reach it within a block of steps, the range check of the linear walk fails,
    and the direction is walked again in the log domain.  The result must not care."""
    lx, ly = [70, 30], [20, 90]
    b = _logprob_case(lx, ly, 6, -0.1, -66.0)
    pkg = _pkg()
    dev = torch.device("cuda:0")
    xs = b["x"].to(dev)
    lxd, lyd = torch.from_numpy(b["lx"]).to(dev), torch.from_numpy(b["ly"]).to(dev)
    ys = torch.from_numpy(b["yp"]).to(dev)
    costs, st = pkg.rnnt_forward(xs, lxd, ys, lyd, 0, False)
    modes = _walk_modes(st)
    assert (modes & 1 == 0).all() and (modes & 6 == 6).all()      # both directions were done again
    assert int(st.status[0].item()) == 0
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "logprob")
    np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL)
    np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL)
    # the alpha / beta export reads the log-domain values of such a sequence
    alphas, betas = pkg.lattice_state(st, lxd, lyd, max(lx), max(ly) + 1)
    off = orc.row_offsets_i64(b["lx"], b["ly"])
    g = orc.gather(b["x_ref"], b["lx"], b["yp"], b["ly"], 0)
    for n, (T, U) in enumerate(zip(lx, ly)):
        lp = g[off[n]:off[n + 1]].reshape(T, U + 1, 2)
        np.testing.assert_allclose(alphas[n, :T, :U + 1].cpu().numpy(), orc.alphas(lp), rtol=1e-6, atol=1e-3)
        np.testing.assert_allclose(betas[n, :T, :U + 1].cpu().numpy(), orc.betas(lp), rtol=1e-6, atol=1e-3)


def test_uniform_lattice_of_tiny_probabilities_matches_the_closed_form():
    """One log-probability c = -66 nats (2^-95) everywhere: the loss is (T+U)*(-c) minus the log
    of the number of paths, C(T+U-1, U); sixteen steps shrink a value by 2^-1523, which the linear
    walk's per-block rescaling must carry."""
    c = -66.0
    lx, ly = [70, 30], [20, 90]
    b = _logprob_case(lx, ly, 6, c, c)
    dev = run_device(b, False)
    want = [-(T + U) * c - (math.lgamma(T + U) - math.lgamma(U + 1) - math.lgamma(T)) for T, U in zip(lx, ly)]
    np.testing.assert_allclose(dev["costs"], want, rtol=LOSS_RTOL)
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "logprob")
    np.testing.assert_allclose(dev["G"], ref["G"], rtol=0, atol=GRAD_ATOL)


@pytest.mark.parametrize("with_grad", [True, False])
@pytest.mark.parametrize("N", [1, 5, 64, 150])
def test_reduction_folded_into_the_forward_call(with_grad, N):
    """cwr_forward_reduced / cwr_loss_reduced: sum and mean of the costs come out of the call that
    computes them (cwarp_rnnt/__init__.py:66-71), identical from run to run."""
    pkg = _pkg()
    rng = np.random.default_rng(N)
    b = make_batch(rng.integers(1, 20, N), rng.integers(0, 9, N), 12, seed=N)
    dev = torch.device("cuda:0")
    xs = b["x"].to(dev)
    lx, ly = torch.from_numpy(b["lx"]).to(dev), torch.from_numpy(b["ly"]).to(dev)
    ys = torch.from_numpy(b["yp"]).to(dev)
    seen = set()
    for _ in range(3):
        costs, st = pkg.rnnt_forward(xs, lx, ys, ly, 0, True, with_grad=with_grad, reduce=True)
        red = st.reduced.cpu().numpy()
        c = costs.double().cpu().numpy()
        np.testing.assert_allclose(red[0], c.sum(), rtol=1e-6)
        np.testing.assert_allclose(red[1], c.mean(), rtol=1e-6)
        seen.add((float(red[0]), float(red[1])))
    assert len(seen) == 1
    ref = orc.loss_and_grad(b["x_ref"], b["lx"], b["yp"], b["ly"], 0, "fused", want_dense=False)
    np.testing.assert_allclose(red[1], ref["costs"].mean(), rtol=LOSS_RTOL)


def test_reduction_is_nan_when_a_sequence_is_skipped():
    pkg = _pkg()
    b = make_batch([6, 4, 9], [2, 3, 1], 10, seed=2)
    dev = torch.device("cuda:0")
    xs = b["x"].to(dev)
    lx = torch.tensor([6, 0, 9], dtype=torch.int32, device=dev)       # a sequence without frames
    ly = torch.from_numpy(b["ly"]).to(dev)
    ys = torch.from_numpy(b["yp"]).to(dev)
    costs, st = pkg.rnnt_forward(xs, lx, ys, ly, 0, True, reduce=True)
    assert int(st.status[0].item()) & 2
    assert torch.isnan(costs[1]) and torch.isnan(st.reduced).all()
    lx0 = torch.zeros(3, dtype=torch.int32, device=dev)                # nothing usable at all
    costs, st = pkg.rnnt_forward(xs, lx0, ys, ly, 0, True, reduce=True)
    assert torch.isnan(costs).all() and torch.isnan(st.reduced).all()


def test_peaked_rows_keep_the_absolute_accuracy_of_small_costs():
    """Logits of large magnitude over a tiny vocabulary: most rows are one-hot, log-probabilities of
    the likely entries are ~1e-6 below zero and a cost can be a few hundredths of a nat while the
    row maxima are ~25.  The log-probabilities must not inherit the rounding of the fp32
    log-sum-exp (half an ulp of 25 per cell)."""
    rng = np.random.default_rng(4242)
    for case in range(60):
        N = 12
        lx = rng.integers(1, 40, N)
        ly = rng.integers(0, 30, N)
        dtype = ["f32", "bf16", "f64"][case % 3]
        b = make_batch(lx, ly, 2, seed=int(rng.integers(1 << 30)), sigma=12.0, dtype=dtype, blank=case % 2)
        check_case(b, True, "2d", dtype=dtype, seed=case)


def test_near_certain_sequences_do_not_flag_a_mismatch():
    """A blank that is all but certain and sequences without labels: costs of ~1e-7, where the
    reference's relative forward/backward rule (cwarp_cuda_rnnt_kernel.cu:353-366) compares two
    roundings of zero.  No flag, costs within 1e-6 of the oracle."""
    b = make_batch([52, 46, 10, 2], [0, 80, 56, 0], 24, seed=3, dtype="bf16", blank=14)
    x = b["x"].float()
    x[:, 14] += 25.0
    b["x"] = x.to(torch.bfloat16)
    b["x_ref"] = b["x"].double().numpy()
    check_case(b, True, "2d", dtype="bf16")


# ----------------------------------------------------------------------------- randomised sweep
@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_against_oracle(seed):
    """Twenty random batches per seed: sizes, vocabularies (aligned or not), storage types, modes,
    blank positions, label layouts and logit scales drawn together, so that combinations no
    hand-written case lists still meet the oracle."""
    rng = np.random.default_rng(9000 + seed)
    for case in range(20):
        N = int(rng.integers(1, 9))
        big_u = rng.random() < 0.15
        lx = rng.integers(1, 40, N)
        ly = rng.integers(0, 200 if big_u else 30, N)
        V = int(rng.choice([2, 3, 7, 16, 29, 41, 64, 96, 130, 255, 256, 300, 511, 1024, 1031, 2048, 4099]))
        if (lx * (ly + 1)).sum() * V > 6e6:
            V = int(rng.choice([7, 16, 41, 64]))
        dtype = str(rng.choice(["f32", "f32", "f32", "f16", "bf16", "f64"]))
        fused = bool(rng.integers(0, 2))
        blank = int(rng.integers(0, V))
        sigma = float(rng.choice([0.5, 1.0, 2.0, 6.0]))
        labels = str(rng.choice(["2d", "1d"]))
        b = make_batch(lx, ly, V, seed=int(rng.integers(1 << 30)), sigma=sigma, dtype=dtype, blank=blank,
                       normalised=not fused)
        try:
            check_case(b, fused, labels, dtype=dtype, seed=case)
        except AssertionError as err:
            raise AssertionError(f"seed {seed} case {case}: N={N} lx={lx.tolist()} ly={ly.tolist()} V={V} "
                                 f"{dtype} fused={fused} blank={blank} sigma={sigma} labels={labels}\n{err}")


@pytest.mark.parametrize("seed", range(6))
def test_random_hard_regimes_against_oracle(seed):
    """Twenty-five random batches per seed from the regimes that leave the comfortable number range:
    steep logits (sigma 20 to 80), one column shifted far from the others, -inf entries no label
    uses, many strips (up to 2500 labels: past 2047 the sequential walk) and long sequences (up to 900 frames)."""
    rng = np.random.default_rng(31000 + seed)
    for case in range(25):
        N = int(rng.integers(1, 5))
        kind = str(rng.choice(["steep", "columns", "mask", "strips", "longt"]))
        lx = rng.integers(1, 60, N)
        ly = rng.integers(0, 90, N)
        V = int(rng.choice([3, 8, 24, 64, 130]))
        fused = bool(rng.integers(0, 2))
        sigma = float(rng.choice([20.0, 40.0, 80.0])) if kind == "steep" else 1.0
        if kind == "strips":
            # up to twenty strips of 128 labels: past sixteen, the sequential log-domain walk
            ly, lx, V = rng.integers(60, 2500 if rng.random() < 0.4 else 1300, N), rng.integers(1, 50, N), int(rng.choice([3, 8]))
        if kind == "longt":
            lx, ly, V = rng.integers(300, 900, N), rng.integers(0, 70, N), int(rng.choice([3, 8]))
        dtype = str(rng.choice(["f32", "f32", "f16", "bf16", "f64"]))
        blank = int(rng.integers(0, V))
        b = make_batch(lx, ly, V, seed=int(rng.integers(1 << 30)), sigma=sigma, dtype=dtype, blank=blank,
                       normalised=not fused)
        if kind in ("columns", "mask"):
            x = b["x"].clone().float()
            if kind == "columns" and fused:
                x[:, blank] += float(rng.choice([-30.0, -50.0, 25.0]))
            elif kind == "columns":
                x[:, blank] = float(rng.choice([-10.0, -30.0, -45.0, -62.0]))
            else:
                used = set(np.unique(b["yp"]).tolist()) | {blank}
                free = [v for v in range(V) if v not in used]
                if free:
                    x[:, free[: max(1, len(free) // 2)]] = -float("inf")
            b["x"] = x.to(TORCH_DT[dtype])
            b["x_ref"] = b["x"].double().numpy()
        try:
            check_case(b, fused, str(rng.choice(["2d", "1d"])), dtype=dtype, seed=case)
        except AssertionError as err:
            raise AssertionError(f"seed {seed} case {case} ({kind}): N={N} lx={lx.tolist()} ly={ly.tolist()} V={V} "
                                 f"{dtype} fused={fused} blank={blank} sigma={sigma}\n{err}")


@pytest.mark.parametrize("seed", range(4))
def test_random_small_batches_against_the_c_restatement(seed):
    """Four hundred small random batches per seed (one to six sequences, 1 to 120 frames, 0 to 300
    labels so that strips of every width and up to three strips occur, V from 3 to 32, both modes,
    logits of scale 0.5 to 12, some rows peaked, any blank) through the forward call, against the C
    restatement of the oracle (pinned to the NumPy oracle in tests/test_oracle_pins.py): costs within
    1e-5 relative + 1e-6 absolute, per-row gradients within 1e-4, no flag raised."""
    from oracle import build_c
    lib = build_c.load()
    pkg = _pkg()
    dev = torch.device("cuda:0")
    for case in range(400):
        rng = np.random.default_rng(7700000 + 1000 * seed + case)
        N = int(rng.integers(1, 7))
        kind = int(rng.integers(0, 4))
        tmax, umax = [(6, 4), (40, 70), (120, 140), (30, 300)][kind]
        lx = rng.integers(1, tmax + 1, N).astype(np.int32)
        ly = rng.integers(0, umax + 1, N).astype(np.int32)
        if rng.random() < 0.2:
            ly[rng.integers(0, N)] = 0
        if rng.random() < 0.2:
            lx[rng.integers(0, N)] = 1
        V = int(rng.choice([3, 4, 8, 17, 32]))
        fused = bool(rng.integers(0, 2))
        sigma = float(rng.choice([0.5, 1.0, 2.0, 5.0, 12.0]))
        R = int((lx.astype(np.int64) * (ly + 1)).sum())
        x = (rng.standard_normal((R, V)) * sigma).astype(np.float32)
        if rng.random() < 0.15:
            x[np.arange(R), rng.integers(0, V, R)] += 30.0
        if not fused:
            x = orc.log_softmax(x.astype(np.float64)).astype(np.float32)
        blank = int(rng.integers(0, V))
        yp = np.zeros((N, max(int(ly.max()), 1)), dtype=np.int32)
        for n in range(N):
            lab = rng.integers(0, V - 1, int(ly[n])).astype(np.int32)
            lab[lab >= blank] += 1
            yp[n, : ly[n]] = lab
        ref = build_c.loss_and_grad(lib, x, lx, yp, ly, blank, fused, None, want_G=True, want_grad=False)
        costs, st = pkg.rnnt_forward(torch.from_numpy(x).to(dev), torch.from_numpy(lx).to(dev),
                                     torch.from_numpy(yp).to(dev), torch.from_numpy(ly).to(dev), blank, fused)
        what = f"seed {seed} case {case}: lx={lx.tolist()} ly={ly.tolist()} V={V} fused={fused} sigma={sigma} blank={blank}"
        assert int(st.status[0].item()) == 0, what
        np.testing.assert_allclose(costs.cpu().numpy(), ref["costs"], rtol=LOSS_RTOL, atol=1e-6, err_msg=what)
        np.testing.assert_allclose(st.grads.cpu().numpy(), ref["G"], rtol=0, atol=GRAD_ATOL, err_msg=what)
