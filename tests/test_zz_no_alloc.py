"""cwr_forward_noalloc (scratch inside the library, no allocation) against cwr_forward on the same
inputs, through the C ABI: two calls in a row on one GPU, the second on a smaller batch, so that
what the first call left in the shared scratch must not leak into the second."""
import numpy as np
import pytest
import torch

from oracle import rnnt_oracle as orc

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-4


def _batch(lx, ly, V, seed, sigma):
    rng = np.random.default_rng(seed)
    lx = np.asarray(lx, np.int32)
    ly = np.asarray(ly, np.int32)
    R = int(orc.row_offsets_i64(lx, ly)[-1])
    x = (rng.standard_normal((R, V)) * sigma).astype(np.float32)
    yp = np.zeros((len(lx), int(ly.max())), np.int32)
    for n in range(len(lx)):
        yp[n, : ly[n]] = rng.integers(1, V, int(ly[n]))
    return dict(lx=lx, ly=ly, yp=yp, x=x, R=R, V=V, N=len(lx))


def _call(lib, b, fused, noalloc, watch_memory=False):
    from compactwarprnntloss_amd import _lib
    dev = torch.device("cuda:0")
    N, R, V = b["N"], b["R"], b["V"]
    max_u = b["yp"].shape[1]
    x = torch.from_numpy(b["x"]).to(dev)
    lx, ly, y = (torch.from_numpy(b[k]).to(dev) for k in ("lx", "ly", "yp"))
    row_off = torch.empty(N + 1, dtype=torch.int64, device=dev)
    lab_off = torch.empty(N + 1, dtype=torch.int64, device=dev)
    status = torch.empty(4, dtype=torch.int32, device=dev)
    # outputs start from a pattern no result can be mistaken for
    rowinfo = torch.full((R, 2), -7, dtype=torch.int32, device=dev)
    lse = torch.full((R,), float("nan"), device=dev)
    grads = torch.full((R, 2), float("nan"), device=dev)
    costs = torch.full((N,), float("nan"), device=dev)
    mode = _lib.MODE_FUSED if fused else _lib.MODE_LOGPROB
    head = (x.data_ptr(), _lib.F32, R, V, lx.data_ptr(), ly.data_ptr(), y.data_ptr(), max_u, y.numel(), N, 0, mode,
            max_u)
    tail = (row_off.data_ptr(), lab_off.data_ptr(), status.data_ptr(), rowinfo.data_ptr(), lse.data_ptr(),
            grads.data_ptr(), costs.data_ptr(), torch.cuda.current_stream().cuda_stream)
    if noalloc:
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
        rc = lib.cwr_forward_noalloc(*head, *tail)
        torch.cuda.synchronize()
        if watch_memory:  # once the library's code is resident, a call must leave the free memory alone
            assert torch.cuda.mem_get_info(dev)[0] == free_before
    else:
        nbytes = lib.cwr_workspace_bytes(N, R, max_u)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.cwr_forward(*head, ws.data_ptr(), nbytes, *tail)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    out = dict(row_off=row_off, lab_off=lab_off, status=status[:1], rowinfo=rowinfo, grads=grads, costs=costs)
    if fused:
        out["lse"] = lse
    return {k: v.cpu().numpy() for k, v in out.items()}


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False])
def test_noalloc_forward_matches_forward_twice_in_a_row(fused):
    from compactwarprnntloss_amd import _lib
    lib = _lib.load()
    sigma = 2.0
    big = _batch([120, 90, 150, 33, 70, 1], [70, 20, 130, 0, 64, 5], 96, seed=11, sigma=sigma)
    small = _batch([40, 7, 25], [9, 3, 66], 96, seed=12, sigma=sigma)
    for b in (big, small):  # same GPU, same scratch; the second batch is the smaller one
        if not fused:
            b["x"] = orc.log_softmax(b["x"].astype(np.float64)).astype(np.float32)
        got = _call(lib, b, fused, noalloc=True, watch_memory=b is small)
        want = _call(lib, b, fused, noalloc=False)
        assert int(got["status"][0]) == 0 and int(want["status"][0]) == 0
        for k in ("row_off", "lab_off", "rowinfo"):  # integer outputs: exact
            assert np.array_equal(got[k], want[k]), k
        np.testing.assert_allclose(got["costs"], want["costs"], rtol=LOSS_RTOL, atol=0)
        np.testing.assert_allclose(got["grads"], want["grads"], rtol=0, atol=GRAD_ATOL)
        if fused:
            np.testing.assert_allclose(got["lse"], want["lse"], rtol=1e-6, atol=0)
        # the same kernels on the same inputs: the two entry points agree to the last bit
        for k in ("costs", "grads") + (("lse",) if fused else ()):
            assert np.array_equal(got[k], want[k]), k
        # and with the oracle
        ref = orc.loss_and_grad(b["x"].astype(np.float64), b["lx"], b["yp"], b["ly"], 0,
                                "fused" if fused else "logprob", want_dense=False)
        np.testing.assert_allclose(got["costs"], ref["costs"], rtol=LOSS_RTOL, atol=1e-6)
        np.testing.assert_allclose(got["grads"], ref["G"], rtol=0, atol=GRAD_ATOL)


def test_noalloc_forward_rejects_what_its_scratch_cannot_hold():
    from compactwarprnntloss_amd import _lib
    lib = _lib.load()
    N, V, max_u = 4, 8, 400
    R = 3_000_000
    assert lib.cwr_workspace_bytes(N, R, max_u) > _lib.NOALLOC_SCRATCH_BYTES
    one = np.zeros(16, dtype=np.int64)  # host memory, never read: the sizes are refused before any HIP call
    p = one.ctypes.data
    rc = lib.cwr_forward_noalloc(p, _lib.F32, R, V, p, p, p, max_u, N * max_u, N, 0, _lib.MODE_FUSED, max_u,
                                 p, p, p, p, p, p, p, None)
    assert rc == 8 and "scratch" in _lib.strerror(rc)  # CWR_ERR_TOO_LARGE
