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
