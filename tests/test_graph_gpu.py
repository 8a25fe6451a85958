"""The forward and backward calls launch kernels only (no allocation, copy, memset or
synchronisation inside the library), so a caller may record them into a HIP graph.  The graph is
replayed several times with new logits and labels written into the captured buffers, with eager
work and synchronisations in between, and every replay is compared with the eager result."""
import numpy as np
import pytest
import torch

from compactwarprnntloss_amd import workloads as wl
from oracle import rnnt_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.mark.parametrize("fused", [True, False])
def test_graph_replays_match_eager(fused):
    import compactwarprnntloss_amd as pkg
    cfg = wl.make_config(2, scale=0.2)
    lx_np, ly_np = cfg["lx"].astype(np.int32), cfg["ly"].astype(np.int32)
    N, V, R = cfg["N"], 256, cfg["R"]
    gen = torch.Generator(device=DEV).manual_seed(1)

    def fresh():
        x = torch.randn((R, V), device=DEV, generator=gen) * 2
        if not fused:
            x = torch.log_softmax(x, dim=1)
        y = torch.randint(1, V, (N, int(ly_np.max())), device=DEV, dtype=torch.int32, generator=gen)
        return x, y

    lx, ly = torch.from_numpy(lx_np).to(DEV), torch.from_numpy(ly_np).to(DEV)
    x, y = fresh()
    go = torch.full((N,), 0.5, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up on the capture stream, as graph capture asks for
        c, st = pkg.rnnt_forward(x, lx, y, ly, 0, fused)
        pkg.rnnt_backward(x, lx, y, ly, 0, st, go)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        costs_g, st_g = pkg.rnnt_forward(x, lx, y, ly, 0, fused)
        grad_g = pkg.rnnt_backward(x, lx, y, ly, 0, st_g, go)

    for replay in range(4):
        xn, yn = fresh()
        x.copy_(xn)
        y.copy_(yn)
        graph.replay()
        torch.cuda.synchronize()
        costs_e, st_e = pkg.rnnt_forward(x, lx, y, ly, 0, fused)     # eager work between replays
        grad_e = pkg.rnnt_backward(x, lx, y, ly, 0, st_e, go)
        torch.cuda.synchronize()
        assert int(st_g.status[0].item()) & ~8 == 0
        assert torch.equal(costs_g, costs_e), replay
        assert torch.equal(grad_g, grad_e), replay
        assert torch.isfinite(costs_g).all()
