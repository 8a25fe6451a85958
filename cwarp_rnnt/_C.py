"""The three functions the reference's extension module exports (cwarp_cuda.cpp:138-153), with the
same names, arguments and return values, on top of the C ABI of include/cwarp_rnnt_hip.h.

The reference's Python layer does `import cwarp_rnnt._C as core` and calls
`core._cwarp_rnnt_forward`, `core._cwarp_rnnt_loss` and `core._cwarp_rnnt_backward`
(cwarp_rnnt/__init__.py:3,14,20,27); an autograd node written against those three calls runs
unchanged on this module.  Semantics are the reference's: `xs` holds log-probabilities, the
gradient is non-zero in the blank and label columns only.

Differences a caller can observe:
  - `_cwarp_rnnt_backward` does not rescale `grads` in place (cwarp_cuda_rnnt_kernel.cu:518-519
    does); calling it twice on one forward result gives the same answer twice.
  - `alphas` / `betas` need the largest frame count on the host, which costs one synchronisation
    (the reference pays four per forward call, cwarp_cuda_gather_kernel.cu:85-86 and
    cwarp_cuda_rnnt_kernel.cu:395-396).  Set `RETURN_LATTICE = False` to get `None` for both and a
    forward call that never synchronises; `_TransLoss` drops them anyway
    (cwarp_rnnt/__init__.py:14-16).
"""
from __future__ import annotations

import torch

from compactwarprnntloss_amd import _lib
from compactwarprnntloss_amd.loss import _DTYPES, _check_inputs, _stream_ptr, lattice_state, rnnt_forward

RETURN_LATTICE = True


def _cwarp_rnnt_forward(xs: torch.Tensor, lx: torch.Tensor, ys: torch.Tensor, ly: torch.Tensor, blank: int):
    """cwarp_cuda.cpp:84-108: (costs (N,), grads (R,2), alphas (N,T,U+1), betas (N,T,U+1)), all in
    xs.dtype; T = max(lx), U+1 = ys.size(1)+1 (the reference asserts ys.size(1) == max(ly))."""
    costs, st = rnnt_forward(xs, lx, ys, ly, int(blank), fused=False)
    alphas = betas = None
    if RETURN_LATTICE:
        t_pad = int(lx.max().item()) if lx.numel() else 0
        alphas, betas = lattice_state(st, lx, ly, t_pad, ys.size(1) + 1)
        alphas, betas = alphas.to(xs.dtype), betas.to(xs.dtype)
    return costs.to(xs.dtype), st.grads.to(xs.dtype), alphas, betas


def _cwarp_rnnt_loss(xs: torch.Tensor, lx: torch.Tensor, ys: torch.Tensor, ly: torch.Tensor, blank: int):
    """cwarp_cuda.cpp:58-82: costs (N,) in xs.dtype, from the beta recursion alone."""
    costs, _ = rnnt_forward(xs, lx, ys, ly, int(blank), fused=False, with_grad=False)
    return costs.to(xs.dtype)


def _cwarp_rnnt_backward(grads: torch.Tensor, grad_costs: torch.Tensor, ys: torch.Tensor, lx: torch.Tensor,
                         ly: torch.Tensor, blank: int, V: int) -> torch.Tensor:
    """cwarp_cuda.cpp:110-136: the (R,V) gradient w.r.t. the log-probabilities, zero except
    [r, blank] = grads[r,0] * grad_costs[n(r)] and [r, label(r)] = grads[r,1] * grad_costs[n(r)]
    (the label entry written last, cwarp_cuda_gather_kernel.cu:70-73)."""
    if grads.dim() != 2 or grads.size(1) != 2:
        raise RuntimeError("grads must be (sum_i T_i*(U_i+1), 2)")
    if grads.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {grads.dtype}")
    _check_inputs(grads, lx, ys, ly)
    if not grad_costs.is_cuda:
        raise RuntimeError("grad_costs must be a CUDA tensor")  # cwarp_cuda.cpp:118 CHECK_CUDA
    lib = _lib.load()
    dev = grads.device
    N, R = lx.numel(), grads.size(0)
    if grad_costs.numel() != N:
        raise RuntimeError("grad_costs must hold one value per sequence")
    g32 = grads if grads.dtype == torch.float32 else grads.float()
    g32 = g32.contiguous()
    gc = grad_costs.to(dtype=torch.float32).contiguous()
    y_stride, y_len = (ys.size(1), ys.numel()) if ys.dim() == 2 else (-1, ys.numel())
    meta = torch.empty(2 * (N + 1) + 2, dtype=torch.int64, device=dev)
    row_off, lab_off = meta[: N + 1], meta[N + 1: 2 * (N + 1)]
    status = meta[2 * (N + 1):].view(torch.int32)
    rowinfo = torch.empty((R, 2), dtype=torch.int32, device=dev)
    out = torch.empty((R, int(V)), dtype=grads.dtype, device=dev)
    with torch.cuda.device(dev):
        stream = _stream_ptr(dev)
        # the reference rebuilds its offsets from lx and ly here as well (cwarp_cuda.cpp:124-129)
        _lib.check(lib.cwr_offsets(lx.data_ptr(), ly.data_ptr(), N, R, row_off.data_ptr(), lab_off.data_ptr(),
                                   status.data_ptr(), stream), "cwr_offsets")
        _lib.check(lib.cwr_rowinfo(lx.data_ptr(), ly.data_ptr(), ys.data_ptr(), y_stride, y_len, N, R, int(V),
                                   row_off.data_ptr(), lab_off.data_ptr(), rowinfo.data_ptr(), stream), "cwr_rowinfo")
        _lib.check(lib.cwr_backward(None, _DTYPES[grads.dtype], R, int(V), lx.data_ptr(), ly.data_ptr(),
                                    ys.data_ptr(), y_stride, y_len, N, int(blank), _lib.MODE_LOGPROB,
                                    row_off.data_ptr(), lab_off.data_ptr(), rowinfo.data_ptr(), g32.data_ptr(), None,
                                    gc.data_ptr(), 1, 1.0, out.data_ptr(), stream), "cwr_backward")
    return out
