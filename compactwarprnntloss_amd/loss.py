"""Host side of the compact RNN-T loss: the `transducer_loss` entry point and its autograd node.

Mirrors cwarp_rnnt/__init__.py:10-73 of CompactWarpRNNTLoss (same positional arguments, same
asserts, same reductions) on top of the C ABI in include/cwarp_rnnt_hip.h.  Differences, all
additive keyword arguments:

  gather             accepted for call-site compatibility with warp_rnnt-style callers; the
                     gather is unconditional here, as it is in the reference (cwarp_cuda.cpp:79,105)
  fused_log_softmax  False (default): x holds log-probabilities and the gradient is the
                     reference's sparse one.  True: x holds raw logits, log-softmax over V is
                     fused into the gather pass, the gradient w.r.t. the logits is dense.
  max_u              host-known upper bound of max(ly) for concatenated 1-D labels
  validate           read the device status word back (one synchronisation) and raise on
                     data-dependent problems.  Off by default: the hot path never synchronises.
"""
from __future__ import annotations

from typing import Any, Optional

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16,
           torch.float64: _lib.F64}


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _label_args(ys: torch.Tensor):
    """(y_stride, y_len) for padded 2-D or concatenated 1-D labels."""
    if ys.dim() == 2:
        return (ys.size(1), ys.numel())
    return (-1, ys.numel())


class ForwardState:
    """What a forward call leaves behind for the backward pass and for inspection."""
    __slots__ = ("row_off", "lab_off", "status", "rowinfo", "lse", "grads", "workspace", "N", "R", "V", "mode",
                 "max_u")


def _check_inputs(xs, lx, ys, ly):
    if not xs.is_cuda:
        raise RuntimeError("xs must be a CUDA tensor")          # cwarp_cuda.cpp:46 CHECK_CUDA
    if not xs.is_contiguous():
        raise RuntimeError("xs must be contiguous")            # cwarp_cuda.cpp:47
    for name, t in (("lx", lx), ("ys", ys), ("ly", ly)):       # cwarp_cuda.cpp:49-52 CHECK_INPUT
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.dtype != torch.int32:
            raise RuntimeError(f"{name} must be torch::ScalarType::Int")
    if xs.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {xs.dtype}")
    if xs.dim() != 2:
        raise RuntimeError("xs must be (sum_i T_i*(U_i+1), V)")


def rnnt_forward(xs, lx, ys, ly, blank: int, fused: bool, max_u: Optional[int] = None,
                 with_grad: bool = True):
    """Binding of cwr_forward / cwr_loss.  Returns (costs fp32 (N,), ForwardState)."""
    _check_inputs(xs, lx, ys, ly)
    lib = _lib.load()
    dev = xs.device
    N = lx.numel()
    R, V = xs.shape
    y_stride, y_len = _label_args(ys)
    if max_u is None:
        max_u = ys.size(1) if ys.dim() == 2 else ys.numel()
    mode = _lib.MODE_FUSED if fused else _lib.MODE_LOGPROB

    st = ForwardState()
    st.N, st.R, st.V, st.mode, st.max_u = N, R, V, mode, int(max_u)
    meta = torch.empty(2 * (N + 1) + 2, dtype=torch.int64, device=dev)
    st.row_off = meta[: N + 1]
    st.lab_off = meta[N + 1: 2 * (N + 1)]
    st.status = meta[2 * (N + 1):].view(torch.int32)
    ws_bytes = lib.cwr_workspace_bytes(N, R, int(max_u))
    st.workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    costs = torch.empty(N, dtype=torch.float32, device=dev)
    st.lse = torch.empty(R, dtype=torch.float32, device=dev) if (fused and with_grad) else None
    st.grads = torch.empty((R, 2), dtype=torch.float32, device=dev) if with_grad else None
    st.rowinfo = torch.empty((R, 2), dtype=torch.int32, device=dev) if with_grad else None

    with torch.cuda.device(dev):
        common = (xs.data_ptr(), _DTYPES[xs.dtype], R, V, lx.data_ptr(), ly.data_ptr(), ys.data_ptr(),
                  y_stride, y_len, N, int(blank), mode, int(max_u),
                  st.workspace.data_ptr(), ws_bytes, st.row_off.data_ptr(), st.lab_off.data_ptr(),
                  st.status.data_ptr())
        if with_grad:
            rc = lib.cwr_forward(*common, st.rowinfo.data_ptr(),
                                 st.lse.data_ptr() if st.lse is not None else None,
                                 st.grads.data_ptr(), costs.data_ptr(), _stream_ptr(dev))
            _lib.check(rc, "cwr_forward")
        else:
            rc = lib.cwr_loss(*common, costs.data_ptr(), _stream_ptr(dev))
            _lib.check(rc, "cwr_loss")
    return costs, st


def rnnt_backward(xs, lx, ys, ly, blank: int, st: ForwardState, grad_costs: torch.Tensor,
                  out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """Binding of cwr_backward.  Returns the (R,V) gradient in xs.dtype.

    grad_costs holds d(total)/d(cost): one value per sequence, or a single value that is
    broadcast (stride 0); `scale` multiplies it (1/N of a mean reduction)."""
    lib = _lib.load()
    dev = lx.device
    fused = st.mode == _lib.MODE_FUSED
    y_stride, y_len = _label_args(ys)
    gc = grad_costs
    if gc.dtype != torch.float32 or not gc.is_contiguous():
        gc = gc.to(dtype=torch.float32).contiguous()
    if gc.numel() not in (1, st.N):
        raise RuntimeError("grad_costs must hold one value or one value per sequence")
    stride = 0 if (gc.numel() == 1 and st.N != 1) else 1
    dtype = xs.dtype
    if out is None:
        out = torch.empty((st.R, st.V), dtype=dtype, device=dev)
    with torch.cuda.device(dev):
        rc = lib.cwr_backward(xs.data_ptr() if fused else None, _DTYPES[dtype], st.R, st.V,
                              lx.data_ptr(), ly.data_ptr(), ys.data_ptr(), y_stride, y_len, st.N,
                              int(blank), st.mode, st.row_off.data_ptr(), st.lab_off.data_ptr(),
                              st.rowinfo.data_ptr(), st.grads.data_ptr(),
                              st.lse.data_ptr() if fused else None, gc.data_ptr(), stride, float(scale),
                              out.data_ptr(), _stream_ptr(dev))
        _lib.check(rc, "cwr_backward")
    return out


def _raise_on_flags(st: ForwardState):
    flags = int(st.status[0].item())
    hard = flags & ~_lib.FLAG_FB_MISMATCH
    if hard:
        raise RuntimeError("transducer_loss: " + _lib.describe_flags(hard))


class _TransLoss(torch.autograd.Function):
    """cwarp_rnnt/__init__.py:10-29: gradient path when xs requires grad, beta-only path otherwise.
    The reduction (cwarp_rnnt/__init__.py:66-71) is part of the node, so that the backward pass
    receives one scalar for 'mean' / 'sum' and folds it (and the 1/N) into the gradient kernel
    instead of materialising an expanded per-sequence tensor."""

    @staticmethod
    def forward(ctx: Any, xs, lx, ys, ly, blank, fused, max_u, validate, reduction):
        need_grad = xs.requires_grad
        costs, st = rnnt_forward(xs, lx, ys, ly, blank, fused, max_u, with_grad=need_grad)
        if validate:
            _raise_on_flags(st)
        if need_grad:
            st.workspace = None  # alpha / beta are not needed again
            ctx.state = st
            ctx.blank = blank
            ctx.reduction = reduction
            ctx.save_for_backward(xs, lx, ys, ly)
        if xs.dtype not in (torch.float16, torch.bfloat16):
            costs = costs.to(xs.dtype)
        if reduction == "mean":
            return costs.mean()
        if reduction == "sum":
            return costs.sum()
        return costs

    @staticmethod
    def backward(ctx: Any, grad_outputs):
        xs, lx, ys, ly = ctx.saved_tensors
        scale = 1.0 / ctx.state.N if ctx.reduction == "mean" else 1.0
        grad_input = rnnt_backward(xs, lx, ys, ly, ctx.blank, ctx.state, grad_outputs, scale=scale)
        return grad_input, None, None, None, None, None, None, None, None


def transducer_loss(x: torch.Tensor, lx: torch.Tensor, y: torch.Tensor, ly: torch.Tensor, blank: int = 0,
                    reduction: Optional[str] = "mean", *, gather: bool = True,
                    fused_log_softmax: bool = False, max_u: Optional[int] = None,
                    validate: bool = False) -> torch.Tensor:
    """Transducer loss for compact-layout input (cwarp_rnnt/__init__.py:32-73).

    x   (sum_i T_i*(U_i+1), V) log-probabilities (or raw logits with fused_log_softmax=True)
    lx  (N,) int32 frame counts;  ly (N,) int32 label counts
    y   (N, Umax) int32 padded labels as in the reference, or (sum_i U_i,) concatenated labels
    """
    assert lx.dtype == torch.int32
    assert ly.dtype == torch.int32
    assert y.dtype == torch.int32
    assert reduction in ["mean", "sum", "none"] or reduction is None
    assert y.dim() in (1, 2)
    if y.dim() == 2:
        assert y.size(0) == lx.size(0)
        assert y.size(0) == ly.size(0)
    assert lx.size(0) == ly.size(0)
    assert blank >= 0 and blank < x.size(-1)
    del gather  # always on, as in the reference
    # x: (STU, V)
    assert x.dim() == 2, "input must be compact: (sum_i T_i*(U_i+1), V)"

    if reduction not in ("mean", "sum", "none", None):
        raise ValueError
    return _TransLoss.apply(x, lx, y, ly, blank, bool(fused_log_softmax), max_u, bool(validate),
                            reduction if reduction in ("mean", "sum") else "none")
