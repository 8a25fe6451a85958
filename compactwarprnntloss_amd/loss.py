"""Host side of the compact RNN-T loss: the `transducer_loss` entry point and its autograd node.

Mirrors cwarp_rnnt/__init__.py:10-73 of CompactWarpRNNTLoss (same positional arguments, same
asserts, same reductions) on top of the C ABI in include/cwarp_rnnt_hip.h.  Differences, all
additive keyword arguments:

  gather             accepted for call-site compatibility with warp_rnnt-style callers; the
                     gather is unconditional here, as it is in the reference (cwarp_cuda.cpp:79,105)
  fused_log_softmax  False (default): x holds log-probabilities and the gradient is the
                     reference's sparse one.  True: x holds raw logits, log-softmax over V is
                     fused into the gather pass, the gradient w.r.t. the logits is dense.
  x of 4 dims        a padded (N, T, U+1, V) tensor is packed first (pack_padded), as the
                     reference does through gather.cat (cwarp_rnnt/__init__.py:52-59)
  max_u              host-known upper bound of max(ly).  Padded labels give one for free (their
                     width); with concatenated 1-D labels and no max_u the maximum of ly is read
                     back from the device (one synchronisation per call)
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
                 "max_u", "reduced")


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
                 with_grad: bool = True, reduce: bool = False):
    """Binding of cwr_forward / cwr_loss (and their *_reduced forms).  Returns (costs fp32 (N,),
    ForwardState); with reduce=True the state also holds `reduced` = (sum, mean) of the costs."""
    _check_inputs(xs, lx, ys, ly)
    lib = _lib.load()
    dev = xs.device
    N = lx.numel()
    R, V = xs.shape
    y_stride, y_len = _label_args(ys)
    if max_u is None:
        # padded labels bound max(ly) by their width.  Concatenated labels carry no such bound (their
        # total would size the workspace and the lattice kernel for one sequence holding every label
        # of the batch: 8x the memory on a typical batch), so the true maximum is read back: one
        # synchronisation, which callers avoid by passing max_u.
        max_u = ys.size(1) if ys.dim() == 2 else (int(ly.max().item()) if ly.numel() else 0)
    mode = _lib.MODE_FUSED if fused else _lib.MODE_LOGPROB

    st = ForwardState()
    st.N, st.R, st.V, st.mode, st.max_u = N, R, V, mode, int(max_u)
    meta = torch.empty(2 * (N + 1) + 2, dtype=torch.int64, device=dev)
    st.row_off = meta[: N + 1]
    st.lab_off = meta[N + 1: 2 * (N + 1)]
    st.status = meta[2 * (N + 1):].view(torch.int32)
    ws_bytes = lib.cwr_workspace_bytes(N, R, int(max_u))
    st.workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    # the costs and, behind them, their sum and mean
    cbuf = torch.empty(N + 2, dtype=torch.float32, device=dev)
    costs = cbuf[:N]
    st.reduced = cbuf[N:] if (reduce and N > 0) else None
    st.lse = torch.empty(R, dtype=torch.float32, device=dev) if (fused and with_grad) else None
    st.grads = torch.empty((R, 2), dtype=torch.float32, device=dev) if with_grad else None
    st.rowinfo = torch.empty((R, 2), dtype=torch.int32, device=dev) if with_grad else None

    with torch.cuda.device(dev):
        common = (xs.data_ptr(), _DTYPES[xs.dtype], R, V, lx.data_ptr(), ly.data_ptr(), ys.data_ptr(),
                  y_stride, y_len, N, int(blank), mode, int(max_u),
                  st.workspace.data_ptr(), ws_bytes, st.row_off.data_ptr(), st.lab_off.data_ptr(),
                  st.status.data_ptr())
        red = (st.reduced.data_ptr(),) if st.reduced is not None else ()
        if with_grad:
            fn = lib.cwr_forward_reduced if red else lib.cwr_forward
            rc = fn(*common, st.rowinfo.data_ptr(), st.lse.data_ptr() if st.lse is not None else None,
                    st.grads.data_ptr(), costs.data_ptr(), *red, _stream_ptr(dev))
            _lib.check(rc, "cwr_forward")
        else:
            fn = lib.cwr_loss_reduced if red else lib.cwr_loss
            rc = fn(*common, costs.data_ptr(), *red, _stream_ptr(dev))
            _lib.check(rc, "cwr_loss")
    return costs, st


RESIDENT_JOINT_SIZES = tuple(range(128, 1025, 64))  # joint sizes whose rows a wave keeps in registers


def _joint_state(like, weight, bias, lx, ys, ly, R: int, max_u: Optional[int]):
    """Checks and allocations shared by the two joint_forward bindings."""
    if like.dtype not in (torch.float16, torch.bfloat16) or weight.dtype != like.dtype:
        raise RuntimeError("the joint rows (or f and g) and weight must all be float16 or all bfloat16")
    if weight.dim() != 2 or like.size(-1) != weight.size(1):
        raise RuntimeError("weight must be (V, H) with the joint dimension H of the rows")
    if like.size(-1) % 32 != 0:
        raise RuntimeError("the joint dimension must be a multiple of 32")
    if not weight.is_cuda or not weight.is_contiguous():
        raise RuntimeError("weight must be a contiguous CUDA tensor")
    lib = _lib.load()
    dev = like.device
    N = lx.numel()
    V = weight.size(0)
    if max_u is None:
        max_u = ys.size(1) if ys.dim() == 2 else (int(ly.max().item()) if ly.numel() else 0)
    b32 = None
    if bias is not None:
        if bias.numel() != V:
            raise RuntimeError("bias must hold one value per vocabulary entry")
        b32 = bias.detach().to(dtype=torch.float32).contiguous()
    st = ForwardState()
    st.N, st.R, st.V, st.mode, st.max_u = N, R, V, _lib.MODE_FUSED, int(max_u)
    meta = torch.empty(2 * (N + 1) + 2, dtype=torch.int64, device=dev)
    st.row_off = meta[: N + 1]
    st.lab_off = meta[N + 1: 2 * (N + 1)]
    st.status = meta[2 * (N + 1):].view(torch.int32)
    ws_bytes = lib.cwr_workspace_bytes(N, R, int(max_u))
    st.workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    costs = torch.empty(N, dtype=torch.float32, device=dev)
    st.reduced = None
    st.lse = torch.empty(R, dtype=torch.float32, device=dev)
    st.grads = torch.empty((R, 2), dtype=torch.float32, device=dev)
    st.rowinfo = torch.empty((R, 2), dtype=torch.int32, device=dev)
    return lib, st, costs, b32, ws_bytes


def joint_forward(h, weight, bias, lx, ys, ly, blank: int, max_u: Optional[int] = None):
    """Binding of cwr_joint_forward: the loss of logits = h @ weight.T + bias without ever storing
    them.  h (R,H) and weight (V,H) fp16 or bf16, bias (V,) or None.  Returns (costs fp32 (N,),
    ForwardState) like rnnt_forward in fused mode."""
    if h.dim() != 2:
        raise RuntimeError("h must be (R, H)")
    _check_inputs(h, lx, ys, ly)
    R, H = h.shape
    lib, st, costs, b32, ws_bytes = _joint_state(h, weight, bias, lx, ys, ly, R, max_u)
    dev = h.device
    V, N = st.V, st.N
    y_stride, y_len = _label_args(ys)
    with torch.cuda.device(dev):
        rc = lib.cwr_joint_forward(h.data_ptr(), weight.data_ptr(), b32.data_ptr() if b32 is not None else None,
                                   _DTYPES[h.dtype], R, H, V, lx.data_ptr(), ly.data_ptr(), ys.data_ptr(), y_stride,
                                   y_len, N, int(blank), st.max_u, st.workspace.data_ptr(), ws_bytes,
                                   st.row_off.data_ptr(), st.lab_off.data_ptr(), st.status.data_ptr(),
                                   st.rowinfo.data_ptr(), st.lse.data_ptr(), st.grads.data_ptr(), costs.data_ptr(),
                                   _stream_ptr(dev))
        _lib.check(rc, "cwr_joint_forward")
    return costs, st


def joint_forward_fg(f, g, act: int, weight, bias, lx, ys, ly, blank: int, total_rows: int,
                     max_u: Optional[int] = None, keep_rows: bool = False):
    """Binding of cwr_joint_forward_fg: the loss of logits = act(f[n,t] + g[n,u]) @ weight.T + bias
    with the joint rows formed inside the kernel.  f (N,T,H), g (N,U+1,H), weight (V,H) fp16 or bf16;
    act 0 / 1 / 2 = none / tanh / relu; H one of RESIDENT_JOINT_SIZES.  Returns (costs, ForwardState,
    h): h the (R,H) joint rows when keep_rows, else None."""
    if f.dim() != 3 or g.dim() != 3 or f.size(0) != g.size(0) or f.size(2) != g.size(2) or f.dtype != g.dtype:
        raise RuntimeError("f must be (N, T, H) and g (N, U+1, H) of one dtype")
    for name, t in (("f", f), ("g", g), ("lx", lx), ("ly", ly), ("y", ys)):
        if not t.is_cuda or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous CUDA tensor")
    if lx.dtype != torch.int32 or ly.dtype != torch.int32 or ys.dtype != torch.int32:
        raise RuntimeError("lx, ly and y must be int32")
    if lx.numel() != f.size(0) or ly.numel() != f.size(0):
        raise RuntimeError("lx, ly must hold one entry per sequence")
    H = f.size(2)
    if H not in RESIDENT_JOINT_SIZES:
        raise RuntimeError(f"joint dimension {H} not in {RESIDENT_JOINT_SIZES}: use compact_join + joint_forward")
    R = int(total_rows)
    lib, st, costs, b32, ws_bytes = _joint_state(f, weight, bias, lx, ys, ly, R, max_u)
    dev = f.device
    V, N = st.V, st.N
    y_stride, y_len = _label_args(ys)
    h = torch.empty((R, H), dtype=f.dtype, device=dev) if keep_rows else None
    with torch.cuda.device(dev):
        rc = lib.cwr_joint_forward_fg(f.data_ptr(), g.data_ptr(), int(act), f.size(1), g.size(1),
                                      h.data_ptr() if h is not None else None, weight.data_ptr(),
                                      b32.data_ptr() if b32 is not None else None, _DTYPES[f.dtype], R, H, V,
                                      lx.data_ptr(), ly.data_ptr(), ys.data_ptr(), y_stride, y_len, N, int(blank),
                                      st.max_u, st.workspace.data_ptr(), ws_bytes, st.row_off.data_ptr(),
                                      st.lab_off.data_ptr(), st.status.data_ptr(), st.rowinfo.data_ptr(),
                                      st.lse.data_ptr(), st.grads.data_ptr(), costs.data_ptr(), _stream_ptr(dev))
        _lib.check(rc, "cwr_joint_forward_fg")
    return costs, st, h


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


def lattice_state(st: ForwardState, lx, ly, t_pad: int, up_pad: int, with_alpha: bool = True):
    """Binding of cwr_export_lattice: (alphas, betas) as (N, t_pad, up_pad) float64 natural logs, zero
    outside each sequence's lattice, from the workspace a forward call left in `st` (the reference
    returns both from its forward, cwarp_cuda_rnnt_kernel.cu:383-384,496).  After a loss-only call
    only beta exists: pass with_alpha=False."""
    if st.workspace is None:
        raise RuntimeError("the forward state holds no workspace any more")
    lib = _lib.load()
    dev = lx.device
    alphas = torch.empty((st.N, t_pad, up_pad), dtype=torch.float64, device=dev) if with_alpha else None
    betas = torch.empty((st.N, t_pad, up_pad), dtype=torch.float64, device=dev)
    with torch.cuda.device(dev):
        rc = lib.cwr_export_lattice(lx.data_ptr(), ly.data_ptr(), st.N, st.R, st.max_u, st.workspace.data_ptr(),
                                    st.workspace.numel(), int(t_pad), int(up_pad),
                                    alphas.data_ptr() if with_alpha else None, betas.data_ptr(), _stream_ptr(dev))
        _lib.check(rc, "cwr_export_lattice")
    return alphas, betas


def _offsets(lx, ly, total_rows: int):
    """Binding of cwr_offsets: (row_off (N+1) int64, status 4 x int32) on the device."""
    lib = _lib.load()
    dev = lx.device
    N = lx.numel()
    meta = torch.empty(2 * (N + 1) + 2, dtype=torch.int64, device=dev)
    status = meta[2 * (N + 1):].view(torch.int32)
    with torch.cuda.device(dev):
        rc = lib.cwr_offsets(lx.data_ptr(), ly.data_ptr(), N, int(total_rows), meta.data_ptr(),
                             meta[N + 1:].data_ptr(), status.data_ptr(), _stream_ptr(dev))
        _lib.check(rc, "cwr_offsets")
    return meta[: N + 1], status


class _Pack(torch.autograd.Function):
    """Padded (N, T, U+1, V) -> compact (R, V) and its backward (cwr_pack / cwr_unpack)."""

    @staticmethod
    def forward(ctx: Any, x4, lx, ly, total_rows, row_off, status):
        lib = _lib.load()
        N, T, Up, V = x4.shape
        out = torch.empty((total_rows, V), dtype=x4.dtype, device=x4.device)
        with torch.cuda.device(x4.device):
            rc = lib.cwr_pack(x4.data_ptr(), _DTYPES[x4.dtype], N, T, Up, V, lx.data_ptr(), ly.data_ptr(),
                              row_off.data_ptr(), total_rows, out.data_ptr(), status.data_ptr(),
                              _stream_ptr(x4.device))
            _lib.check(rc, "cwr_pack")
        ctx.save_for_backward(lx, ly, row_off)
        ctx.shape = (N, T, Up, V)
        return out

    @staticmethod
    def backward(ctx: Any, g):
        lx, ly, row_off = ctx.saved_tensors
        N, T, Up, V = ctx.shape
        lib = _lib.load()
        g = g.contiguous()
        out = torch.empty((N, T, Up, V), dtype=g.dtype, device=g.device)
        with torch.cuda.device(g.device):
            rc = lib.cwr_unpack(g.data_ptr(), _DTYPES[g.dtype], N, T, Up, V, lx.data_ptr(), ly.data_ptr(),
                                row_off.data_ptr(), g.size(0), out.data_ptr(), _stream_ptr(g.device))
            _lib.check(rc, "cwr_unpack")
        return out, None, None, None, None, None


def _raise_on_status(status: torch.Tensor, what: str):
    """Reads a status word back (one synchronisation) and raises on any problem but a
    forward/backward mismatch, which the reference only reports."""
    hard = int(status[0].item()) & ~_lib.FLAG_FB_MISMATCH
    if hard:
        raise RuntimeError(f"{what}: " + _lib.describe_flags(hard))


def pack_padded(x: torch.Tensor, lx: torch.Tensor, ly: torch.Tensor,
                total_rows: Optional[int] = None, validate: bool = False) -> torch.Tensor:
    """Compact layout (sum_i T_i*(U_i+1), V) of a padded joiner output (N, T, U+1, V): for every
    sequence the rows of its own T_i x (U_i+1) sub-lattice, t-major (test/test.py:44-46).
    Differentiable.  Takes the place of `gather.cat` in cwarp_rnnt/__init__.py:52-59, which keeps the
    FIRST T_i*(U_i+1) rows of the flattened sequence instead and therefore only agrees with the
    compact layout when every U_i equals the padded width.

    total_rows: sum_i T_i*(U_i+1) if the caller knows it; otherwise it is computed on the device and
    read back (one synchronisation).
    validate: read the status word back (one synchronisation) and raise when the lengths do not add
    up to total_rows or a sequence does not fit the padded tensor (the reference asserts
    `lx.max() == T` and `y.size(1)+1 == Up`, cwarp_rnnt/__init__.py:57-58).  Without it such rows
    are zeros, never uninitialised memory."""
    if x.dim() != 4:
        raise RuntimeError("x must be (N, T, U+1, V)")
    if not x.is_cuda or not x.is_contiguous():
        raise RuntimeError("x must be a contiguous CUDA tensor")
    if x.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {x.dtype}")
    for name, t in (("lx", lx), ("ly", ly)):
        if not t.is_cuda or t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous CUDA int32 tensor")
    if lx.numel() != x.size(0) or ly.numel() != x.size(0):
        raise RuntimeError("lx, ly must hold one entry per sequence")
    if total_rows is None:
        total_rows = int((lx.long() * (ly.long() + 1)).sum().item())
    row_off, status = _offsets(lx, ly, int(total_rows))
    out = _Pack.apply(x, lx, ly, int(total_rows), row_off, status)
    if validate:
        _raise_on_status(status, "pack_padded")
    return out


def _raise_on_flags(st: ForwardState):
    _raise_on_status(st.status, "transducer_loss")


class _TransLoss(torch.autograd.Function):
    """cwarp_rnnt/__init__.py:10-29: gradient path when xs requires grad, beta-only path otherwise.
    The reduction (cwarp_rnnt/__init__.py:66-71) is part of the node, so that the backward pass
    receives one scalar for 'mean' / 'sum' and folds it (and the 1/N) into the gradient kernel
    instead of materialising an expanded per-sequence tensor."""

    @staticmethod
    def forward(ctx: Any, xs, lx, ys, ly, blank, fused, max_u, validate, reduction, fastemit_lambda=0.0):
        need_grad = xs.requires_grad
        costs, st = rnnt_forward(xs, lx, ys, ly, blank, fused, max_u, with_grad=need_grad,
                                 reduce=reduction in ("mean", "sum"))
        if validate:
            _raise_on_flags(st)
        if need_grad:
            st.workspace = None  # alpha / beta are not needed again
            if fastemit_lambda:
                st.grads[:, 1] *= 1.0 + fastemit_lambda
            ctx.state = st
            ctx.blank = blank
            ctx.reduction = reduction
            ctx.save_for_backward(xs, lx, ys, ly)
        out_dtype = xs.dtype if xs.dtype not in (torch.float16, torch.bfloat16) else torch.float32
        if st.reduced is not None:  # summed on the device by the kernel that wrote the last cost
            return st.reduced[1 if reduction == "mean" else 0].to(out_dtype)
        costs = costs.to(out_dtype)
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
        return grad_input, None, None, None, None, None, None, None, None, None


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
    if x.dim() == 4:
        # cwarp_rnnt/__init__.py:52-59
        import warnings
        warnings.warn("transducer_loss: 4-D input is packed into the compact layout first; pass compact "
                      "(sum_i T_i*(U_i+1), V) input to skip that copy", stacklevel=2)
        if y.dim() == 2:
            # cwarp_rnnt/__init__.py:57 asserts y.size(1)+1 == Up; a wider padded tensor is fine here
            assert y.size(1) + 1 <= x.size(2), "x must hold U+1 label positions"
        x = pack_padded(x if x.is_contiguous() else x.contiguous(), lx, ly, validate=bool(validate))
    # x: (STU, V)
    assert x.dim() == 2, "input must be compact: (sum_i T_i*(U_i+1), V)"

    if reduction not in ("mean", "sum", "none", None):
        raise ValueError
    return _TransLoss.apply(x, lx, y, ly, blank, bool(fused_log_softmax), max_u, bool(validate),
                            reduction if reduction in ("mean", "sum") else "none")


def rnnt_loss(log_probs: torch.Tensor, labels: torch.Tensor, frames_lengths: torch.Tensor,
              labels_lengths: torch.Tensor, average_frames: bool = False, reduction: Optional[str] = None,
              blank: int = 0, gather: bool = False, fastemit_lambda: float = 0.0,
              compact: bool = False, max_u: Optional[int] = None) -> torch.Tensor:
    """Front end with the call signature of `warp_rnnt.rnnt_loss`, the sibling API the reference's own
    test drives next to `transducer_loss` (test/test.py:4,67), on top of the same kernels.

    log_probs       (N, T, U+1, V) log-probabilities, or with compact=True (sum_i T_i*(U_i+1), V)
    labels          (N, U) padded, or with compact=True (sum_i U_i,) concatenated (padded accepted)
    average_frames  divide every sequence's loss by its frame count
    reduction       None / "none", "mean", "sum"
    gather          accepted; the gather of the blank and label columns is always on here
    fastemit_lambda scales the gradient of every label emission by (1 + lambda) and leaves the loss
                    value alone (FastEmit as a gradient re-weighting)
    max_u           (not in warp_rnnt) upper bound of max(labels_lengths) known to the host; without
                    it, concatenated labels cost one synchronisation per call to read the maximum back
    """
    assert reduction in (None, "none", "mean", "sum")
    del gather
    if labels.dtype != torch.int32:
        labels = labels.int()
    lx = frames_lengths if frames_lengths.dtype == torch.int32 else frames_lengths.int()
    ly = labels_lengths if labels_lengths.dtype == torch.int32 else labels_lengths.int()
    x = log_probs
    if not compact:
        if x.dim() != 4:
            raise RuntimeError("log_probs must be (N, T, U+1, V) unless compact=True")
        x = pack_padded(x if x.is_contiguous() else x.contiguous(), lx, ly)
    elif x.dim() != 2:
        raise RuntimeError("compact log_probs must be (sum_i T_i*(U_i+1), V)")
    costs = _TransLoss.apply(x, lx, labels.contiguous(), ly, int(blank), False, max_u, False, "none",
                             float(fastemit_lambda))
    if average_frames:
        costs = costs / lx.to(costs.dtype)
    if reduction == "mean":
        return costs.mean()
    if reduction == "sum":
        return costs.sum()
    return costs
