"""Compact joiner: the step that produces the (sum_i T_i*(U_i+1), V) rows the loss consumes.

The reference repository holds no joiner; its callers form the padded (N, T, U+1, H) broadcast sum
of encoder frames and predictor states, run the output layer over all of it and pass padded logits
to cwarp_rnnt/__init__.py:52-59.  `compact_join` forms the sum for the cells of each sequence's own
lattice only, directly in the compact row order of test/test.py:44-46 (kernels in csrc/join.hip,
entry points cwr_join / cwr_join_backward); the output layer is then a plain GEMM over (R, H) rows,
which `CompactJoiner.forward` leaves to torch (hipBLASLt).  `fused_joint_loss` / `CompactJoiner.loss`
go one step further for fp16 / bf16: the output layer is multiplied on the matrix cores inside the
loss (csrc/joint.hip, cwr_joint_forward / cwr_joint_backward) and the (R, V) logits are never stored."""
from typing import Any, Optional

import torch

from . import _lib
from .loss import (RESIDENT_JOINT_SIZES, _DTYPES, _offsets, _raise_on_flags, _raise_on_status, _stream_ptr,
                   joint_forward, joint_forward_fg)

_ACTS = {None: 0, "none": 0, "tanh": 1, "relu": 2}
_DW_SPLIT = 16  # parts the rows of a block are cut into for the weight-gradient product


class _Join(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, f, g, lx, ly, total_rows, act, row_off, status):
        lib = _lib.load()
        N, T, H = f.shape
        Up = g.size(1)
        out = torch.empty((total_rows, H), dtype=f.dtype, device=f.device)
        with torch.cuda.device(f.device):
            rc = lib.cwr_join(f.data_ptr(), g.data_ptr(), _DTYPES[f.dtype], act, N, T, Up, H, lx.data_ptr(),
                              ly.data_ptr(), row_off.data_ptr(), total_rows, out.data_ptr(), status.data_ptr(),
                              _stream_ptr(f.device))
            _lib.check(rc, "cwr_join")
        ctx.save_for_backward(lx, ly, row_off, out if act else None)
        ctx.dims = (N, T, Up, H)
        ctx.act = act
        return out

    @staticmethod
    def backward(ctx: Any, dh):
        lx, ly, row_off, out = ctx.saved_tensors
        N, T, Up, H = ctx.dims
        lib = _lib.load()
        dh = dh.contiguous()
        df = torch.empty((N, T, H), dtype=dh.dtype, device=dh.device)
        dg = torch.empty((N, Up, H), dtype=dh.dtype, device=dh.device)
        with torch.cuda.device(dh.device):
            rc = lib.cwr_join_backward(dh.data_ptr(), out.data_ptr() if out is not None else None,
                                       _DTYPES[dh.dtype], ctx.act, N, T, Up, H, lx.data_ptr(), ly.data_ptr(),
                                       row_off.data_ptr(), dh.size(0), df.data_ptr(), dg.data_ptr(),
                                       _stream_ptr(dh.device))
            _lib.check(rc, "cwr_join_backward")
        return df, dg, None, None, None, None, None, None


def compact_join(f: torch.Tensor, g: torch.Tensor, lx: torch.Tensor, ly: torch.Tensor,
                 activation: Optional[str] = None, total_rows: Optional[int] = None,
                 validate: bool = False) -> torch.Tensor:
    """h[row(n,t,u), :] = act(f[n, t, :] + g[n, u, :]) for t < lx[n], u <= ly[n], as (R, H) compact
    rows (sequence-major, then t, then u).  Differentiable in f and g.

    f: (N, T, H) encoder frames; g: (N, U+1, H) predictor states; lx, ly: (N,) int32 frame and label
    counts; activation: None, "tanh" or "relu"; total_rows: sum_i lx_i*(ly_i+1) if known, else it is
    computed on the device and read back (one synchronisation); validate: read the status word
    back (one synchronisation) and raise when the lengths do not add up to total_rows or a sequence
    does not fit f / g.  Without it the rows no valid cell maps to are zeros."""
    if activation not in _ACTS:
        raise RuntimeError(f"activation must be one of {sorted(k for k in _ACTS if k)} or None")
    if f.dim() != 3 or g.dim() != 3 or f.size(0) != g.size(0) or f.size(2) != g.size(2):
        raise RuntimeError("f must be (N, T, H) and g (N, U+1, H)")
    if f.dtype != g.dtype or f.dtype not in _DTYPES:
        raise RuntimeError(f"f and g must share a supported dtype, got {f.dtype} and {g.dtype}")
    if not f.is_cuda or not g.is_cuda:
        raise RuntimeError("f and g must be CUDA tensors")
    for name, t in (("lx", lx), ("ly", ly)):
        if not t.is_cuda or t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous CUDA int32 tensor")
    if lx.numel() != f.size(0) or ly.numel() != f.size(0):
        raise RuntimeError("lx, ly must hold one entry per sequence")
    if total_rows is None:
        total_rows = int((lx.long() * (ly.long() + 1)).sum().item())
    row_off, status = _offsets(lx, ly, int(total_rows))
    out = _Join.apply(f.contiguous(), g.contiguous(), lx, ly, int(total_rows), _ACTS[activation], row_off, status)
    if validate:
        _raise_on_status(status, "compact_join")
    return out


class _JointLoss(torch.autograd.Function):
    """Loss of logits = h @ weight.T + bias that are never stored.

    Forward: cwr_joint_forward (the output layer on the matrix cores, every tile reduced on the spot
    to the row's log-sum-exp and its blank / label logits).  Backward: cwr_joint_backward forms the
    logits of a block of rows again on the matrix cores and writes their gradient, rounded once to
    the 16-bit type; library GEMMs multiply the block into dh, dW and dbias.  Only
    `chunk_rows` x V logit gradients exist at any moment."""

    @staticmethod
    def forward(ctx: Any, h, weight, bias, lx, ys, ly, blank, reduction, max_u, validate, chunk_rows):
        costs, st = joint_forward(h, weight, bias, lx, ys, ly, blank, max_u)
        if validate:
            _raise_on_flags(st)
        st.workspace = None
        ctx.state = st
        ctx.blank, ctx.reduction, ctx.chunk_rows = blank, reduction, int(chunk_rows)
        ctx.save_for_backward(h, weight, bias if bias is not None else h.new_empty(0), lx, ys, ly)
        ctx.has_bias = bias is not None
        if reduction == "mean":
            return costs.mean()
        if reduction == "sum":
            return costs.sum()
        return costs

    @staticmethod
    def backward(ctx: Any, grad_out):
        h, weight, bias, lx, ys, ly = ctx.saved_tensors
        dh, dw, db = _joint_backward(h, weight, bias if ctx.has_bias else None, ctx.state, grad_out, ctx.reduction,
                                     ctx.blank, ctx.chunk_rows)
        return dh, dw, db, None, None, None, None, None, None, None, None


_BLOCK_BYTES = 384 << 20   # logit gradients alive at a time when the caller sets no block size
_BLOCK_MIN_ROWS = 65536    # fewer rows than this no longer fill the GPU with 128-row workgroups


def _balanced_block(R: int, V: int, itemsize: int) -> int:
    """Rows per block of the backward pass: the fewest blocks of at most _BLOCK_BYTES of logit
    gradients, all of the same size (a short last block runs the matrix kernels at a fraction of
    their speed: N=32, V=1024, H=512, R=311449: 131072 + 131072 + 49305 rows 1.97 ms forward +
    backward, two blocks of 155725 rows 1.83 ms, one block 1.74 ms)."""
    limit = max(_BLOCK_MIN_ROWS, _BLOCK_BYTES // max(1, V * itemsize))
    blocks = max(1, -(-R // limit))
    return max(1, (-(-R // blocks) + 255) // 256 * 256)


def _joint_backward(h, weight, bias, st, grad_out, reduction, blank, chunk_rows):
    """(dh, dW, dbias) of the loss of logits = h @ weight.T + bias from the state its forward call left:
    cwr_joint_backward a block of rows at a time, library GEMMs on each block."""
    lib = _lib.load()
    dev = h.device
    R, H = h.shape
    V = weight.size(0)
    N = st.N
    gc = grad_out.to(torch.float32).reshape(-1)
    if gc.numel() == 1:
        gc = gc.expand(N)
    gc = (gc / N if reduction == "mean" else gc).contiguous()
    dh = torch.empty_like(h)
    dw = torch.zeros((V, H), dtype=torch.float32, device=dev)
    db = torch.zeros(V, dtype=torch.float32, device=dev) if bias is not None else None
    bias_f = bias.to(torch.float32).contiguous() if bias is not None else None
    chunk = max(1, min(int(chunk_rows), R)) if chunk_rows > 0 else _balanced_block(R, V, h.element_size())
    z = torch.empty((chunk, V), dtype=h.dtype, device=dev)
    with torch.cuda.device(dev):
        stream = _stream_ptr(dev)
        for r0 in range(0, R, chunk):
            r1 = min(R, r0 + chunk)
            zc = z[: r1 - r0]
            rc = lib.cwr_joint_backward(h[r0:].data_ptr(), weight.data_ptr(),
                                        bias_f.data_ptr() if bias_f is not None else None, _DTYPES[h.dtype],
                                        r1 - r0, H, V, N, int(blank), st.rowinfo[r0:].data_ptr(),
                                        st.grads[r0:].data_ptr(), st.lse[r0:].data_ptr(), gc.data_ptr(), 1, 1.0,
                                        zc.data_ptr(), stream)
            _lib.check(rc, "cwr_joint_backward")
            torch.mm(zc, weight, out=dh[r0:r1])
            # dW += zc^T h[r0:r1].  The contraction runs over the rows, the result is only (V, H): as one
            # GEMM the library fills a quarter of the GPU with it, so the rows are cut into _DW_SPLIT
            # parts multiplied as a batch (16-bit products of a part each, summed in fp32)
            n = r1 - r0
            m = (n // _DW_SPLIT) * _DW_SPLIT
            if m:
                part = torch.bmm(zc[:m].view(_DW_SPLIT, m // _DW_SPLIT, V).transpose(1, 2),
                                 h[r0:r0 + m].view(_DW_SPLIT, m // _DW_SPLIT, H))
                dw.add_(part.sum(dim=0, dtype=torch.float32))
            if n > m:
                dw.add_(torch.mm(zc[m:n].t(), h[r0 + m:r1]))
            if db is not None:
                db.add_(zc.sum(dim=0, dtype=torch.float32))
    dbias = db.to(bias.dtype) if db is not None else None
    return dh, dw.to(weight.dtype), dbias


class _JoinerLoss(torch.autograd.Function):
    """The whole joiner behind the loss: rows act(f[n,t] + g[n,u]) formed inside the output-layer kernel
    (cwr_joint_forward_fg).  When nothing asks for a gradient the (R, H) rows never exist; otherwise
    the kernel leaves them behind for the backward pass (logit gradients, weight-gradient product,
    cwr_join_backward)."""

    @staticmethod
    def forward(ctx: Any, f, g, weight, bias, lx, ys, ly, blank, reduction, act, total_rows, max_u, validate,
                chunk_rows):
        need = any(ctx.needs_input_grad[:4])
        costs, st, h = joint_forward_fg(f, g, act, weight, bias, lx, ys, ly, blank, total_rows, max_u, keep_rows=need)
        if validate:
            _raise_on_flags(st)
        st.workspace = None
        ctx.state = st
        ctx.blank, ctx.reduction, ctx.chunk_rows, ctx.act = blank, reduction, int(chunk_rows), act
        ctx.dims = (f.size(0), f.size(1), g.size(1), f.size(2))
        ctx.has_bias = bias is not None
        if need:
            ctx.save_for_backward(h, weight, bias if bias is not None else f.new_empty(0), lx, ly)
        if reduction == "mean":
            return costs.mean()
        if reduction == "sum":
            return costs.sum()
        return costs

    @staticmethod
    def backward(ctx: Any, grad_out):
        h, weight, bias, lx, ly = ctx.saved_tensors
        st = ctx.state
        dh, dw, db = _joint_backward(h, weight, bias if ctx.has_bias else None, st, grad_out, ctx.reduction,
                                     ctx.blank, ctx.chunk_rows)
        N, T, Up, H = ctx.dims
        lib = _lib.load()
        df = torch.empty((N, T, H), dtype=dh.dtype, device=dh.device)
        dg = torch.empty((N, Up, H), dtype=dh.dtype, device=dh.device)
        with torch.cuda.device(dh.device):
            rc = lib.cwr_join_backward(dh.data_ptr(), h.data_ptr() if ctx.act else None, _DTYPES[dh.dtype], ctx.act,
                                       N, T, Up, H, lx.data_ptr(), ly.data_ptr(), st.row_off.data_ptr(), dh.size(0),
                                       df.data_ptr(), dg.data_ptr(), _stream_ptr(dh.device))
            _lib.check(rc, "cwr_join_backward")
        return df, dg, dw, db, None, None, None, None, None, None, None, None, None, None


def fused_joiner_loss(f: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                      lx: torch.Tensor, y: torch.Tensor, ly: torch.Tensor, blank: int = 0,
                      reduction: Optional[str] = "mean", activation: Optional[str] = "tanh", *,
                      total_rows: Optional[int] = None, max_u: Optional[int] = None, validate: bool = False,
                      chunk_rows: Optional[int] = None, one_kernel: Optional[bool] = None) -> torch.Tensor:
    """transducer_loss of the logits act(f[n,t] + g[n,u]) @ weight.T + bias, the joiner's whole chain,
    with neither the (R, H) joint rows nor the (R, V) logits in memory on the way to the loss: f
    (N, T, H) encoder frames and g (N, U+1, H) predictor states projected to the joint space, weight
    (V, H) and bias (V,) or None the output layer, fp16 or bf16.  Differentiable in f, g, weight and
    bias (the backward pass does hold the joint rows and chunk_rows x V logit gradients).

    one_kernel: True forms the joint rows inside the output-layer kernel (cwr_joint_forward_fg; joint
    sizes in RESIDENT_JOINT_SIZES only), False runs compact_join and fused_joint_loss one after the
    other, None picks by speed: the one-kernel form wins up to H = 384 (N=32, V=1024, H=256, bf16:
    forward 0.28 against 0.31 ms) and loses beyond (H=512: 0.53 against 0.46 ms: every wave of the GPU
    forms its rows at the same moment, with no matrix work of another wave to hide behind), where it
    remains the choice of a caller who cannot afford the (R, H) rows in memory."""
    if activation not in _ACTS:
        raise RuntimeError(f"activation must be one of {sorted(k for k in _ACTS if k)} or None")
    assert lx.dtype == torch.int32 and ly.dtype == torch.int32 and y.dtype == torch.int32
    assert reduction in ["mean", "sum", "none"] or reduction is None
    assert blank >= 0 and blank < weight.size(0)
    if total_rows is None:
        total_rows = int((lx.long() * (ly.long() + 1)).sum().item())
    if one_kernel is None:
        one_kernel = f.size(-1) in RESIDENT_JOINT_SIZES and f.size(-1) <= 384
    if one_kernel and f.size(-1) not in RESIDENT_JOINT_SIZES:
        raise RuntimeError(f"one_kernel needs a joint dimension in {RESIDENT_JOINT_SIZES}")
    if not one_kernel:
        h = compact_join(f, g, lx, ly, activation, total_rows, validate)
        return fused_joint_loss(h, weight, bias, lx, y, ly, blank, reduction, max_u=max_u, validate=validate,
                                chunk_rows=chunk_rows)
    return _JoinerLoss.apply(f.contiguous(), g.contiguous(), weight.contiguous(), bias, lx, y, ly, int(blank),
                             reduction if reduction in ("mean", "sum") else "none", _ACTS[activation],
                             int(total_rows), max_u, bool(validate), -1 if chunk_rows is None else int(chunk_rows))


def fused_joint_loss(h: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], lx: torch.Tensor,
                     y: torch.Tensor, ly: torch.Tensor, blank: int = 0, reduction: Optional[str] = "mean", *,
                     max_u: Optional[int] = None, validate: bool = False, chunk_rows: Optional[int] = None) -> torch.Tensor:
    """transducer_loss(h @ weight.T + bias, lx, y, ly, blank, reduction, fused_log_softmax=True) without
    the (R, V) logits: h (R, H) compact joint activations (e.g. from compact_join), weight (V, H) and
    bias (V,) or None the output layer, fp16 or bf16.  Differentiable in h, weight and bias; the
    backward pass holds at most chunk_rows x V logit gradients at a time (None: equal blocks of at
    most 384 MiB each)."""
    assert lx.dtype == torch.int32 and ly.dtype == torch.int32 and y.dtype == torch.int32
    assert reduction in ["mean", "sum", "none"] or reduction is None
    assert blank >= 0 and blank < weight.size(0)
    return _JointLoss.apply(h.contiguous(), weight.contiguous(), bias, lx, y, ly, int(blank),
                            reduction if reduction in ("mean", "sum") else "none", max_u, bool(validate),
                            -1 if chunk_rows is None else int(chunk_rows))


class CompactJoiner(torch.nn.Module):
    """Projection of encoder and predictor outputs to a joint space, their compact broadcast sum
    with an activation, and the output layer: (N,T,E), (N,U+1,P) -> (R, V) logits in the layout
    `transducer_loss(..., fused_log_softmax=True)` takes.  The three linear layers are library
    GEMMs; only the sum is done here, and only for the cells the loss will read."""

    def __init__(self, enc_dim: int, pred_dim: int, joint_dim: int, vocab: int, activation: str = "tanh"):
        super().__init__()
        self.enc = torch.nn.Linear(enc_dim, joint_dim)
        self.pred = torch.nn.Linear(pred_dim, joint_dim, bias=False)
        self.out = torch.nn.Linear(joint_dim, vocab)
        self.activation = activation

    def forward(self, enc_out, pred_out, lx, ly, total_rows: Optional[int] = None):
        h = compact_join(self.enc(enc_out), self.pred(pred_out), lx, ly, self.activation, total_rows)
        return self.out(h)

    def loss(self, enc_out, pred_out, lx, y, ly, blank: int = 0, reduction: Optional[str] = "mean",
             total_rows: Optional[int] = None):
        """The transducer loss of this joiner's logits without storing them (fp16 / bf16 modules): the
        broadcast sum, the activation and the output layer all run inside the loss's own kernel
        (fused_joiner_loss)."""
        return fused_joiner_loss(self.enc(enc_out), self.pred(pred_out), self.out.weight, self.out.bias, lx, y, ly,
                                 blank, reduction, self.activation, total_rows=total_rows)
