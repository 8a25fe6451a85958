/*
 * cwarp_rnnt_hip.h -- C ABI of libcwarp_rnnt_hip.so: RNN-T loss and gradient for compact-layout
 * inputs on AMD MI355X (gfx950).
 *
 * The three compute entry points replace the three functions the reference exports through
 * pybind11 (CompactWarpRNNTLoss, cwarp_cuda.cpp:138-153):
 *
 *     _cwarp_rnnt_forward   (cwarp_cuda.cpp:84-108)   ->  cwr_forward
 *     _cwarp_rnnt_loss      (cwarp_cuda.cpp:58-82)    ->  cwr_loss
 *     _cwarp_rnnt_backward  (cwarp_cuda.cpp:110-136)  ->  cwr_backward
 *
 * plus cwr_offsets for the row-offset computation the reference repeats inline in each of them
 * (cwarp_cuda.cpp:72-77, 98-103, 124-129).
 *
 * Conventions
 *   - Every pointer named below is a DEVICE pointer unless stated otherwise.  The library never
 *     allocates, frees or synchronises; all kernels are enqueued on `stream` (a hipStream_t
 *     passed as void*; NULL = the default stream).
 *   - Every function returns a cwr_status (0 = success).  Argument validation happens on the
 *     host before any HIP call, so invalid calls can be exercised without a GPU.
 *   - Data-dependent problems (lengths that do not add up to R, labels outside [0,V), ...) cannot
 *     be seen by the host without a synchronisation; kernels guard every access, never touch
 *     memory outside the given buffers, and record CWR_FLAG_* bits in status[0].
 *   - Compact layout: x has R = sum_n lx[n]*(ly[n]+1) rows of V entries; the row of sequence n,
 *     frame t, label position u is row_off[n] + t*(ly[n]+1) + u
 *     (cwarp_cuda_gather_kernel.cu:36, test/test.py:44-46).
 *   - Labels: y_stride >= 0 -> padded 2-D labels, label u of sequence n is y[n*y_stride + u]
 *     (the reference layout, cwarp_rnnt/__init__.py:45-49);
 *     y_stride < 0 -> concatenated 1-D labels, label u of sequence n is y[lab_off[n] + u].
 *     y_len is the number of int32 entries behind y; reads beyond it are refused and flagged.
 */
#ifndef CWARP_RNNT_HIP_H
#define CWARP_RNNT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of x and of the gradient w.r.t. x (all arithmetic is done in fp32) */
enum cwr_dtype { CWR_F32 = 0, CWR_F16 = 1, CWR_BF16 = 2, CWR_F64 = 3 };

/* CWR_MODE_LOGPROB: x holds log-probabilities; the gradient is non-zero only in the blank and
 *                   label columns (exactly what the reference computes).
 * CWR_MODE_FUSED:   x holds raw logits; log-softmax over V is fused into the gather pass and the
 *                   gradient w.r.t. the logits is dense. */
enum cwr_mode { CWR_MODE_LOGPROB = 0, CWR_MODE_FUSED = 1 };

enum cwr_status {
    CWR_OK = 0,
    CWR_ERR_NULL = 1,      /* a required pointer is NULL */
    CWR_ERR_DTYPE = 2,     /* dtype is not a cwr_dtype */
    CWR_ERR_MODE = 3,      /* mode is not a cwr_mode */
    CWR_ERR_SHAPE = 4,     /* negative or inconsistent N, R, V, max_u */
    CWR_ERR_BLANK = 5,     /* blank outside [0, V) (cwarp_rnnt/__init__.py:50) */
    CWR_ERR_ALIGN = 6,     /* a buffer is not aligned to its element size */
    CWR_ERR_LAUNCH = 7,    /* the HIP runtime refused a launch */
    CWR_ERR_TOO_LARGE = 8, /* a size exceeds what the kernels index, or what the built-in scratch holds */
    CWR_ERR_RUNTIME = 9    /* a HIP runtime call other than a launch failed */
};

/* bits of status[0], written by the kernels */
enum cwr_flag {
    CWR_FLAG_ROWS_MISMATCH = 1, /* sum lx*(ly+1) != R */
    CWR_FLAG_BAD_LENGTH = 2,    /* some lx <= 0 or ly < 0 (that sequence is skipped, cost = NaN) */
    CWR_FLAG_BAD_LABEL = 4,     /* a label outside [0, V) or beyond the label array was met (that
                                   sequence's cost is NaN) */
    CWR_FLAG_FB_MISMATCH = 8,   /* forward and backward log-likelihood differ by > 0.1 % (and by
                                   more than 1e-5, so that a likelihood within rounding of 1 does
                                   not count) for some sequence; the cost is their mean, as in the
                                   reference (cwarp_cuda_rnnt_kernel.cu:356-364, which prints) */
    CWR_FLAG_U_TOO_LARGE = 16,  /* some ly exceeds the max_u given to the call, or some lx exceeds
                                   2^19 frames */
    CWR_FLAG_INTERNAL = 32      /* a bounded wait inside a kernel ran out (the cost of the sequence it
                                   happened in is NaN) */
};

int cwr_version(void);
const char* cwr_strerror(int status);

/* Bytes of scratch cwr_forward / cwr_loss need for a batch of N sequences, R rows and at most
 * max_u labels per sequence.  The scratch holds the gathered blank / label records, alpha and beta
 * (O(R) plus a per-sequence padding that grows with max_u, so pass a tight max_u); nothing in it
 * is needed by cwr_backward.  Must be 256-byte aligned. */
size_t cwr_workspace_bytes(int64_t N, int64_t R, int64_t max_u);

/* Location of the lattice state inside the workspace after cwr_forward, for analysis tools (the
 * reference returns alpha and beta, cwarp_cuda_rnnt_kernel.cu:383-384).  which:
 *   0  gathered probabilities, 8 bytes per cell: fp32 P(blank), P(label)
 *   7  gathered log-probabilities, 8 bytes per cell: fp32 log2 P(blank), log2 P(label)
 *   1  alpha, 2  beta: one fp64 per cell
 *   3  pad_off: N+1 int64, first cell slot of each sequence, -1 for a skipped sequence
 *   4  seqmode: N+1 int32 (N used), how the sequence was walked.  0 = both directions in the
 *      scaled linear domain; bit 0 = both in the log domain (log-probs outside what the linear
 *      walk carries); bit 1 / bit 2 = alpha / beta was walked again in the log domain.  A sequence
 *      with more than 16 strips of 128 labels is always in the log domain.
 *   5  scale_a, 6  scale_b: int32 scale exponents of the linear-domain walk
 * Cell (t,u) of sequence n lives at element pad_off[n] + cwr_lattice_slot(t,u,T,U): row
 * t + (u%128)/2 + 32 of its strip, whose rows are nl rounded up to even slots apart.
 * Log-domain values are base-2 logarithms (multiply by ln 2).  Linear-domain values are
 * value * 2^C: a strip s = u/128 of width nl = min(128, U+1-128s) is walked by L = ceil(nl/2) lanes,
 * lane l = (u%128)/2 holding columns 2l and 2l+1; the walk step is k = t+l (alpha) or
 * T+L-2-(t+l) (beta) and C = scale[(pad_off[n] + s*(T+127)*128)/16 + (k/16)*L + l].
 * cwr_export_lattice does this. */
int cwr_workspace_section(int64_t N, int64_t R, int64_t max_u, int which, size_t* offset, size_t* bytes);
int64_t cwr_lattice_slot(int64_t t, int64_t u, int64_t T, int64_t U); /* host helper */

/* Host helper: the rule that turns a sequence's two likelihoods into its cost, exactly as the
 * kernels apply it (cwarp_cuda_rnnt_kernel.cu:345-366).  fwd_log2 = log2 of alpha at the last cell
 * times that cell's blank probability, bwd_log2 = log2 beta[0][0].  *cost = -bwd in nats; when the
 * two differ by more than 0.1 % of the larger (and by more than 1e-5 bits: a floor the reference
 * does not have, for likelihoods within rounding of 1) the cost is minus their mean and the
 * function returns 1 -- the case in which the kernels raise CWR_FLAG_FB_MISMATCH and the reference
 * prints a warning.  Returns 0 otherwise, -1 for a NULL cost. */
int cwr_cost_rule(double fwd_log2, double bwd_log2, float* cost);

/* Row and label offsets by a device prefix scan.
 *   row_off[n] = sum_{j<n} lx[j]*(ly[j]+1), n = 0..N   (N+1 entries, int64)
 *   lab_off[n] = sum_{j<n} ly[j],           n = 0..N   (N+1 entries, int64)
 * Replaces cwarp_cuda.cpp:72-77 (which keeps the first N entries as int32).
 * status: 4 x int32, zeroed then flagged.  R < 0 skips the row-count check. */
int cwr_offsets(const int32_t* lx, const int32_t* ly, int64_t N, int64_t R,
                int64_t* row_off, int64_t* lab_off, int32_t* status, void* stream);

/* Loss with the state the backward pass needs.  Replaces _cwarp_rnnt_forward
 * (cwarp_cuda.cpp:84-108 -> gather_cuda_forward + cwarp_cuda_costs_with_grad).
 *   x        (R,V) of `dtype`, contiguous
 *   lx, ly   (N,) int32 frame / label counts;  y, y_stride: labels (see above)
 *   max_u    an upper bound of max(ly) known to the host (e.g. the padded label width); a
 *            sequence with more labels, or with more than 2^19 frames, is skipped (cost NaN,
 *            CWR_FLAG_U_TOO_LARGE)
 * outputs
 *   row_off, lab_off (N+1) int64;  status 4 x int32 (word 0: CWR_FLAG_* bits; the others are
 *            scratch of the call)
 *   rowinfo  (R,2) int32 per-row record for cwr_backward: (label of the row or -1, sequence of the
 *            row or -1)
 *   lse      (R,) fp32 log-sum-exp of each row            [CWR_MODE_FUSED only, else may be NULL]
 *   grads    (R,2) fp32 d cost / d(blank log-prob, label log-prob) per row, as the reference's
 *            `grads` (cwarp_cuda_rnnt_kernel.cu:275-332)
 *   costs    (N,) fp32 -log P(y|x)  (cwarp_cuda_rnnt_kernel.cu:334-367) */
int cwr_forward(const void* x, int dtype, int64_t R, int64_t V,
                const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                int64_t N, int32_t blank, int mode, int64_t max_u,
                void* workspace, size_t workspace_bytes,
                int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo,
                float* lse, float* grads, float* costs, void* stream);

/* cwr_forward for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * forward allocates eight tensors per call, cwarp_cuda_rnnt_kernel.cu:399-404).  Same arguments,
 * outputs and results as cwr_forward, without the workspace: the scratch is an array of
 * CWR_NOALLOC_SCRATCH_BYTES inside the library's device code, one copy per GPU, there for as long as
 * the process lives.  The call makes no allocation of any kind.
 *   - cwr_workspace_bytes(N, R, max_u) must not exceed CWR_NOALLOC_SCRATCH_BYTES, else
 *     CWR_ERR_TOO_LARGE.  128 MiB: the N=32, T~175, U~50 batch (R = 3.1e5) needs 39 MiB, the
 *     long-form N=4, T~1250, U~300 batch (R = 1.5e6) 119 MiB.
 *   - The array is part of the library's device code: every process that loads the library holds
 *     128 MiB on every GPU it runs the library's kernels on, whether or not it ever calls this entry
 *     point.
 *   - The first call on a GPU looks the array's address up (hipGetSymbolAddress); make it outside
 *     a stream capture.  Calls with arguments the host can reject (null or misaligned pointers, bad
 *     sizes) return before that look-up and touch no GPU.
 *   - Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams,
 *     two threads) race.  Calls in stream order on one stream are safe; nothing from an earlier
 *     call is relied on, the kernels initialise what they read.
 *   - The array holds the lattice state of the LAST call on that GPU only; cwr_export_lattice does
 *     not reach it. */
#define CWR_NOALLOC_SCRATCH_BYTES (128u << 20)
int cwr_forward_noalloc(const void* x, int dtype, int64_t R, int64_t V,
                        const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                        int64_t N, int32_t blank, int mode, int64_t max_u,
                        int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo,
                        float* lse, float* grads, float* costs, void* stream);

/* Loss only (no gradient state).  Replaces _cwarp_rnnt_loss (cwarp_cuda.cpp:58-82 ->
 * gather_cuda_forward + cwarp_cuda_cal_costs): beta recursion only, costs = -beta[0][0]. */
int cwr_loss(const void* x, int dtype, int64_t R, int64_t V,
             const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
             int64_t N, int32_t blank, int mode, int64_t max_u,
             void* workspace, size_t workspace_bytes,
             int64_t* row_off, int64_t* lab_off, int32_t* status,
             float* costs, void* stream);

/* cwr_forward / cwr_loss with the reduction of cwarp_rnnt/__init__.py:66-71 folded in: besides
 * costs, reduced[0] = sum of the N costs and reduced[1] = their mean (2 x fp32), written by
 * whichever wave writes the last cost and summed in a fixed order, so that 'mean' / 'sum' need no
 * further kernel.  A skipped sequence (cost NaN) makes both NaN.  N = 0 writes nothing. */
int cwr_forward_reduced(const void* x, int dtype, int64_t R, int64_t V,
                        const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                        int64_t N, int32_t blank, int mode, int64_t max_u,
                        void* workspace, size_t workspace_bytes,
                        int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo,
                        float* lse, float* grads, float* costs, float* reduced, void* stream);
int cwr_loss_reduced(const void* x, int dtype, int64_t R, int64_t V,
                     const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                     int64_t N, int32_t blank, int mode, int64_t max_u,
                     void* workspace, size_t workspace_bytes,
                     int64_t* row_off, int64_t* lab_off, int32_t* status,
                     float* costs, float* reduced, void* stream);

/* Gradient w.r.t. x.  Replaces _cwarp_rnnt_backward (cwarp_cuda.cpp:110-136 ->
 * cwarp_cuda_backward_ + zeros(R,V) + gather_cuda_backward_) in one streaming pass that does
 * not modify `grads`.
 *   CWR_MODE_LOGPROB: grad_x[r,:] = 0 except [blank] = grads[r,0]*g and [label] = grads[r,1]*g
 *                     (label written after blank, cwarp_cuda_gather_kernel.cu:70-73); x unused.
 *   CWR_MODE_FUSED:   grad_x[r,v] = g*(softmax(x_r)[v]*gamma_r + grads[r,0][v==blank]
 *                     + grads[r,1][v==label]),  gamma_r = -(grads[r,0]+grads[r,1]).
 * with g = grad_costs[n*grad_stride]*grad_scale for the row's sequence n
 * (cwarp_cuda_rnnt_kernel.cu:518-519).  grad_stride is 1 for a per-sequence gradient or 0 to
 * broadcast grad_costs[0] (what a mean / sum reduction hands back), grad_scale folds the 1/N of a
 * mean reduction in, so that neither needs a kernel of its own.
 *   rowinfo  as written by cwr_forward (or cwr_rowinfo); lx, ly, y, row_off, lab_off are accepted
 *            for symmetry with the reference's signature and may be NULL.
 *   grad_x   (R,V) of `dtype`, fully written. */
int cwr_backward(const void* x, int dtype, int64_t R, int64_t V,
                 const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                 int64_t N, int32_t blank, int mode,
                 const int64_t* row_off, const int64_t* lab_off, const int32_t* rowinfo,
                 const float* grads, const float* lse, const float* grad_costs,
                 int64_t grad_stride, float grad_scale, void* grad_x, void* stream);

/* The per-row record cwr_backward reads, rebuilt from the lengths and labels, for a caller that
 * kept `grads` but not the `rowinfo` cwr_forward wrote (the reference's backward likewise rebuilds
 * its offsets from lx and ly, cwarp_cuda.cpp:124-129).  row_off / lab_off as from cwr_offsets. */
int cwr_rowinfo(const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                int64_t N, int64_t R, int64_t V, const int64_t* row_off, const int64_t* lab_off,
                int32_t* rowinfo, void* stream);

/* alpha and beta of the last cwr_forward (beta only after cwr_loss: pass alphas = NULL), copied
 * out of its workspace as padded (N, T_pad, Up_pad) fp64 arrays of NATURAL logarithms, zero
 * outside each sequence's own T x (U+1) lattice -- what the reference returns from its forward
 * call (cwarp_cuda_rnnt_kernel.cu:383-384, 399-400, 496).  lx, ly, N, R, max_u, workspace as in
 * that call; cells with t >= T_pad or u >= Up_pad are not exported.  Either output may be NULL. */
int cwr_export_lattice(const int32_t* lx, const int32_t* ly, int64_t N, int64_t R, int64_t max_u,
                       const void* workspace, size_t workspace_bytes, int64_t T_pad, int64_t Up_pad,
                       double* alphas, double* betas, void* stream);

/* Padded -> compact rows.  Replaces the 4-D input branch cwarp_rnnt/__init__.py:52-59 (which
 * calls the external gather.cat on the flattened tensor): for every sequence n the rows of its own
 * sub-lattice, x_compact[row_off[n] + t*(ly[n]+1) + u, :] = x_padded[n, t, u, :] for t < lx[n],
 * u <= ly[n] (the compact order of test/test.py:44-46).
 *   x_padded (N, T_pad, Up_pad, V) contiguous;  x_compact (R, V);  row_off from cwr_offsets
 *   status   optional 4 x int32 already initialised by cwr_offsets: CWR_FLAG_BAD_LENGTH is added
 *            when a sequence does not fit (lx[n] > T_pad or ly[n]+1 > Up_pad).
 * Every row of x_compact is written: rows whose cell lies beyond the padded array, and rows that
 * belong to no sequence (R larger than the lengths add up to), are zeroed. */
int cwr_pack(const void* x_padded, int dtype, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t V,
             const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* x_compact,
             int32_t* status, void* stream);

/* Backward of cwr_pack: g_padded[n, t, u, :] = g_compact[row, :] inside the sub-lattice and 0
 * elsewhere; every element of g_padded is written. */
int cwr_unpack(const void* g_compact, int dtype, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t V,
               const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* g_padded,
               void* stream);

/* Compact joiner front: h[row_off[n] + t*(ly[n]+1) + u, :] = act(f[n, t, :] + g[n, u, :]) for
 * t < lx[n], u <= ly[n] -- the broadcast sum of encoder frames and predictor states for the cells
 * of each sequence's own lattice only, in the compact row order of test/test.py:44-46.  The
 * reference repository has no joiner (its callers form the padded (N,T,U+1,H) sum and pass padded
 * logits to cwarp_rnnt/__init__.py:52-59); the linear layer that follows is left to a library GEMM
 * over the (R, H) rows.
 *   f (N, T_pad, H), g (N, Up_pad, H) contiguous;  h (R, H);  act a cwr_activation
 *   status as for cwr_pack; rows of h no valid cell maps to are zeroed, as there. */
enum cwr_activation { CWR_ACT_NONE = 0, CWR_ACT_TANH = 1, CWR_ACT_RELU = 2 };
int cwr_join(const void* f, const void* g, int dtype, int act, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t H,
             const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* h, int32_t* status,
             void* stream);

/* Backward of cwr_join: df[n, t, :] = sum over u of dz, dg[n, u, :] = sum over t of dz, where
 * dz = dh * act'(z) with act' taken from the stored output h (unused, may be NULL, for
 * CWR_ACT_NONE).  Sums run in a fixed order (no atomics); every element of df and dg is written,
 * zeros outside each sequence's lattice. */
int cwr_join_backward(const void* dh, const void* h, int dtype, int act, int64_t N, int64_t T_pad, int64_t Up_pad,
                      int64_t H, const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* df,
                      void* dg, void* stream);

/* cwr_forward for logits that are never stored: the joiner's output layer
 * logits[r, v] = sum_k h[r, k] * w[v, k] + bias[v] is multiplied tile by tile on the matrix cores
 * (16-bit inputs, fp32 accumulation) and every tile is reduced on the spot to what the loss needs
 * of a row: its log-sum-exp over V and its blank and label logits.  The reference repository has
 * no joiner; this replaces, for its callers, the output-layer GEMM, the log-softmax
 * (test/test.py:19-20) and the gather pass (cwarp_cuda_gather_kernel.cu:19-43) that cwr_forward in
 * CWR_MODE_FUSED would run on stored logits, and removes the (R, V) logits from memory.
 *   h     (R, H) compact joint activations (e.g. from cwr_join), w (V, H) output-layer weight (the
 *         layout of a torch.nn.Linear weight), both of `dtype` = CWR_F16 or CWR_BF16, contiguous,
 *         16-byte aligned;  H a multiple of 32 (a multiple of 64 from 128 to 1024 is read exactly
 *         once, every wave keeping its rows in registers; any other size is streamed once per tile
 *         of 128 vocabulary entries, at less than half the speed)
 *   bias  (V,) fp32 or NULL
 * All other arguments and every output as for cwr_forward with mode = CWR_MODE_FUSED; lse, rowinfo
 * and grads are what cwr_joint_backward reads. */
int cwr_joint_forward(const void* h, const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                      const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                      int64_t N, int32_t blank, int64_t max_u, void* workspace, size_t workspace_bytes,
                      int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                      float* grads, float* costs, void* stream);

/* cwr_joint_forward with the joint rows formed inside the kernel: the whole chain of the joiner,
 * h[row(n,t,u), :] = act(f[n,t,:] + g[n,u,:]) (cwr_join's arithmetic: sum and activation in fp32, one
 * rounding to `dtype`), output layer, log-softmax and gather, as ONE kernel behind the loss.  f and g
 * are a few MB and are served by the L2; neither the (R, H) joint rows nor the (R, V) logits have to
 * exist in memory.  The reference repository has no joiner (see cwr_join).
 *   f (N, T_pad, H), g (N, Up_pad, H), w (V, H) of `dtype` = CWR_F16 or CWR_BF16, contiguous, 16-byte
 *         aligned;  act a cwr_activation
 *   H     a multiple of 64 from 128 to 1024 (the sizes whose rows a wave keeps in registers);
 *         any other H: CWR_ERR_SHAPE, and the caller runs cwr_join + cwr_joint_forward instead
 *   h_out (R, H) or NULL: receives the joint rows, bit-identical to cwr_join's, for a backward pass
 *         that needs them (cwr_joint_backward, the weight-gradient product, cwr_join_backward)
 * A cell that lies outside f or g (lx[n] > T_pad or ly[n]+1 > Up_pad) raises CWR_FLAG_BAD_LENGTH
 * and counts as a row of zeros, as in cwr_join.  Everything else as for cwr_joint_forward. */
int cwr_joint_forward_fg(const void* f, const void* g, int act, int64_t T_pad, int64_t Up_pad, void* h_out,
                         const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                         const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                         int64_t N, int32_t blank, int64_t max_u, void* workspace, size_t workspace_bytes,
                         int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                         float* grads, float* costs, void* stream);

/* Backward of cwr_joint_forward, one block of rows at a time: the logits of rows [0, R) of the block
 * are formed again on the matrix cores (fp32 accumulators) and turned in registers into
 *   dlogits[r, v] = g * (softmax(logits_r)[v] * gamma_r + grads[r,0] [v == blank] + grads[r,1] [v == label]),
 * cwr_backward's CWR_MODE_FUSED formula (cwarp_cuda_rnnt_kernel.cu:518-519 and
 * cwarp_cuda_gather_kernel.cu:52-74 behind a log-softmax), rounded once to `dtype` and written to
 * dlogits (R, V).  The caller multiplies the block into dh = dlogits w, dW += dlogits^T h,
 * dbias += column sums (plain GEMMs) and reuses the buffer for the next block, so that at most one
 * block of logit gradients exists at a time.  The reference repository has no joiner.
 *   h, rowinfo, grads, lse, dlogits  point at the block's first row;  rowinfo, grads, lse as
 *   written by cwr_joint_forward;  w, bias, dtype, H, V, N, blank as there;
 *   dlogits  aligned to 16 bytes when V is a multiple of 8 (rows then leave as 16-byte stores), to
 *            8 bytes when V is a multiple of 4, else to its element size;
 *   grad_costs, grad_stride, grad_scale as for cwr_backward. */
int cwr_joint_backward(const void* h, const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                       int64_t N, int32_t blank, const int32_t* rowinfo, const float* grads, const float* lse,
                       const float* grad_costs, int64_t grad_stride, float grad_scale, void* dlogits, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CWARP_RNNT_HIP_H */
