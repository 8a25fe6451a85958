// Fused output layer of the joiner: logits[r, v] = sum_k h[r, k] * W[v, k] + bias[v] are formed
// tile by tile on the matrix cores and consumed where they are formed, so that the (R, V) logits
// never exist in memory.
//
//   forward   k_joint_fwd: per compact row the log-sum-exp over V and the blank / label logits,
//             i.e. exactly what the gather pass of the loss (cwarp_cuda_gather_kernel.cu:19-43 plus
//             the log-softmax the reference's callers run first, test/test.py:19-20) extracts from
//             stored logits; the lattice then runs as usual.
//   backward  k_joint_dz: the same tiles are formed again and turned, in registers, into
//             d loss / d logits = softmax * gamma + [blank] + [label] terms (what the gradient pass of
//             the loss would write from stored logits, cwarp_cuda_gather_kernel.cu:52-74 plus the
//             log-softmax backward), rounded once to the 16-bit type and written for a block of rows
//             at a time; the caller multiplies that block into dh, dW and dbias and reuses the buffer.
//
// The reference repository has no joiner; its callers hand stored logits to
// cwarp_rnnt/__init__.py:32-73.
//
// gfx950, wave64, v_mfma_f32_32x32x16 on 16-bit inputs with fp32 accumulation.  The product is
// formed TRANSPOSED, C^T = W_tile * h_tile^T: in the accumulator layout of a 32x32 block a lane then
// holds 16 vocabulary entries of ONE data row, so the running maximum and the sum of exponentials of
// a row (forward) and the row's gradient coefficients (backward) are per-lane values, with no
// cross-lane traffic until the very end.  Two tilings share the per-tile work:
//   resident   (the joint sizes in use) a wave keeps the operand fragments of its own 32 or 64 data
//              rows in registers for the whole kernel and only the weight tile travels through LDS;
//   streaming  (any H that is a multiple of 32) a workgroup of four waves owns 256 rows and walks the
//              vocabulary in tiles of 128, both operand tiles through LDS in K-slices of 32; waves
//              split the tile 2 x 2: wave (wd, wv) multiplies the data rows [128 wd, 128 wd + 128)
//              with the vocabulary entries [64 wv, 64 wv + 64) of the tile.
#include "cwr_act.hpp"
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// streaming tiling
constexpr int kJM = 256;     // data rows per workgroup
constexpr int kJN = 128;     // vocabulary entries per tile
constexpr int kJK = 32;      // K-slice
constexpr int kJPitch = 40;  // LDS row pitch in elements: 80 bytes, so that the 16-byte reads of 16 consecutive
                             // rows fall into 16 different groups of four banks

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
    static __device__ __forceinline__ f32x16 mac(v4i a, v4i b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
};
template <> struct Mfma<__half> {
    static __device__ __forceinline__ f32x16 mac(v4i a, v4i b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
};

// (maximum, sum of exp(x - maximum)) of two disjoint sets merged; a set that is empty has -inf, 0
__device__ __forceinline__ void lse_merge(float& m, float& s, float m2, float s2) {
    const float mn = fmaxf(m, m2);
    const float a = m == mn ? s : s * fast_exp2((m - mn) * kLog2e);
    const float b = m2 == mn ? s2 : s2 * fast_exp2((m2 - mn) * kLog2e);
    m = mn;
    s = a + b;
}

// Vocabulary entry held by accumulator register r of a 32x32 block, relative to the block's first
// entry, for a lane of half `hf` = lane / 32 (the block's data row is lane % 32).
__device__ __forceinline__ constexpr int acc_row(int r, int hf) { return 8 * (r >> 2) + 4 * hf + (r & 3); }

// The walk of the streaming kernels: every complete tile of logits is handed to
// tile(acc, first vocabulary entry of this wave's part); acc[mv][nd] is the 32x32 block of vocabulary
// entries [32 mv, 32 mv + 32) of the wave's part and data rows [32 nd, 32 nd + 32) of its 128.
template <typename T> struct StreamLds {
    T h[2][kJM][kJPitch];
    T w[2][kJN][kJPitch];
    float bias[2][kJN];  // what the accumulators of a tile start from
};

template <typename T, typename TileFn>
__device__ __forceinline__ void walk_streaming(const T* __restrict__ h, const T* __restrict__ W,
                                               const float* __restrict__ bias, i64 R, int H, int V, i64 row0,
                                               StreamLds<T>& lds, TileFn&& tile) {
    auto& s_h = lds.h;
    auto& s_w = lds.w;
    auto& s_bias = lds.bias;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wd = w & 1, wv = w >> 1;
    const int hf = lane >> 5, l32 = lane & 31;

    // ---- global -> LDS staging: thread t moves 16-byte piece (t % 4) of rows t / 4 + 64 p ----------
    // The loads of a K-slice are issued TWO slices ahead of its use (two register sets taking turns):
    // one slice of matrix work is shorter than a trip to L2.
    const int st_row = tid >> 2, st_piece = tid & 3;
    // rows beyond the tensor are multiplied like the last one and dropped
    const i64 last_row = R - 1;
    const int nk = H / kJK;
    const int nvt = (V + kJN - 1) / kJN;
    const int iters = nk * nvt;
    struct Pre { v4i h[4], w[2]; };
    Pre pre[2];

    auto fetch = [&](int it, Pre& q) {
        const int vt = it / nk, kc = it - vt * nk;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            i64 r = row0 + st_row + 64 * p;
            r = r < last_row ? r : last_row;
            q.h[p] = *reinterpret_cast<const v4i*>(h + r * (i64)H + kc * kJK + st_piece * 8);
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            int v = vt * kJN + st_row + 64 * p;
            if (v >= V) v = V - 1;  // entries beyond the vocabulary are masked in the accumulator
            q.w[p] = *reinterpret_cast<const v4i*>(W + (i64)v * H + kc * kJK + st_piece * 8);
        }
    };
    auto stage = [&](int buf, const Pre& q) {
#pragma unroll
        for (int p = 0; p < 4; ++p) *reinterpret_cast<v4i*>(&s_h[buf][st_row + 64 * p][st_piece * 8]) = q.h[p];
#pragma unroll
        for (int p = 0; p < 2; ++p) *reinterpret_cast<v4i*>(&s_w[buf][st_row + 64 * p][st_piece * 8]) = q.w[p];
    };

    // the bias of a tile (-inf beyond the vocabulary, which no finite product changes and which drops
    // out of both the maximum and the sum) is fetched by the first 128 threads one tile ahead
    auto bias_of = [&](int vt) {
        const int v = vt * kJN + tid;
        return v < V ? (bias ? bias[v] : 0.f) : -INFINITY;
    };
    float bias_next = 0.f;
    if (tid < kJN) s_bias[0][tid] = bias_of(0);

    f32x16 acc[2][4];
    fetch(0, pre[0]);
    if (iters > 1) fetch(1, pre[1]);
    stage(0, pre[0]);
    __syncthreads();

    // one slice: slice `it` is multiplied out of LDS buffer it & 1; the loads of slice it + 2 go out
    // into the register set that slice it's own loads came through, and slice it + 1 (loaded during
    // slice it - 1) moves from the other set into the other buffer
    auto slice = [&](const int it, Pre& mine, Pre& next) {
        const int vt = it / nk, kc = it - vt * nk;
        const int buf = it & 1;
        const int v_wave = vt * kJN + 64 * wv;  // first vocabulary entry of this wave's part of the tile
        if (kc == 0) {
#pragma unroll
            for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const float4 bq = *reinterpret_cast<const float4*>(&s_bias[vt & 1][64 * wv + 32 * mv + 8 * b4 + 4 * hf]);
#pragma unroll
                    for (int nd = 0; nd < 4; ++nd) {
                        acc[mv][nd][4 * b4 + 0] = bq.x; acc[mv][nd][4 * b4 + 1] = bq.y;
                        acc[mv][nd][4 * b4 + 2] = bq.z; acc[mv][nd][4 * b4 + 3] = bq.w;
                    }
                }
            if (tid < kJN && vt + 1 < nvt) bias_next = bias_of(vt + 1);
        }
        if (kc == nk - 1 && tid < kJN && vt + 1 < nvt) s_bias[(vt + 1) & 1][tid] = bias_next;  // before the barrier below
        if (it + 2 < iters) fetch(it + 2, mine);
#pragma unroll
        for (int ks = 0; ks < kJK / 16; ++ks) {
            v4i fa[2], fb[4];
#pragma unroll
            for (int mv = 0; mv < 2; ++mv)
                fa[mv] = *reinterpret_cast<const v4i*>(&s_w[buf][64 * wv + 32 * mv + l32][16 * ks + 8 * hf]);
#pragma unroll
            for (int nd = 0; nd < 4; ++nd)
                fb[nd] = *reinterpret_cast<const v4i*>(&s_h[buf][128 * wd + 32 * nd + l32][16 * ks + 8 * hf]);
#pragma unroll
            for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                for (int nd = 0; nd < 4; ++nd) acc[mv][nd] = Mfma<T>::mac(fa[mv], fb[nd], acc[mv][nd]);
        }
        if (it + 1 < iters) stage(buf ^ 1, next);
        __syncthreads();
        if (kc != nk - 1) return;

        tile(acc, v_wave);
    };
    for (int it = 0; it < iters; it += 2) {
        slice(it, pre[0], pre[1]);
        if (it + 1 < iters) slice(it + 1, pre[1], pre[0]);
    }

}

// ---------------------------------------------------------------------------------------------
// what the forward kernels do with a finished tile
// ---------------------------------------------------------------------------------------------
// Per lane and data row: the running (maximum, sum of exponentials) over the vocabulary entries the
// lane has seen, and the two logits the loss wants (0 until seen; exactly one lane sees each).
template <int ND> struct FwdRows {
    float m[ND], s[ND], xl[ND], xb[ND];
    int lab[ND];
};

// The rows' labels, in two steps around the loads of the resident rows.  begin: for up to 64 sequences
// lane i asks for everything about sequence i (one round of loads, the oldest in the queue);
// finish: a ballot places the wave's first row, the lanes step over the few sequence boundaries
// inside the wave's rows, cross-lane reads hand out the sequence's values, and the label itself is
// the one dependent load (needed when the first tile is folded).  More sequences than lanes: the
// rows are placed by a search through memory in begin.
struct SeqTable {
    i64 off, pad, lab;
    int T, U;
};

template <int ND>
__device__ __forceinline__ SeqTable fwd_rows_begin(FwdRows<ND>& q, i64 rbase, i64 R, const int* __restrict__ lx,
                                                   const int* __restrict__ ly, const int* __restrict__ y,
                                                   i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
                                                   const i64* __restrict__ lab_off, const i64* __restrict__ pad_off,
                                                   int N, int V, int* __restrict__ status) {
    SeqTable tb;
    tb.off = 0x7fffffffffffffffLL; tb.pad = -1; tb.lab = 0; tb.T = 0; tb.U = 0;
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) { q.m[nd] = -INFINITY; q.s[nd] = 0.f; q.xl[nd] = 0.f; q.xb[nd] = 0.f; q.lab[nd] = kNoLabel; }
    const int lane = threadIdx.x & 63;
    if (N <= 64) {
        if (lane < N) {
            tb.off = row_off[lane]; tb.pad = pad_off[lane]; tb.lab = lab_off[lane];
            tb.T = lx[lane]; tb.U = ly[lane];
        }
        return tb;
    }
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = rbase + 32 * nd;
        if (r < R) {
            const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
            if (ri.n >= 0 && pad_off[ri.n] >= 0) q.lab[nd] = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        }
    }
    return tb;
}

__device__ __forceinline__ i64 lane_i64(i64 v, int src) {  // v of lane src (src may differ between lanes)
    const int lo = __shfl((int)(v & 0xffffffffLL), src), hi = __shfl((int)(v >> 32), src);
    return ((i64)hi << 32) | (i64)(unsigned)lo;
}

template <int ND>
__device__ __forceinline__ void fwd_rows_finish(FwdRows<ND>& q, const SeqTable& tb, i64 row0, i64 rbase, i64 R,
                                                const int* __restrict__ y, i64 y_stride, i64 y_len, int N, int V,
                                                int* __restrict__ status) {
    if (N > 64 || N <= 0) return;
    const unsigned long long m = __ballot(tb.off <= row0);
    const int n0 = m ? 63 - __clzll((long long)m) : 0;  // sequence of the wave's first row
    const i64 r_last = row0 + 32 * ND - 1;
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = rbase + 32 * nd;
        int n = n0;
        for (int j = n0 + 1; j < N; ++j) {
            const i64 oj = lane_i64(tb.off, j);
            if (oj > r_last) break;
            n += oj <= r ? 1 : 0;
        }
        const i64 off = lane_i64(tb.off, n), pad = lane_i64(tb.pad, n), labbase = lane_i64(tb.lab, n);
        const int T = __shfl(tb.T, n), U = __shfl(tb.U, n);
        const i64 rem = r - off;
        const i64 cells = (i64)T * (i64)(U + 1);
        if (r >= R || T <= 0 || U < 0 || rem < 0 || rem >= cells || off + cells > R || pad < 0) continue;
        const int u = cells < 0x7fffffffLL ? (int)((unsigned)rem % (unsigned)(U + 1)) : (int)(rem % (U + 1));
        if (u >= U) continue;
        const i64 at = (y_stride >= 0 ? (i64)n * y_stride : labbase) + u;
        const int lab = (at >= 0 && at < y_len && (y_stride < 0 || u < y_stride)) ? y[at] : -1;
        if (lab < 0 || lab >= V) { raise_flag(status, CWR_FLAG_BAD_LABEL); q.lab[nd] = kBadLabel; } else q.lab[nd] = lab;
    }
}

// acc[mv][nd]: vocabulary entries v_first + 32 mv + acc_row(., hf) of the lane's data row nd
template <int NMV, int ND>
__device__ __forceinline__ void fwd_fold_tile(const f32x16 (&acc)[NMV][ND], int v_first, int blank, int hf,
                                              FwdRows<ND>& q) {
    constexpr int SPAN = 32 * NMV;
    const int blank_key = (blank >= v_first && blank < v_first + SPAN && (((blank - v_first) >> 2) & 1) == hf)
                              ? blank - v_first : -1;
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        float mx = acc[0][nd][0];
#pragma unroll
        for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc[mv][nd][r]);
        const float mn = fmaxf(q.m[nd], mx);
        if (mn > -INFINITY) {
            const float ms = mn * kLog2e;
            float sum = 0.f;
#pragma unroll
            for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += fast_exp2(fmaf(acc[mv][nd][r], kLog2e, -ms));
            // every exponent above is off by what ms lost to rounding (up to half an ulp of
            // mn log2 e, the same for the whole tile): the fma recovers it exactly, so that s stays
            // the sum of exp(x - m) and a row whose cost is tiny keeps its absolute accuracy
            const float kept = q.m[nd] == mn ? q.s[nd] : q.s[nd] * fast_exp2((q.m[nd] - mn) * kLog2e);  // -inf: 0
            q.s[nd] = fmaf(sum, fmaf(-fmaf(mn, kLog2e, -ms), kLn2, 1.f), kept);
            q.m[nd] = mn;
        }
        // the label's logit, if it sits in this lane's half of this part of the tile
        const int lv = q.lab[nd] - v_first;
        const int key = (q.lab[nd] >= 0 && lv >= 0 && lv < SPAN && ((lv >> 2) & 1) == hf) ? lv : -1;
        if (__ballot(key >= 0) != 0) {
#pragma unroll
            for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
                for (int r = 0; r < 16; ++r) q.xl[nd] = key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : q.xl[nd];
        }
        if (__ballot(blank_key >= 0) != 0) {
#pragma unroll
            for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    q.xb[nd] = blank_key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : q.xb[nd];
        }
    }
}

// the two halves of a wave hold disjoint vocabulary entries of the same rows
template <int ND> __device__ __forceinline__ void fwd_merge_halves(FwdRows<ND>& q) {
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        lse_merge(q.m[nd], q.s[nd], __shfl_xor(q.m[nd], 32), __shfl_xor(q.s[nd], 32));
        q.xl[nd] += __shfl_xor(q.xl[nd], 32);  // exactly one half held the entry, the other 0
        q.xb[nd] += __shfl_xor(q.xb[nd], 32);
    }
}

struct FwdOut {
    LpStore lp;
    float* lse;
    int2* rowinfo;
    float2* grads_skipped;
    int* seqmode;
};

__device__ __forceinline__ void fwd_row_out(i64 r, i64 R, float m, float s, float xb, float xl, int lab,
                                            const int* __restrict__ lx, const int* __restrict__ ly,
                                            const i64* __restrict__ row_off, const i64* __restrict__ pad_off, int N,
                                            const FwdOut& o) {
    const Lse lse = {m, log2_of_sum(s)};
    o.lse[r] = lse.value();
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    o.rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
    if (pad >= 0)
        o.lp[pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1)] = make_lp(xb, xl, lse, lab, o.seqmode + ri.n);
    else if (o.grads_skipped) o.grads_skipped[r] = make_float2(0.f, 0.f);
}

// ---------------------------------------------------------------------------------------------
// what the backward kernels do with a finished tile
// ---------------------------------------------------------------------------------------------
// Per lane and data row the coefficients of
//   dz[r, v] = softmax(z_r)[v] * cg + [v == blank] * cb + [v == label] * cl,   softmax = 2^(z log2 e + nls)
// i.e. cwr_backward's CWR_MODE_FUSED formula on logits that live in the accumulators.
template <int ND> struct DzRows {
    float cg[ND], cb[ND], cl[ND], nls[ND];
    int lab[ND];
};

// in two steps around the loads of the resident rows: the row records are requested first (begin);
// the coefficients, which need one dependent load (the sequence's incoming gradient), are formed
// once the rows' loads are out (finish)
template <int ND> struct DzRaw {
    int2 info[ND];
    float2 g[ND];
    float lse[ND];
};

template <int ND>
__device__ __forceinline__ void dz_rows_begin(DzRaw<ND>& w, i64 rbase, i64 R, const int2* __restrict__ rowinfo,
                                              const float2* __restrict__ grads, const float* __restrict__ lse) {
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = rbase + 32 * nd;
        w.info[nd] = make_int2(-1, -1); w.g[nd] = make_float2(0.f, 0.f); w.lse[nd] = 0.f;
        if (r >= R) continue;
        w.info[nd] = rowinfo[r]; w.g[nd] = grads[r]; w.lse[nd] = lse[r];
    }
}

template <int ND>
__device__ __forceinline__ void dz_rows_finish(DzRows<ND>& q, const DzRaw<ND>& w, i64 rbase, i64 R, int N,
                                               const GradOut go) {
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        q.cg[nd] = 0.f; q.cb[nd] = 0.f; q.cl[nd] = 0.f; q.lab[nd] = -1;
        q.nls[nd] = -INFINITY;  // a row of no usable sequence: 2^-inf * 0 = 0 whatever its logits
        const int2 info = w.info[nd];
        if (rbase + 32 * nd >= R || info.y < 0 || info.y >= N) continue;
        const float g = go.p[(i64)info.y * go.stride] * go.scale;
        const float2 gr = w.g[nd];
        q.lab[nd] = info.x;
        q.cb[nd] = gr.x * g;
        q.cl[nd] = info.x >= 0 ? gr.y * g : 0.f;
        q.cg[nd] = -(gr.x + (info.x >= 0 ? gr.y : 0.f)) * g;
        q.nls[nd] = -w.lse[nd] * kLog2e;
    }
}

template <typename T> struct Pack4;
template <> struct Pack4<bf16_t> {
    typedef __bf16 h2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ uint2 of(const float (&o)[4]) {
        const h2 a = {(__bf16)o[0], (__bf16)o[1]}, b = {(__bf16)o[2], (__bf16)o[3]};
        return make_uint2(__builtin_bit_cast(unsigned, a), __builtin_bit_cast(unsigned, b));
    }
};
template <> struct Pack4<__half> {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ uint2 of(const float (&o)[4]) {
        const h2 a = {(_Float16)o[0], (_Float16)o[1]}, b = {(_Float16)o[2], (_Float16)o[3]};
        return make_uint2(__builtin_bit_cast(unsigned, a), __builtin_bit_cast(unsigned, b));
    }
};

// A wave's corner of LDS for turning a block of logit gradients (a lane holds runs of four entries
// of ONE row, 32 rows side by side: 8-byte stores 2 V bytes apart) into whole rows: written as the
// lanes hold it, read back with 16 lanes per row, stored as 64 NMV contiguous bytes per row.  Without
// it the stores cost a fifth of the kernel (0.60 -> 0.49 ms with the stores removed).
template <typename T, int NMV, int WAVES = 4> struct DzTranspose {
    static constexpr int kPitch = 32 * NMV + 8;  // elements; rows stay 16-byte aligned
    T rows[WAVES][32 * kPitch];
};

// acc[mv][nd] as in fwd_fold_tile; rbase = the lane's data row of nd = 0.  A lane holds runs of four
// consecutive vocabulary entries of one row.  FAST: the whole tile lies inside the tensor and rows
// start on 8-byte boundaries (V a multiple of 4): every run leaves as one unguarded 8-byte store.
// Otherwise element by element, guarded.  BLANK: the blank column lies in this part of the tile.
template <typename T, int NMV, int ND, bool FAST, bool BLANK>
__device__ __forceinline__ void dz_store_tile_as(const f32x16 (&acc)[NMV][ND], int v_first, int V, int blank, int hf,
                                                 i64 rbase, i64 R, const DzRows<ND>& q, T* __restrict__ dz, T* tbuf) {
    constexpr int kTP = DzTranspose<T, NMV>::kPitch;
    const int lane = threadIdx.x & 63, l32 = lane & 31;
    const int bl = blank - v_first;  // same for the whole wave
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = rbase + 32 * nd;
        // the label's place among the entries of this lane's half, or -1
        const int lv = q.lab[nd] - v_first - 4 * hf;
        const int key = (q.lab[nd] >= 0 && lv >= 0 && lv < 32 * NMV && (lv & 4) == 0) ? lv : -1;
        T* row = dz + r * (i64)V + v_first + 4 * hf;
#pragma unroll
        for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                const int e0 = 32 * mv + 8 * b4;  // entry of o[0], relative to v_first + 4 hf
                float o[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float p = fast_exp2(fmaf(acc[mv][nd][4 * b4 + c], kLog2e, q.nls[nd]));
                    o[c] = fmaf(p, q.cg[nd], key == e0 + c ? q.cl[nd] : 0.f);
                }
                if (BLANK && bl >= e0 && bl < e0 + 8) {  // it lies in this run of one of the two halves
                    const int cb_at = bl - e0 - 4 * hf;
#pragma unroll
                    for (int c = 0; c < 4; ++c) o[c] += c == cb_at ? q.cb[nd] : 0.f;
                }
                if (FAST) {
                    if (tbuf) *reinterpret_cast<uint2*>(tbuf + l32 * kTP + e0 + 4 * hf) = Pack4<T>::of(o);
                    else *reinterpret_cast<uint2*>(row + e0) = Pack4<T>::of(o);
                    continue;
                }
                if (r >= R) continue;
                const int v = v_first + 4 * hf + e0;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (v + c < V) row[e0 + c] = Elem<T>::from_f32(o[c]);
            }
        if (FAST && tbuf) {
            // back out of LDS a row at a time: PPR lanes take the 16-byte pieces of one row's 32 NMV entries
            constexpr int PPR = 4 * NMV, RPI = 64 / PPR;
            const int rr = lane / PPR, pc = lane % PPR;
            T* out = dz + (rbase - l32 + 32 * nd + rr) * (i64)V + v_first + pc * 8;
#pragma unroll
            for (int j = 0; j < 32 / RPI; ++j)
                *reinterpret_cast<v4i*>(out + (i64)(j * RPI) * V) =
                    *reinterpret_cast<const v4i*>(tbuf + (rr + j * RPI) * kTP + pc * 8);
        }
    }
}

// wave_rows_end: one past the last data row of this wave; tbuf: this wave's DzTranspose rows, or null
template <typename T, int NMV, int ND>
__device__ __forceinline__ void dz_store_tile(const f32x16 (&acc)[NMV][ND], int v_first, int V, int blank, int hf,
                                              i64 rbase, i64 wave_rows_end, i64 R, const DzRows<ND>& q,
                                              T* __restrict__ dz, T* tbuf) {
    const bool fast = (V & 3) == 0 && v_first + 32 * NMV <= V && wave_rows_end <= R;
    const bool has_blank = blank >= v_first && blank < v_first + 32 * NMV;
    T* const tb = (V & 7) == 0 ? tbuf : nullptr;
    if (fast && !has_blank) dz_store_tile_as<T, NMV, ND, true, false>(acc, v_first, V, blank, hf, rbase, R, q, dz, tb);
    else if (fast) dz_store_tile_as<T, NMV, ND, true, true>(acc, v_first, V, blank, hf, rbase, R, q, dz, tb);
    else dz_store_tile_as<T, NMV, ND, false, true>(acc, v_first, V, blank, hf, rbase, R, q, dz, nullptr);
}

// ---------------------------------------------------------------------------------------------
// streaming kernels (any H that is a multiple of 32)
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256, 2) void k_joint_fwd(
    const T* __restrict__ h, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int H, int V,
    const int* __restrict__ lx, const int* __restrict__ ly, const int* __restrict__ y, i64 y_stride, i64 y_len,
    const i64* __restrict__ row_off, const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N,
    int blank, const FwdOut out, int* __restrict__ status) {
    __shared__ __attribute__((aligned(16))) StreamLds<T> lds;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wd = w & 1, wv = w >> 1;
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * kJM;
    const i64 rbase = row0 + 128 * wd + l32;  // the rows this lane reduces: rbase + 32 nd, nd = 0..3

    FwdRows<4> q;
    const SeqTable tb = fwd_rows_begin<4>(q, rbase, R, lx, ly, y, y_stride, y_len, row_off, lab_off, pad_off, N, V, status);
    fwd_rows_finish<4>(q, tb, row0 + 128 * wd, rbase, R, y, y_stride, y_len, N, V, status);
    walk_streaming<T>(h, W, bias, R, H, V, row0, lds,
                      [&](const f32x16 (&acc)[2][4], int v_wave) { fwd_fold_tile<2, 4>(acc, v_wave, blank, hf, q); });

    // ---- merge: the two halves of a wave, then the two waves that share the data rows ----------
    float* s_merge = reinterpret_cast<float*>(&lds.h[0][0][0]);  // the staging buffers are free now
    fwd_merge_halves<4>(q);
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) {
        if (wv == 1 && hf == 0) {
            float* p = s_merge + ((wd * 4 + nd) * 32 + l32) * 4;
            p[0] = q.m[nd]; p[1] = q.s[nd]; p[2] = q.xl[nd]; p[3] = q.xb[nd];
        }
    }
    __syncthreads();
    if (wv != 0 || hf != 0) return;
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) {
        const i64 r = rbase + 32 * nd;
        if (r >= R) continue;
        const float* p = s_merge + ((wd * 4 + nd) * 32 + l32) * 4;
        lse_merge(q.m[nd], q.s[nd], p[0], p[1]);
        fwd_row_out(r, R, q.m[nd], q.s[nd], q.xb[nd] + p[3], q.xl[nd] + p[2], q.lab[nd], lx, ly, row_off, pad_off, N,
                    out);
    }
}

template <typename T>
__global__ __launch_bounds__(256, 2) void k_joint_dz(
    const T* __restrict__ h, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int H, int V, int N,
    int blank, const int2* __restrict__ rowinfo, const float2* __restrict__ grads, const float* __restrict__ lse,
    const GradOut go, T* __restrict__ dz) {
    __shared__ __attribute__((aligned(16))) StreamLds<T> lds;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wd = w & 1;
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * kJM;
    const i64 rbase = row0 + 128 * wd + l32;
    DzRows<4> q;
    DzRaw<4> raw;
    dz_rows_begin<4>(raw, rbase, R, rowinfo, grads, lse);
    dz_rows_finish<4>(q, raw, rbase, R, N, go);
    walk_streaming<T>(h, W, bias, R, H, V, row0, lds, [&](const f32x16 (&acc)[2][4], int v_wave) {
        dz_store_tile<T, 2, 4>(acc, v_wave, V, blank, hf, rbase, row0 + 128 * wd + 128, R, q, dz, nullptr);
    });
}

// ---------------------------------------------------------------------------------------------
// data rows resident in registers
// ---------------------------------------------------------------------------------------------
// The streaming kernels above read their h tile once per vocabulary tile: V / 128 times in all, from
// HBM, since the tiles of all resident workgroups together exceed the L2 (measured on N=32, V=1024,
// H=512: 3.3 GB fetched for 0.32 GB of h, and the kernel runs at the speed of that traffic).  Here
// every wave keeps the MFMA operand fragments of its OWN 32 ND data rows in registers for the whole
// kernel (ND * H / 16 registers of 16 bytes per lane: the whole K range), so h is read exactly once;
// only the weight tile travels through LDS, in K-slices of 64, and every wave multiplies its rows
// with the whole tile of 128 vocabulary entries.  Needs H known at compile time (the fragments are
// indexed statically).
// (the weight tile's K-slice RK is a parameter; its LDS rows are RK + 8 elements apart: 16 bytes past a
// multiple of 128, so that 8 consecutive rows start in 8 different groups of four banks)

// Workgroup barrier that waits for this wave's LDS traffic only, never for the global loads it has in
// flight (a __syncthreads() drains those too: the weight loads issued ahead, and at the start of
// a workgroup the loads of the resident rows).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0); vmcnt and expcnt untouched
    __builtin_amdgcn_s_barrier();
}

template <typename T, int NMV, int RK> struct ResLds {
    T w[2][32 * NMV][RK + 8];
    float bias[2][32 * NMV];  // what the accumulators of a tile start from
};

// this wave's data rows [row0, row0 + 32 ND), as MFMA operand fragments
template <typename T, int ND, int KS /* H / 16 */>
__device__ __forceinline__ void load_resident_rows(const T* __restrict__ h, i64 R, i64 row0, v4i (&hreg)[ND][KS]) {
    const int lane = threadIdx.x & 63;
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 last_row = R - 1;
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        i64 r = row0 + 32 * nd + l32;
        r = r < last_row ? r : last_row;  // rows beyond the tensor are multiplied like the last one and dropped
        const T* src = h + r * (i64)(KS * 16) + 8 * hf;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) hreg[nd][ks] = *reinterpret_cast<const v4i*>(src + 16 * ks);
    }
}

// The same fragments formed on the spot from the joiner's two inputs, row(n,t,u) = act(f[n,t,:] +
// g[n,u,:]) (the arithmetic of the join kernels: sum and activation in fp32, one rounding to the
// 16-bit type), for callers that never want the (R,H) joint rows in memory: f and g are a few MB and
// come out of the L2.  h_out (may be null) receives the rows for a backward pass that needs them.
template <typename T> struct JoinSrc {
    const T* f;
    const T* g;
    T* h_out;
    int act;
    int T_pad, Up_pad;
    const int* lx;
    const int* ly;
    const i64* row_off;
    int N;
    int* status;
};

template <typename T, int ACT, int ND, int KS>
__device__ __forceinline__ void join_resident_rows_as(const JoinSrc<T>& s, i64 R, i64 row0, v4i (&hreg)[ND][KS]) {
    constexpr int H = KS * 16;
    const int lane = threadIdx.x & 63;
    const int hf = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = row0 + 32 * nd + l32;
        const RowInfo ri = decode_row(r < R ? r : R - 1, R, s.row_off, s.lx, s.ly, s.N);
        const bool ok = ri.n >= 0 && ri.t < s.T_pad && ri.u < s.Up_pad;
        if (ri.n >= 0 && !ok) raise_flag(s.status, CWR_FLAG_BAD_LENGTH);  // the cell lies outside the padded inputs
        // a row no valid cell maps to is a row of zeros, as in the join kernels
        const T* pf = s.f + (ok ? ((i64)ri.n * s.T_pad + ri.t) * H : 0) + 8 * hf;
        const T* pg = s.g + (ok ? ((i64)ri.n * s.Up_pad + ri.u) * H : 0) + 8 * hf;
        T* po = (s.h_out && r < R) ? s.h_out + r * (i64)H + 8 * hf : nullptr;
        // All of f's fragments are requested at once, straight into the registers the row will live
        // in; g's follow in batches of kBatch into spare registers and each batch is folded in as it
        // arrives.  (One fragment of each at a time, which is what the loop would otherwise compile
        // to, pays a trip to the L2 per fragment: 32 of them in a row at H = 512.)
        constexpr int kBatch = (KS >= 24 || KS % 8 != 0) ? 4 : 8;  // the longer the resident row, the fewer spare registers
        static_assert(KS % kBatch == 0, "whole batches");
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) hreg[nd][ks] = *reinterpret_cast<const v4i*>(pf + 16 * ks);
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += kBatch) {
            v4i gq[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) gq[i] = *reinterpret_cast<const v4i*>(pg + 16 * (k0 + i));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                PackT<T, 8> a, b, o;
                __builtin_memcpy(&a, &hreg[nd][k0 + i], 16);
                __builtin_memcpy(&b, &gq[i], 16);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    o.e[e] = ok ? Arith<T>::down(activate<ACT, T>(Arith<T>::up(a.e[e]) + Arith<T>::up(b.e[e])))
                                : Arith<T>::down(0.f);
                v4i v;
                __builtin_memcpy(&v, &o, 16);
                hreg[nd][k0 + i] = v;
                if (po) *reinterpret_cast<v4i*>(po + 16 * (k0 + i)) = v;
                __builtin_amdgcn_sched_barrier(0);  // one fragment's temporaries at a time
            }
        }
    }
}

template <typename T, int ND, int KS>
__device__ __forceinline__ void join_resident_rows(const JoinSrc<T>& s, i64 R, i64 row0, v4i (&hreg)[ND][KS]) {
    if (s.act == kActTanh) join_resident_rows_as<T, kActTanh, ND, KS>(s, R, row0, hreg);
    else if (s.act == kActRelu) join_resident_rows_as<T, kActRelu, ND, KS>(s, R, row0, hreg);
    else join_resident_rows_as<T, kActNone, ND, KS>(s, R, row0, hreg);
}

// tile(acc, v0) receives acc[mv][nd] = vocabulary entries [v0 + 32 mv, v0 + 32 mv + 32) x data rows
// [row0 + 32 nd, row0 + 32 nd + 32) of this wave; the vocabulary is walked in tiles of JN = 32 NMV.
// Order of the start-up, which every workgroup of a round runs at the same time as every other: the
// first weight slice is requested, then the resident rows (from HBM), then after_issue() runs
// (what the caller still has to do about its rows: loads issued here queue up BEHIND the rows',
// whatever the caller asked for earlier is served before them), and the first tile starts as
// soon as the first fragments are there.
template <typename T, int ND, int KS, int NMV, int WAVES, int RK, bool D2, typename LoadRows, typename AfterIssue,
          typename TileFn>
__device__ __forceinline__ void walk_resident(LoadRows&& load_rows, const T* __restrict__ W,
                                              const float* __restrict__ bias, int V, ResLds<T, NMV, RK>& lds,
                                              AfterIssue&& after_issue, TileFn&& tile) {
    constexpr int JN = 32 * NMV;
    constexpr int H = KS * 16;
    constexpr int NK = H / RK;  // K-slices per vocabulary tile
    static_assert(H % RK == 0, "whole K-slices");
    auto& s_w = lds.w;
    auto& s_bias = lds.bias;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int hf = lane >> 5, l32 = lane & 31;

    // ---- weight tile: a row of the slice is PPR pieces of 16 bytes; thread t moves piece t % PPR of rows
    // t / PPR + RPP p ----------
    constexpr int PPR = RK / 8;
    constexpr int RPP = 64 * WAVES / PPR;  // rows the workgroup moves per pass
    constexpr int NP = JN / RPP;           // passes per K-slice
    static_assert(JN % RPP == 0, "whole passes");
    const int st_row = tid / PPR, st_piece = tid % PPR;
    struct Pre { v4i w[NP]; };
    Pre pre[D2 ? 2 : 1];
    const int nvt = (V + JN - 1) / JN;
    auto fetch = [&](int vt, int kc, Pre& q) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int v = vt * JN + st_row + RPP * p;
            if (v >= V) v = V - 1;  // entries beyond the vocabulary are masked in the accumulator
            q.w[p] = *reinterpret_cast<const v4i*>(W + (i64)v * H + kc * RK + st_piece * 8);
        }
    };
    auto stage = [&](int buf, const Pre& q) {
#pragma unroll
        for (int p = 0; p < NP; ++p) *reinterpret_cast<v4i*>(&s_w[buf][st_row + RPP * p][st_piece * 8]) = q.w[p];
    };

    // slices are numbered it = vt * NK + kc; slice it is multiplied out of buffer it & 1 (NK is even
    // or the parity is carried), its loads were issued two slices earlier
    // the bias of a tile (-inf beyond the vocabulary, which no finite product changes and which drops
    // out of both the maximum and the sum) is fetched by the first 128 threads one tile ahead
    auto bias_of = [&](int vt) {
        const int v = vt * JN + tid;
        return v < V ? (bias ? bias[v] : 0.f) : -INFINITY;
    };
    float bias_next = 0.f;
    if (tid < JN) s_bias[0][tid] = bias_of(0);
    v4i hreg[ND][KS];
    load_rows(hreg);
    after_issue();
    fetch(0, 0, pre[0]);
    if (D2 && (NK > 1 || nvt > 1)) fetch(NK > 1 ? 0 : 1, NK > 1 ? 1 : 0, pre[1]);
    stage(0, pre[0]);
    lds_barrier();

    f32x16 acc[NMV][ND];
    int par = 0;  // buffer of the current slice
    // one vocabulary tile.  The first is a copy of its own: it follows the loads of the resident rows
    // in straight-line code, so its K-steps wait for the fragments they use, one after the other,
    // instead of for all of them in front of the loop.
    auto one_tile = [&](const int vt) {
#pragma unroll
        for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                const float4 bq = *reinterpret_cast<const float4*>(&s_bias[vt & 1][32 * mv + 8 * b4 + 4 * hf]);
#pragma unroll
                for (int nd = 0; nd < ND; ++nd) {
                    acc[mv][nd][4 * b4 + 0] = bq.x; acc[mv][nd][4 * b4 + 1] = bq.y;
                    acc[mv][nd][4 * b4 + 2] = bq.z; acc[mv][nd][4 * b4 + 3] = bq.w;
                }
            }
        if (tid < JN && vt + 1 < nvt) bias_next = bias_of(vt + 1);
#pragma unroll
        for (int kc = 0; kc < NK; ++kc) {
            if (kc == NK - 1 && tid < JN && vt + 1 < nvt) s_bias[(vt + 1) & 1][tid] = bias_next;  // before its barrier
            // register set kc & 1 held this slice's loads (already staged); it now takes slice it + 2
            if (D2) {
                const int k2 = kc + 2;
                const int vt2 = vt + k2 / NK, kc2 = k2 % NK;
                if (vt2 < nvt) fetch(vt2, kc2, pre[(kc + (NK & 1) * vt) & 1]);
            } else {
                const int k1 = kc + 1;
                const int vt1 = vt + k1 / NK, kc1 = k1 % NK;
                if (vt1 < nvt) fetch(vt1, kc1, pre[0]);
            }
            // The four weight fragments of a K-step are requested together and the matrix
            // instructions follow as they arrive (left to itself the compiler reuses ONE fragment
            // register and pays the LDS latency in front of every matrix instruction).
#pragma unroll
            for (int ks = 0; ks < RK / 16; ++ks) {
                v4i fa[NMV];
#pragma unroll
                for (int mv = 0; mv < NMV; ++mv)
                    fa[mv] = *reinterpret_cast<const v4i*>(&s_w[par][32 * mv + l32][16 * ks + 8 * hf]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mv = 0; mv < NMV; ++mv)
#pragma unroll
                    for (int nd = 0; nd < ND; ++nd)
                        acc[mv][nd] = Mfma<T>::mac(fa[mv], hreg[nd][kc * (RK / 16) + ks], acc[mv][nd]);
                __builtin_amdgcn_sched_barrier(0);
            }
            {
                const int k1 = kc + 1;
                const int vt1 = vt + k1 / NK;
                if (vt1 < nvt) stage(par ^ 1, pre[D2 ? (kc + 1 + (NK & 1) * vt) & 1 : 0]);
            }
            lds_barrier();
            par ^= 1;
        }
        tile(acc, vt * JN);
    };
    one_tile(0);
    for (int vt = 1; vt < nvt; ++vt) one_tile(vt);
}

template <typename T, int ND, int KS, int NMV, int WAVES, int RK, int OCC, bool D2, bool FG>
__global__ __launch_bounds__(64 * WAVES, OCC) void k_joint_fwd_res(
    const T* __restrict__ h, const JoinSrc<T> js, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int V,
    const int* __restrict__ lx, const int* __restrict__ ly, const int* __restrict__ y, i64 y_stride, i64 y_len,
    const i64* __restrict__ row_off, const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N,
    int blank, const FwdOut out, int* __restrict__ status) {
    __shared__ __attribute__((aligned(16))) ResLds<T, NMV, RK> lds;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * (32 * ND * WAVES) + (i64)w * (32 * ND);  // first data row of this wave
    FwdRows<ND> q;
    const SeqTable tb = fwd_rows_begin<ND>(q, row0 + l32, R, lx, ly, y, y_stride, y_len, row_off, lab_off, pad_off, N, V,
                                           status);
    fwd_rows_finish<ND>(q, tb, row0, row0 + l32, R, y, y_stride, y_len, N, V, status);
    walk_resident<T, ND, KS, NMV, WAVES, RK, D2>(
        [&](v4i (&hreg)[ND][KS]) {
            if (FG) join_resident_rows<T, ND, KS>(js, R, row0, hreg);
            else load_resident_rows<T, ND, KS>(h, R, row0, hreg);
        },
        W, bias, V, lds, [&]() {},
        [&](const f32x16 (&acc)[NMV][ND], int v0) { fwd_fold_tile<NMV, ND>(acc, v0, blank, hf, q); });
    fwd_merge_halves<ND>(q);
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = row0 + 32 * nd + l32;
        if (hf != 0 || r >= R) continue;
        fwd_row_out(r, R, q.m[nd], q.s[nd], q.xb[nd], q.xl[nd], q.lab[nd], lx, ly, row_off, pad_off, N, out);
    }
}

template <typename T, int ND, int KS, int NMV, int WAVES, int RK, int OCC, bool D2>
__global__ __launch_bounds__(64 * WAVES, OCC) void k_joint_dz_res(
    const T* __restrict__ h, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int V, int N, int blank,
    const int2* __restrict__ rowinfo, const float2* __restrict__ grads, const float* __restrict__ lse,
    const GradOut go, T* __restrict__ dz) {
    __shared__ __attribute__((aligned(16))) ResLds<T, NMV, RK> lds;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * (32 * ND * WAVES) + (i64)w * (32 * ND);
    __shared__ __attribute__((aligned(16))) DzTranspose<T, NMV, WAVES> tr;
    T* tbuf = tr.rows[w];
    DzRows<ND> q;
    DzRaw<ND> raw;
    dz_rows_begin<ND>(raw, row0 + l32, R, rowinfo, grads, lse);
    walk_resident<T, ND, KS, NMV, WAVES, RK, D2>(
        [&](v4i (&hreg)[ND][KS]) { load_resident_rows<T, ND, KS>(h, R, row0, hreg); }, W, bias, V, lds,
        [&]() { dz_rows_finish<ND>(q, raw, row0 + l32, R, N, go); },
        [&](const f32x16 (&acc)[NMV][ND], int v0) {
            dz_store_tile<T, NMV, ND>(acc, v0, V, blank, hf, row0 + l32, row0 + 32 * ND, R, q, dz, tbuf);
        });
}

// The joint sizes in use take the resident kernels; any other multiple of 32 the streaming ones.
// X(ND, H / 16, NMV, WAVES, RK, workgroups per CU, two register sets of weight loads in flight).
// Measured on R = 311449, V = 1024, bf16, forward call (same GPU for every pair):
//   eight waves per workgroup, one workgroup per CU, against four waves, two workgroups (the same
//   two waves per SIMD, but one weight tile staged per 256 rows instead of per 128: half the L2
//   traffic, staging instructions and LDS writes per matrix instruction):
//       H = 256: 0.279 against 0.347 ms (two row blocks per wave, one wave per SIMD);
//       H = 384: 0.365 against 0.418;  H = 512: 0.46 against 0.49;  H = 640: 0.59 against 0.67 ms;
//       beyond H = 640 the fragments of 32 rows leave no room for two waves per SIMD;
//   K-slices of 128 or 256 instead of 64 (fewer barriers): 0.465 / 0.49 against 0.467 ms at H = 512;
//   two row blocks per wave at one wave per SIMD, H = 512: tiles of 128 entries 0.63 ms (registers
//   spill), tiles of 64 entries 0.49 ms (half the LDS reads per matrix instruction, but a lone wave
//   per SIMD hides neither the LDS latency nor the tile's reduction); streaming kernel 0.63 ms.
//   the backward kernel follows, except at H = 512 (0.61 against 0.57 ms: it keeps four waves).
//   the other multiples of 64 from 128 to 1024 take the shape of their larger neighbour,
//   with one register set of weight loads where the number of K-slices per tile is odd.
#define CWR_JOINT_SHAPES(X) X(1, 8, 4, 8, 64, 1, true) X(1, 12, 4, 8, 64, 1, false) X(1, 16, 4, 8, 64, 1, true) \
                            X(1, 20, 4, 8, 64, 1, false) X(1, 24, 4, 8, 64, 1, true) X(1, 28, 4, 8, 64, 1, false) \
                            X(1, 32, 4, 8, 64, 1, false) X(1, 36, 4, 8, 64, 1, false) X(1, 40, 4, 8, 64, 1, false) \
                            X(1, 44, 4, 4, 64, 1, false) X(1, 48, 4, 4, 64, 1, true) X(1, 52, 4, 4, 64, 1, false) \
                            X(1, 56, 4, 4, 64, 1, true) X(1, 60, 4, 4, 64, 1, false) X(1, 64, 4, 4, 64, 1, true)
#define CWR_JOINT_DZ_SHAPES(X) X(1, 8, 4, 8, 64, 1, true) X(1, 12, 4, 8, 64, 1, false) X(1, 16, 4, 8, 64, 1, true) \
                               X(1, 20, 4, 8, 64, 1, false) X(1, 24, 4, 8, 64, 1, true) X(1, 28, 4, 4, 64, 2, false) \
                               X(1, 32, 4, 4, 64, 2, false) X(1, 36, 4, 8, 64, 1, false) X(1, 40, 4, 8, 64, 1, false) \
                               X(1, 44, 4, 4, 64, 1, false) X(1, 48, 4, 4, 64, 1, true) X(1, 52, 4, 4, 64, 1, false) \
                            X(1, 56, 4, 4, 64, 1, true) X(1, 60, 4, 4, 64, 1, false) X(1, 64, 4, 4, 64, 1, true)

template <typename T>
static int joint_gather_typed(const Batch& b, const Workspace& ws, const JointOperands& j, float* lse, int* rowinfo,
                              float* grads) {
    const FwdOut out = {ws.lp, lse, reinterpret_cast<int2*>(rowinfo), reinterpret_cast<float2*>(grads), ws.seqmode};
    const T* h = static_cast<const T*>(j.h);
    const T* w = static_cast<const T*>(j.w);
    JoinSrc<T> js;
    js.f = static_cast<const T*>(j.f); js.g = static_cast<const T*>(j.g); js.h_out = static_cast<T*>(j.h_out);
    js.act = j.act; js.T_pad = (int)j.T_pad; js.Up_pad = (int)j.Up_pad;
    js.lx = b.lx; js.ly = b.ly; js.row_off = b.row_off; js.N = b.N; js.status = b.status;
    const bool fg = j.h == nullptr;
#define CWR_JOINT_RES(ND, KS, NMV, WAVES, RK, OCC, D2)                                                            \
    if (j.H == 16 * KS) {                                                                                         \
        const i64 blocks = (b.R + 32 * ND * WAVES - 1) / (32 * ND * WAVES);                                       \
        if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;                                                      \
        if (fg)                                                                                                   \
            CWR_LAUNCH((k_joint_fwd_res<T, ND, KS, NMV, WAVES, RK, OCC, D2, true>), dim3((unsigned)blocks),       \
                       dim3(64 * WAVES), 0, b.stream, h, js, w, j.bias, b.R, b.V, b.lx, b.ly, b.y, b.y_stride,    \
                       b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, out, b.status);                   \
        else                                                                                                      \
            CWR_LAUNCH((k_joint_fwd_res<T, ND, KS, NMV, WAVES, RK, OCC, D2, false>), dim3((unsigned)blocks),      \
                       dim3(64 * WAVES), 0, b.stream, h, js, w, j.bias, b.R, b.V, b.lx, b.ly, b.y, b.y_stride,    \
                       b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, out, b.status);                   \
        return check_launch();                                                                                    \
    }
    CWR_JOINT_SHAPES(CWR_JOINT_RES)
#undef CWR_JOINT_RES
    if (fg) return CWR_ERR_SHAPE;  // the rows are formed in registers: resident joint sizes only
    const i64 blocks = (b.R + kJM - 1) / kJM;
    if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
    CWR_LAUNCH((k_joint_fwd<T>), dim3((unsigned)blocks), dim3(256), 0, b.stream, h, w, j.bias, b.R, (int)j.H, b.V,
               b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, out, b.status);
    return check_launch();
}

int launch_joint_gather(const Batch& b, const Workspace& ws, const JointOperands& j, float* lse, int* rowinfo,
                        float* grads) {
    if (b.R == 0) return CWR_OK;
    if (b.dtype == CWR_BF16) return joint_gather_typed<bf16_t>(b, ws, j, lse, rowinfo, grads);
    if (b.dtype == CWR_F16) return joint_gather_typed<__half>(b, ws, j, lse, rowinfo, grads);
    return CWR_ERR_DTYPE;
}

template <typename T>
static int joint_dlogits_typed(const JointOperands& j, i64 R, int V, int N, int blank, const int* rowinfo,
                               const float* grads, const float* lse, const GradOut go, void* dlogits,
                               hipStream_t stream) {
    const int2* ri = reinterpret_cast<const int2*>(rowinfo);
    const float2* gr = reinterpret_cast<const float2*>(grads);
    const T* h = static_cast<const T*>(j.h);
    const T* w = static_cast<const T*>(j.w);
    T* dz = static_cast<T*>(dlogits);
#define CWR_JOINT_RES(ND, KS, NMV, WAVES, RK, OCC, D2)                                                                          \
    if (j.H == 16 * KS) {                                                                                       \
        const i64 blocks = (R + 32 * ND * WAVES - 1) / (32 * ND * WAVES);                                                  \
        if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;                                                    \
        CWR_LAUNCH((k_joint_dz_res<T, ND, KS, NMV, WAVES, RK, OCC, D2>), dim3((unsigned)blocks), dim3(64 * WAVES), 0, stream, h, w,    \
                   j.bias, R, V, N, blank, ri, gr, lse, go, dz);                                                \
        return check_launch();                                                                                  \
    }
    CWR_JOINT_DZ_SHAPES(CWR_JOINT_RES)
#undef CWR_JOINT_RES
    const i64 blocks = (R + kJM - 1) / kJM;
    if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
    CWR_LAUNCH((k_joint_dz<T>), dim3((unsigned)blocks), dim3(256), 0, stream, h, w, j.bias, R, (int)j.H, V, N, blank,
               ri, gr, lse, go, dz);
    return check_launch();
}

int launch_joint_dlogits(int dtype, const JointOperands& j, i64 R, i64 V, i64 N, int blank, const int* rowinfo,
                         const float* grads, const float* lse, const GradOut go, void* dlogits, hipStream_t stream) {
    if (R == 0) return CWR_OK;
    if (dtype == CWR_BF16)
        return joint_dlogits_typed<bf16_t>(j, R, (int)V, (int)N, blank, rowinfo, grads, lse, go, dlogits, stream);
    if (dtype == CWR_F16)
        return joint_dlogits_typed<__half>(j, R, (int)V, (int)N, blank, rowinfo, grads, lse, go, dlogits, stream);
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
