// Fused output layer of the joiner: logits[r, v] = sum_k h[r, k] * W[v, k] + bias[v] are formed
// tile by tile on the matrix cores and consumed where they are formed, so that the (R, V) logits
// never exist in memory.
//
//   forward   k_joint_fwd: per compact row the log-sum-exp over V and the blank / label logits,
//             i.e. exactly what the gather pass of the loss (cwarp_cuda_gather_kernel.cu:19-43 plus
//             the log-softmax the reference's callers run first, test/test.py:19-20) extracts from
//             stored logits; the lattice then runs as usual.
//
// The reference repository has no joiner; its callers hand stored logits to
// cwarp_rnnt/__init__.py:32-73.
//
// Tiling (gfx950, wave64, v_mfma_f32_32x32x16 on 16-bit inputs with fp32 accumulation).  A
// workgroup of four waves owns 256 compact rows and walks the vocabulary in tiles of 128; the two
// operand tiles travel through LDS in K-slices of 32, the next slice's global loads in flight
// while the current one is multiplied.  The product is formed TRANSPOSED, C^T = W_tile * h_tile^T:
// in the accumulator layout of a 32x32 block a lane then holds 16 vocabulary entries of ONE data
// row, so the running maximum and the sum of exponentials of a row are kept per lane with no
// cross-lane traffic until the very end.  Waves split the tile 2 x 2: wave (wd, wv) multiplies the
// data rows [128 wd, 128 wd + 128) with the vocabulary entries [64 wv, 64 wv + 64) of the tile.
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

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

template <typename T>
__global__ __launch_bounds__(256, 2) void k_joint_fwd(
    const T* __restrict__ h, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int H, int V,
    const int* __restrict__ lx, const int* __restrict__ ly, const int* __restrict__ y, i64 y_stride, i64 y_len,
    const i64* __restrict__ row_off, const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N,
    int blank, LpCell* __restrict__ lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    __shared__ __attribute__((aligned(16))) T s_h[2][kJM][kJPitch];
    __shared__ __attribute__((aligned(16))) T s_w[2][kJN][kJPitch];
    __shared__ __attribute__((aligned(16))) float s_bias[2][kJN];  // what the accumulators of a tile start from

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wd = w & 1, wv = w >> 1;
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * kJM;

    // ---- the rows this lane reduces: data rows row0 + 128 wd + 32 nd + l32, nd = 0..3 ----------
    // (only the label is needed during the walk over the vocabulary; the row's place in its lattice
    // is worked out again at the end rather than kept in registers all along)
    int lab[4];
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) {
        const i64 r = row0 + 128 * wd + 32 * nd + l32;
        lab[nd] = kNoLabel;
        if (r < R) {
            const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
            if (ri.n >= 0 && pad_off[ri.n] >= 0) lab[nd] = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        }
    }

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

    // running log-sum-exp state of the lane's rows over the vocabulary entries it has seen, and
    // the two logits the loss wants
    float m[4], s[4], xl[4], xb[4];
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) { m[nd] = -INFINITY; s[nd] = 0.f; xl[nd] = 0.f; xb[nd] = 0.f; }

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

        // ---- the tile's logits are complete: fold them into the rows' running state ----------
        const int blank_key = (blank >= v_wave && blank < v_wave + 64 && (((blank - v_wave) >> 2) & 1) == hf)
                                  ? blank - v_wave : -1;
#pragma unroll
        for (int nd = 0; nd < 4; ++nd) {
            float mx = acc[0][nd][0];
#pragma unroll
            for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc[mv][nd][r]);
            const float mn = fmaxf(m[nd], mx);
            if (mn > -INFINITY) {
                const float ms = mn * kLog2e;
                float sum = s[nd] * fast_exp2(fmaf(m[nd], kLog2e, -ms));  // m = -inf: s = 0 stays 0
#pragma unroll
                for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sum += fast_exp2(fmaf(acc[mv][nd][r], kLog2e, -ms));
                s[nd] = sum;
                m[nd] = mn;
            }
            // the label's logit, if it sits in this lane's half of this wave's part of the tile
            const int lv = lab[nd] - v_wave;
            const int key = (lab[nd] >= 0 && lv >= 0 && lv < 64 && ((lv >> 2) & 1) == hf) ? lv : -1;
            if (__ballot(key >= 0) != 0) {
#pragma unroll
                for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r) xl[nd] = key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : xl[nd];
            }
            if (__ballot(blank_key >= 0) != 0) {
#pragma unroll
                for (int mv = 0; mv < 2; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        xb[nd] = blank_key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : xb[nd];
            }
        }
    };
    for (int it = 0; it < iters; it += 2) {
        slice(it, pre[0], pre[1]);
        if (it + 1 < iters) slice(it + 1, pre[1], pre[0]);
    }

    // ---- merge: the two halves of a wave, then the two waves that share the data rows ----------
    float* s_merge = reinterpret_cast<float*>(&s_h[0][0][0]);  // the staging buffers are free now
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) {
        const float m2 = __shfl_xor(m[nd], 32), s2 = __shfl_xor(s[nd], 32);
        const float xl2 = __shfl_xor(xl[nd], 32), xb2 = __shfl_xor(xb[nd], 32);
        lse_merge(m[nd], s[nd], m2, s2);
        xl[nd] += xl2;  // exactly one of the halves (and of the waves) held the entry, the others 0
        xb[nd] += xb2;
        if (wv == 1 && hf == 0) {
            float* q = s_merge + ((wd * 4 + nd) * 32 + l32) * 4;
            q[0] = m[nd]; q[1] = s[nd]; q[2] = xl[nd]; q[3] = xb[nd];
        }
    }
    __syncthreads();
    if (wv != 0 || hf != 0) return;
#pragma unroll
    for (int nd = 0; nd < 4; ++nd) {
        const i64 r = row0 + 128 * wd + 32 * nd + l32;
        if (r >= R) continue;
        const float* q = s_merge + ((wd * 4 + nd) * 32 + l32) * 4;
        lse_merge(m[nd], s[nd], q[0], q[1]);
        const Lse lse = {m[nd], log2_of_sum(s[nd])};
        lse_out[r] = lse.value();
        const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
        const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
        rowinfo[r] = make_int2(lab[nd] < 0 ? -1 : lab[nd], ri.n);
        if (pad >= 0)
            lp[pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1)] =
                make_lp(xb[nd] + q[3], xl[nd] + q[2], lse, lab[nd], seqmode + ri.n);
        else if (grads_skipped) grads_skipped[r] = make_float2(0.f, 0.f);
    }
}

// ---------------------------------------------------------------------------------------------
// forward, data rows resident in registers
// ---------------------------------------------------------------------------------------------
// The streaming kernel above reads its h tile once per vocabulary tile: V / 128 times in all, from
// HBM, since the tiles of all resident workgroups together exceed the L2 (measured on N=32, V=1024,
// H=512: 3.3 GB fetched for 0.32 GB of h, and the kernel runs at the speed of that traffic).  Here
// every wave keeps the MFMA operand fragments of its OWN 32 ND data rows in registers for the whole
// kernel (ND * H / 16 registers of 16 bytes per lane: the whole K range), so h is read exactly once;
// only the weight tile travels through LDS, in K-slices of 64, and every wave multiplies its rows
// with the whole tile of 128 vocabulary entries.  Needs H known at compile time (the fragments are
// indexed statically).
constexpr int kRK = 64;      // K-slice of the weight tile
constexpr int kRPitch = 72;  // 144 bytes: 16 consecutive rows start in 16 different groups of four banks

template <typename T, int ND, int KS /* H / 16 */, int OCC, bool D2>
__global__ __launch_bounds__(256, OCC) void k_joint_fwd_res(
    const T* __restrict__ h, const T* __restrict__ W, const float* __restrict__ bias, i64 R, int V,
    const int* __restrict__ lx, const int* __restrict__ ly, const int* __restrict__ y, i64 y_stride, i64 y_len,
    const i64* __restrict__ row_off, const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N,
    int blank, LpCell* __restrict__ lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    constexpr int H = KS * 16;
    constexpr int NK = H / kRK;  // K-slices per vocabulary tile
    static_assert(H % kRK == 0, "whole K-slices");
    __shared__ __attribute__((aligned(16))) T s_w[2][kJN][kRPitch];
    __shared__ __attribute__((aligned(16))) float s_bias[2][kJN];  // what the accumulators of a tile start from

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hf = lane >> 5, l32 = lane & 31;
    const i64 row0 = (i64)blockIdx.x * (128 * ND) + (i64)w * (32 * ND);  // first data row of this wave
    const i64 last_row = R - 1;

    // ---- this wave's data rows, as MFMA operand fragments, for good ----------
    v4i hreg[ND][KS];
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        i64 r = row0 + 32 * nd + l32;
        r = r < last_row ? r : last_row;  // rows beyond the tensor are multiplied like the last one and dropped
        const T* src = h + r * (i64)H + 8 * hf;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) hreg[nd][ks] = *reinterpret_cast<const v4i*>(src + 16 * ks);
    }
    int lab[ND];
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        const i64 r = row0 + 32 * nd + l32;
        lab[nd] = kNoLabel;
        if (r < R) {
            const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
            if (ri.n >= 0 && pad_off[ri.n] >= 0) lab[nd] = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        }
    }

    // ---- weight tile: thread t moves 16-byte piece (t % 8) of rows t / 8 + 32 p, p = 0..3 ----------
    const int st_row = tid >> 3, st_piece = tid & 7;
    struct Pre { v4i w[4]; };
    Pre pre[D2 ? 2 : 1];
    const int nvt = (V + kJN - 1) / kJN;
    auto fetch = [&](int vt, int kc, Pre& q) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            int v = vt * kJN + st_row + 32 * p;
            if (v >= V) v = V - 1;  // entries beyond the vocabulary are masked in the accumulator
            q.w[p] = *reinterpret_cast<const v4i*>(W + (i64)v * H + kc * kRK + st_piece * 8);
        }
    };
    auto stage = [&](int buf, const Pre& q) {
#pragma unroll
        for (int p = 0; p < 4; ++p) *reinterpret_cast<v4i*>(&s_w[buf][st_row + 32 * p][st_piece * 8]) = q.w[p];
    };

    float m[ND], s[ND], xl[ND], xb[ND];
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) { m[nd] = -INFINITY; s[nd] = 0.f; xl[nd] = 0.f; xb[nd] = 0.f; }

    // slices are numbered it = vt * NK + kc; slice it is multiplied out of buffer it & 1 (NK is even
    // or the parity is carried), its loads were issued two slices earlier
    // the bias of a tile (-inf beyond the vocabulary, which no finite product changes and which drops
    // out of both the maximum and the sum) is fetched by the first 128 threads one tile ahead
    auto bias_of = [&](int vt) {
        const int v = vt * kJN + tid;
        return v < V ? (bias ? bias[v] : 0.f) : -INFINITY;
    };
    float bias_next = 0.f;
    if (tid < kJN) s_bias[0][tid] = bias_of(0);
    fetch(0, 0, pre[0]);
    if (D2 && (NK > 1 || nvt > 1)) fetch(NK > 1 ? 0 : 1, NK > 1 ? 1 : 0, pre[1]);
    stage(0, pre[0]);
    __syncthreads();

    f32x16 acc[4][ND];
    int par = 0;  // buffer of the current slice
    for (int vt = 0; vt < nvt; ++vt) {
        const int v0 = vt * kJN;
#pragma unroll
        for (int mv = 0; mv < 4; ++mv)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                const float4 bq = *reinterpret_cast<const float4*>(&s_bias[vt & 1][32 * mv + 8 * b4 + 4 * hf]);
#pragma unroll
                for (int nd = 0; nd < ND; ++nd) {
                    acc[mv][nd][4 * b4 + 0] = bq.x; acc[mv][nd][4 * b4 + 1] = bq.y;
                    acc[mv][nd][4 * b4 + 2] = bq.z; acc[mv][nd][4 * b4 + 3] = bq.w;
                }
            }
        if (tid < kJN && vt + 1 < nvt) bias_next = bias_of(vt + 1);
#pragma unroll
        for (int kc = 0; kc < NK; ++kc) {
            if (kc == NK - 1 && tid < kJN && vt + 1 < nvt) s_bias[(vt + 1) & 1][tid] = bias_next;  // before its barrier
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
            for (int ks = 0; ks < kRK / 16; ++ks) {
                v4i fa[4];
#pragma unroll
                for (int mv = 0; mv < 4; ++mv)
                    fa[mv] = *reinterpret_cast<const v4i*>(&s_w[par][32 * mv + l32][16 * ks + 8 * hf]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mv = 0; mv < 4; ++mv)
#pragma unroll
                    for (int nd = 0; nd < ND; ++nd)
                        acc[mv][nd] = Mfma<T>::mac(fa[mv], hreg[nd][kc * (kRK / 16) + ks], acc[mv][nd]);
                __builtin_amdgcn_sched_barrier(0);
            }
            {
                const int k1 = kc + 1;
                const int vt1 = vt + k1 / NK;
                if (vt1 < nvt) stage(par ^ 1, pre[D2 ? (kc + 1 + (NK & 1) * vt) & 1 : 0]);
            }
            __syncthreads();
            par ^= 1;
        }

        // ---- fold the tile's logits into the rows' running state ----------
        const int blank_key = (blank >= v0 && blank < v0 + kJN && (((blank - v0) >> 2) & 1) == hf) ? blank - v0 : -1;
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) {
            float mx = acc[0][nd][0];
#pragma unroll
            for (int mv = 0; mv < 4; ++mv)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc[mv][nd][r]);
            const float mn = fmaxf(m[nd], mx);
            if (mn > -INFINITY) {
                const float ms = mn * kLog2e;
                float sum = s[nd] * fast_exp2(fmaf(m[nd], kLog2e, -ms));  // m = -inf: s = 0 stays 0
#pragma unroll
                for (int mv = 0; mv < 4; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sum += fast_exp2(fmaf(acc[mv][nd][r], kLog2e, -ms));
                s[nd] = sum;
                m[nd] = mn;
            }
            const int lv = lab[nd] - v0;
            const int key = (lab[nd] >= 0 && lv >= 0 && lv < kJN && ((lv >> 2) & 1) == hf) ? lv : -1;
            if (__ballot(key >= 0) != 0) {
#pragma unroll
                for (int mv = 0; mv < 4; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r) xl[nd] = key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : xl[nd];
            }
            if (__ballot(blank_key >= 0) != 0) {
#pragma unroll
                for (int mv = 0; mv < 4; ++mv)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        xb[nd] = blank_key == 32 * mv + acc_row(r, hf) ? acc[mv][nd][r] : xb[nd];
            }
        }
    }

    // ---- the two halves of the wave hold disjoint vocabulary entries of the same rows ----------
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) {
        lse_merge(m[nd], s[nd], __shfl_xor(m[nd], 32), __shfl_xor(s[nd], 32));
        xl[nd] += __shfl_xor(xl[nd], 32);  // exactly one half held the entry, the other 0
        xb[nd] += __shfl_xor(xb[nd], 32);
        const i64 r = row0 + 32 * nd + l32;
        if (hf != 0 || r >= R) continue;
        const Lse lse = {m[nd], log2_of_sum(s[nd])};
        lse_out[r] = lse.value();
        const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
        const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
        rowinfo[r] = make_int2(lab[nd] < 0 ? -1 : lab[nd], ri.n);
        if (pad >= 0)
            lp[pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1)] = make_lp(xb[nd], xl[nd], lse, lab[nd], seqmode + ri.n);
        else if (grads_skipped) grads_skipped[r] = make_float2(0.f, 0.f);
    }
}

template <typename T>
static int joint_gather_typed(const Batch& b, const Workspace& ws, const JointOperands& j, float* lse, int* rowinfo,
                              float* grads) {
    int2* ri = reinterpret_cast<int2*>(rowinfo);
    float2* gz = reinterpret_cast<float2*>(grads);
    const T* h = static_cast<const T*>(j.h);
    const T* w = static_cast<const T*>(j.w);
#define CWR_JOINT_RES(ND, KS, OCC, D2)                                                                              \
    if (j.H == 16 * KS) {                                                                                       \
        const i64 blocks = (b.R + 128 * ND - 1) / (128 * ND);                                                   \
        if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;                                                    \
        CWR_LAUNCH((k_joint_fwd_res<T, ND, KS, OCC, D2>), dim3((unsigned)blocks), dim3(256), 0, b.stream, h, w, j.bias,  \
                   b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N,       \
                   b.blank, ws.lp, lse, ri, gz, ws.seqmode, b.status);                                          \
        return check_launch();                                                                                  \
    }
    // the joint sizes in use; any other multiple of 32 takes the streaming kernel
    // measured on R = 311449, V = 1024, H = 512 (bf16): one data block per wave at two waves per SIMD
    // 0.46 ms; two blocks per wave at one wave per SIMD 0.63 ms (registers spill); streaming kernel 0.63 ms
    CWR_JOINT_RES(2, 16, 1, true) CWR_JOINT_RES(2, 24, 1, true) CWR_JOINT_RES(1, 32, 2, false)
    CWR_JOINT_RES(1, 40, 1, true) CWR_JOINT_RES(1, 48, 1, true) CWR_JOINT_RES(1, 64, 1, true)
#undef CWR_JOINT_RES
    const i64 blocks = (b.R + kJM - 1) / kJM;
    if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
    CWR_LAUNCH((k_joint_fwd<T>), dim3((unsigned)blocks), dim3(256), 0, b.stream, h, w, j.bias, b.R, (int)j.H, b.V,
               b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, ws.lp, lse, ri, gz,
               ws.seqmode, b.status);
    return check_launch();
}

int launch_joint_gather(const Batch& b, const Workspace& ws, const JointOperands& j, float* lse, int* rowinfo,
                        float* grads) {
    if (b.R == 0) return CWR_OK;
    if (b.dtype == CWR_BF16) return joint_gather_typed<bf16_t>(b, ws, j, lse, rowinfo, grads);
    if (b.dtype == CWR_F16) return joint_gather_typed<__half>(b, ws, j, lse, rowinfo, grads);
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
