// Device-side helpers shared by the kernels: wave64 cross-lane primitives (DPP), element packs
// for 128-bit global accesses, and the index arithmetic of the compact and anti-diagonal layouts.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/cwarp_rnnt_hip.h"

namespace cwr {

typedef long long i64;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// "no path" marker of the lattice recursions.  Finite, so that marker - marker = 0 instead of NaN.
constexpr double kNeg = -1.0e30;
constexpr float kLpFloor = -1.0e30f;  // gathered log-probs are clamped to this (keeps -inf logits finite)
// The scaled linear-domain walk renormalises every kPF = 16 steps to a maximum of 2^kLinTarget
// per lane.  A step multiplies a value by at most two factors (a lane walks two columns), each
// within [2^kLinMin, 2^kLinMax], and adds at most doubles it: inside a block the largest value
// stays below 2^(kLinTarget + 2*16*(kLinMax+1)) = 2^964, and the walk's own range check (every
// second step) catches values that shrink towards the bottom of the fp64 range.
constexpr float kLinMin = -100.0f;  // base-2 log-probs below this ...
constexpr float kLinMax = 1.0f;     // ... or above this send the sequence to the log-domain walk
constexpr int kLinTarget = 900;

// ---------------------------------------------------------------------------------------------
// wave64 cross-lane moves.  gfx9-family DPP controls.
// ---------------------------------------------------------------------------------------------
constexpr int DPP_QUAD_XOR1 = 0xB1;    // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;    // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_SHL = 0x100;     // + n: lane i reads lane i+n of its row of 16
constexpr int DPP_ROW_SHR = 0x110;     // + n: lane i reads lane i-n of its row of 16
constexpr int DPP_WAVE_SHL1 = 0x130;   // lane i reads lane i+1
constexpr int DPP_WAVE_SHR1 = 0x138;   // lane i reads lane i-1
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

// Lanes without a valid source (or masked off by ROW_MASK) return `old`.
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float old, float src) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src),
                                                      CTRL, ROW_MASK, BANK_MASK, false));
}
// Lanes without a valid source return 0 (no register has to be cleared first).
template <int CTRL>
__device__ __forceinline__ float dpp_f32_or_zero(float src) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(src), CTRL, 0xF, 0xF, true));
}
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ int dpp_i32(int old, int src) {
    return __builtin_amdgcn_update_dpp(old, src, CTRL, ROW_MASK, BANK_MASK, false);
}
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ i64 dpp_i64(i64 old, i64 src) {
    int lo = dpp_i32<CTRL, ROW_MASK, BANK_MASK>((int)(old & 0xffffffffLL), (int)(src & 0xffffffffLL));
    int hi = dpp_i32<CTRL, ROW_MASK, BANK_MASK>((int)(old >> 32), (int)(src >> 32));
    return ((i64)hi << 32) | (i64)(unsigned)lo;
}

template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ double dpp_f64(double old, double src) {
    int lo = dpp_i32<CTRL, ROW_MASK, BANK_MASK>(__double2loint(old), __double2loint(src));
    int hi = dpp_i32<CTRL, ROW_MASK, BANK_MASK>(__double2hiint(old), __double2hiint(src));
    return __hiloint2double(hi, lo);
}

__device__ __forceinline__ double readlane_f64(double v, int lane) {
    int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}

__device__ __forceinline__ float readlane_f32(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

struct OpMax {
    static __device__ __forceinline__ float identity() { return -INFINITY; }
    static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};
struct OpSum {
    static __device__ __forceinline__ float identity() { return 0.0f; }
    static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};

// All-reduce over aligned groups of W consecutive lanes (W a power of two, 1..64): every lane of
// a group ends up with the group's result.
template <int W, class Op>
__device__ __forceinline__ float group_allreduce(float v) {
    if (W >= 2) v = Op::apply(v, dpp_f32<DPP_QUAD_XOR1>(v, v));
    if (W >= 4) v = Op::apply(v, dpp_f32<DPP_QUAD_XOR2>(v, v));
    if (W >= 8) v = Op::apply(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v, v));
    if (W >= 16) v = Op::apply(v, dpp_f32<DPP_ROW_MIRROR>(v, v));
    if (W == 32) v = Op::apply(v, __shfl_xor(v, 16));
    if (W == 64) {
        // rows 1,3 += row 0,2 ; rows 2,3 += lane 31 ; lane 63 then holds the total
        v = Op::apply(v, dpp_f32<DPP_ROW_BCAST15, 0xA>(Op::identity(), v));
        v = Op::apply(v, dpp_f32<DPP_ROW_BCAST31, 0xC>(Op::identity(), v));
        v = readlane_f32(v, 63);
    }
    return v;
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ i64 wave_inclusive_scan(i64 v) {
    v += dpp_i64<DPP_ROW_SHR + 1>(0, v);
    v += dpp_i64<DPP_ROW_SHR + 2>(0, v);
    v += dpp_i64<DPP_ROW_SHR + 4>(0, v);
    v += dpp_i64<DPP_ROW_SHR + 8>(0, v);
    v += dpp_i64<DPP_ROW_BCAST15, 0xA>(0, v);
    v += dpp_i64<DPP_ROW_BCAST31, 0xC>(0, v);
    return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---------------------------------------------------------------------------------------------
// element packs: VEC consecutive elements moved with one 16-byte access, computed on as fp32
// ---------------------------------------------------------------------------------------------
struct bf16_t { uint16_t v; };

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <> struct Elem<__half> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_f32(__half v) { return __half2float(v); }
    static __device__ __forceinline__ __half from_f32(float v) { return __float2half_rn(v); }
};
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.v << 16); }
    static __device__ __forceinline__ bf16_t from_f32(float f) {
        const __bf16 h = (__bf16)f;  // gfx950's conversion instruction: round to nearest even, NaN kept
        bf16_t r;
        __builtin_memcpy(&r.v, &h, 2);
        return r;
    }
};
template <> struct Elem<double> {
    static constexpr int VEC = 2;
    static __device__ __forceinline__ float to_f32(double v) { return (float)v; }
    static __device__ __forceinline__ double from_f32(float v) { return (double)v; }
};

// 16-byte store of data that nothing on the GPU reads again soon: non-temporal AND system scope.
// The compiler's non-temporal store sets only the first of the two; with both the (R,V) gradient
// stream runs about 3 % faster on MI355X (395 -> 383 us for 1.28 GB read + 1.28 GB written).
typedef int v4i_store_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_streaming_16(void* p, v4i_store_t v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
}

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) PackT { T e[VEC]; };

// ---------------------------------------------------------------------------------------------
// layouts
// ---------------------------------------------------------------------------------------------
// Lattice storage (log-probs, alpha, beta).  A sequence's T x (U+1) lattice is cut into strips
// of kStripCols = 128 label positions; strip s holds nl = min(128, U+1-128s) columns, two per lane
// of the wave that walks it (lane j: columns 2j and 2j+1 of the strip).  Inside a strip, cell
// (t, u = 128s+c) is stored at row t + c/2 + kRowShift, column c, of a dense
// (T + ceil(nl/2) - 1 + 2*kRowShift) x pitch array, pitch = nl rounded up to even: a wave that
// walks the strip with lane j one frame behind lane j-1 touches one contiguous row per step, at a
// constant pitch, and every lane's pair of columns is one aligned 16-byte access (a strip of odd
// width has a column of padding for its last lane's second column).  The rows above and below, and
// the two triangles of slots that hold no cell, are padding too.
constexpr int kPF = 16;               // prefetch depth of the lattice walk, in rows
constexpr int kRowShift = 2 * kPF;    // padding rows in front of (and behind) a strip
constexpr int kBndPad = 192;          // entries a boundary stream holds beyond T
constexpr int kStripCols = 128;       // label positions per strip
constexpr int kStripShift = 7;        // log2(kStripCols)

__host__ __device__ __forceinline__ i64 strip_lanes(i64 nl) { return (nl + 1) >> 1; }
__host__ __device__ __forceinline__ i64 strip_pitch(i64 nl) { return (nl + 1) & ~(i64)1; }
__host__ __device__ __forceinline__ i64 strip_rows(i64 T, i64 nl) { return T + strip_lanes(nl) - 1 + 2 * kRowShift; }
__host__ __device__ __forceinline__ i64 strip_count(i64 Up) { return (Up + kStripCols - 1) >> kStripShift; }
__host__ __device__ __forceinline__ i64 lattice_slots(i64 T, i64 Up) {
    i64 full = (Up - 1) >> kStripShift;  // strips before the last one are full
    i64 nl = Up - (full << kStripShift);
    // always an even number of slots: every strip starts on a 16-byte boundary of the fp64 arrays
    return full * strip_rows(T, kStripCols) * kStripCols + strip_rows(T, nl) * strip_pitch(nl);
}
__host__ __device__ __forceinline__ i64 lattice_slot(i64 t, i64 u, i64 T, i64 Up) {
    i64 s = u >> kStripShift, c = u & (kStripCols - 1);
    i64 nl = Up - (s << kStripShift) < kStripCols ? Up - (s << kStripShift) : kStripCols;
    return s * strip_rows(T, kStripCols) * kStripCols + (t + (c >> 1) + kRowShift) * strip_pitch(nl) + c;
}
__host__ __device__ __forceinline__ i64 boundary_entries(i64 T, i64 Up) {
    return ((Up - 1) >> kStripShift) * (T + kBndPad);
}

// What the gather pass leaves per lattice cell: two 8-byte records in two arrays of the strip
// layout, the probabilities for the linear-domain walk and the logarithms for the log-domain walk
// and the gradient fill.  Kept apart so that a lane of the lattice walk fetches what it needs of its
// two columns with one 16-byte load, and a strip row of the walk touches no byte it does not use:
// the walks are bound by what their memory instructions move through the CU's vector memory path
// as much as by their arithmetic (widening the probabilities to fp64 in this pass, which saves the
// walk four conversions a step and costs it one more 16-byte load, made every walk slower).
struct LpCell {
    float p_blank;  // 2^l_blank
    float p_label;  // 2^l_label
    float l_blank;  // log2 P(blank | t,u)
    float l_label;  // log2 P(y[u] | t,u); 0 in the last column
};
struct LpStore {
    float2* p;  // slot_cap  (P(blank), P(label))
    float2* l;  // slot_cap  (log2 P(blank), log2 P(label))
    struct Ref {
        float2* p;
        float2* l;
        __device__ __forceinline__ void operator=(const LpCell& c) const {
            *p = make_float2(c.p_blank, c.p_label);
            *l = make_float2(c.l_blank, c.l_label);
        }
    };
    __device__ __forceinline__ Ref operator[](i64 i) const { return Ref{p + i, l + i}; }
};

// Cost of a sequence from its two likelihoods, both as base-2 logarithms: fwd = alpha at the last
// cell plus that cell's blank, bwd = beta[0][0].  cwarp_cuda_rnnt_kernel.cu:353-366: cost = -bwd,
// unless the two differ by more than 0.1 % of the larger, in which case the reference prints a
// warning and takes their mean; here the caller raises CWR_FLAG_FB_MISMATCH instead (returns true).
// One deviation: the rule only fires when the two also differ by more than 1e-5 (in bits).  The
// reference's rule is purely relative, and a likelihood within rounding of 1 (both logarithms of
// the order of 1e-7) has no meaningful relative difference.
__host__ __device__ inline bool cost_rule(double fwd_log2, double bwd_log2, float* cost) {
    double fb = bwd_log2;
    const double diff = fwd_log2 > fb ? fwd_log2 - fb : fb - fwd_log2;
    const double larger = fwd_log2 > fb ? fwd_log2 : fb;
    const double ratio = diff / (larger < 0 ? -larger : larger);
    const bool mismatch = ratio > 1e-3 && diff > 1e-5;
    if (mismatch) fb = (fwd_log2 + fb) * 0.5;
    *cost = (float)(-fb * 0.6931471805599453);
    return mismatch;
}

// Which sequence owns compact row r, and where in its lattice the row sits.
struct RowInfo {
    int n;    // -1: the row belongs to no usable sequence
    int t, u;
    int T, U;
    i64 off;  // row_off[n]
};

// Where row r sits inside sequence n.
__device__ __forceinline__ RowInfo place_row(i64 r, int n, i64 R, const i64* __restrict__ row_off,
                                             const int* __restrict__ lx, const int* __restrict__ ly) {
    RowInfo ri;
    ri.n = -1; ri.t = 0; ri.u = 0; ri.T = 0; ri.U = 0; ri.off = 0;
    const i64 off = row_off[n];
    const int T = lx[n], U = ly[n];
    if (T <= 0 || U < 0) return ri;
    const i64 cells = (i64)T * (i64)(U + 1);
    const i64 rem = r - off;
    if (rem < 0 || rem >= cells || off + cells > R) return ri;
    ri.n = n; ri.T = T; ri.U = U; ri.off = off;
    if (cells < 0x7fffffffLL) {
        unsigned q = (unsigned)rem / (unsigned)(U + 1);
        ri.t = (int)q;
        ri.u = (int)((unsigned)rem - q * (unsigned)(U + 1));
    } else {
        ri.t = (int)(rem / (U + 1));
        ri.u = (int)(rem - (i64)ri.t * (U + 1));
    }
    return ri;
}

__device__ __forceinline__ RowInfo decode_row(i64 r, i64 R, const i64* __restrict__ row_off,
                                              const int* __restrict__ lx, const int* __restrict__ ly,
                                              int N) {
    if (N <= 0) {
        RowInfo ri;
        ri.n = -1; ri.t = 0; ri.u = 0; ri.T = 0; ri.U = 0; ri.off = 0;
        return ri;
    }
    int lo = 0, hi = N - 1;
    while (lo < hi) {  // last n with row_off[n] <= r (skips empty sequences)
        int mid = (lo + hi + 1) >> 1;
        if (row_off[mid] <= r) lo = mid; else hi = mid - 1;
    }
    return place_row(r, lo, R, row_off, lx, ly);
}

// Sets a bit of the status word.  A problem in the data usually shows in many rows at once: looking
// first keeps them from queueing on one address (a batch whose labels all lie outside the
// vocabulary took 2.5 ms instead of 0.2 in the gather pass).
__device__ __forceinline__ void raise_flag(int* status, int bit) {
    if ((__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & bit) == 0) atomicOr(status, bit);
}

// What a row's label slot can hold besides a label: nothing (the last column of a lattice emits no
// label), or a label that does not exist (outside [0, V) or beyond the label array).  A bad label
// poisons its sequence: the cost becomes NaN (bit kSeqPoisoned of the sequence's walk-mode word).
constexpr int kNoLabel = -1;
constexpr int kBadLabel = -2;
constexpr int kSeqLogDomain = 1;  // walk-mode bits; 2 and 4 belong to the lattice kernel
constexpr int kSeqPoisoned = 8;

__device__ __forceinline__ int fetch_label(const RowInfo& ri, const int* __restrict__ y, i64 y_stride,
                                           i64 y_len, const i64* __restrict__ lab_off, int V,
                                           int* status) {
    if (ri.n < 0 || ri.u >= ri.U) return kNoLabel;
    i64 at = (y_stride >= 0 ? (i64)ri.n * y_stride : lab_off[ri.n]) + ri.u;
    int lab = (at >= 0 && at < y_len && (y_stride < 0 || ri.u < y_stride)) ? y[at] : -1;
    if (lab < 0 || lab >= V) {
        if (status) raise_flag(status, CWR_FLAG_BAD_LABEL);
        return kBadLabel;
    }
    return lab;
}

// What the lattice walk consumes, two 8-byte records per cell (see LpCell, LpStore): the (blank, label)
// log-probabilities as base-2 logarithms, floored so that -inf logits stay finite, and the same
// two as plain probabilities for the scaled linear-domain walk.  A logarithm outside
// [kLinMin, kLinMax] cannot be carried by that walk within one of its blocks (nor, as a
// probability, by fp32); the sequence is then marked for the log-domain walk.
// A row's log-sum-exp as (maximum m, log2 of the sum of exp(x - m)).  Kept in two parts for the
// cell records: x - m is exact and log2(sum) is small when a row is peaked, so that a
// log-probability close to zero keeps its absolute accuracy however large the logits are (one
// fp32 number m + ln(sum) would carry half an ulp of m into every log-probability).
struct Lse {
    float m, l2s;
    __device__ __forceinline__ float value() const { return fmaf(l2s, kLn2, m); }
};
// log2 of a sum s >= 1 of exponentials whose largest term is 1, and 2^b for a log-probability b:
// series next to s = 1 and b = 0, where the hardware approximations are good to an ulp of their
// RESULT's neighbourhood (about 1e-7 absolute) but a peaked row needs the small difference itself.
__device__ __forceinline__ float log2_of_sum(float s) {
    const float d = s - 1.f;  // exact for s in [1, 2]
    const float series = d * fmaf(d, fmaf(d, 1.f / 3.f, -0.5f), 1.f) * kLog2e;
    return d < 0.015625f ? series : fast_log2(s);
}
__device__ __forceinline__ float exp2_of_logprob(float b) {
    const float z = b * kLn2;
    const float series = fmaf(z, fmaf(z, fmaf(z, 1.f / 6.f, 0.5f), 1.f), 1.f);
    return b > -0.015625f ? series : fast_exp2(b);
}

// lab: the row's label, kNoLabel or kBadLabel.  The walk-mode word is looked at before it is set: a
// batch of steep logits marks its sequences from most rows at once, and unconditional atomics on one
// address per sequence would queue.
__device__ __forceinline__ LpCell make_lp(float xb, float xl, const Lse lse, int lab, int* seqmode_n) {
    const float b = (float)(((double)fmaxf(xb, kLpFloor) - (double)lse.m) * 1.4426950408889634 - (double)lse.l2s);
    const float l = lab >= 0
        ? (float)(((double)fmaxf(xl, kLpFloor) - (double)lse.m) * 1.4426950408889634 - (double)lse.l2s) : 0.f;
    if (!(b >= kLinMin && b <= kLinMax && l >= kLinMin && l <= kLinMax)) raise_flag(seqmode_n, kSeqLogDomain);
    if (lab == kBadLabel) raise_flag(seqmode_n, kSeqPoisoned);
    LpCell c;
    c.p_blank = exp2_of_logprob(b);
    c.p_label = exp2_of_logprob(l);
    c.l_blank = b;
    c.l_label = l;
    return c;
}

}  // namespace cwr
