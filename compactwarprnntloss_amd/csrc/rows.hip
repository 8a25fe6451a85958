// The two passes that stream the (R,V) tensors: the gather pass (forward) and the gradient pass
// (backward).  These carry all the HBM traffic of the loss.
//
// Replaces, for gfx950 (wave64):
//   cwarp_cuda_gather_kernel.cu:19-43   gather_cuda_kernel        -> k_gather_*
//   cwarp_cuda_gather_kernel.cu:52-74   scatter_grad_cuda_kernel  \
//   cwarp_cuda.cpp:134 (zeros(R,V))                                > k_grad_*
//   cwarp_cuda_rnnt_kernel.cu:512-521   cwarp_cuda_backward_      /
//
// Work split: waves are short-lived.  A wave handles one pass -- 64/LPR rows, LPR lanes per row,
// K 16-byte packs per lane -- issues all its loads first, works out the rows' scalars while they
// are in flight, and retires.  Workgroups are dispatched in address order, so at any moment the
// machine streams one compact window of the tensor; measured on MI355X this sustains 6.2-7.0 TB/s
// where waves that loop over many rows stay near 5.1 TB/s.
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

constexpr int kWavesPerBlock = 4;

typedef int v4i __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ v4i load_raw(const void* p) {
    const v4i* q = static_cast<const v4i*>(p);
    return NT ? __builtin_nontemporal_load(q) : *q;
}
template <bool NT>
__device__ __forceinline__ void store_raw(void* p, v4i v) {
    v4i* q = static_cast<v4i*>(p);
    if (NT) store_streaming_16(q, v); else *q = v;
}

// 16-byte pack <-> VEC fp32 values
template <typename T> struct Pack;
template <> struct Pack<float> {
    static __device__ __forceinline__ void unpack(v4i r, float (&o)[4]) {
        o[0] = __int_as_float(r.x); o[1] = __int_as_float(r.y); o[2] = __int_as_float(r.z); o[3] = __int_as_float(r.w);
    }
    static __device__ __forceinline__ v4i pack(const float (&i)[4]) {
        v4i r = {__float_as_int(i[0]), __float_as_int(i[1]), __float_as_int(i[2]), __float_as_int(i[3])};
        return r;
    }
    static __device__ __forceinline__ v4i neg_inf() {
        v4i r = {(int)0xff800000, (int)0xff800000, (int)0xff800000, (int)0xff800000};
        return r;
    }
};
template <> struct Pack<__half> {
    static __device__ __forceinline__ void unpack(v4i r, float (&o)[8]) {
        const int w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            __half2 h = *reinterpret_cast<const __half2*>(&w[j]);
            float2 f = __half22float2(h);
            o[2 * j] = f.x; o[2 * j + 1] = f.y;
        }
    }
    static __device__ __forceinline__ v4i pack(const float (&i)[8]) {
        int w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            __half2 h = __floats2half2_rn(i[2 * j], i[2 * j + 1]);
            w[j] = *reinterpret_cast<const int*>(&h);
        }
        v4i r = {w[0], w[1], w[2], w[3]};
        return r;
    }
    static __device__ __forceinline__ v4i neg_inf() {
        v4i r = {(int)0xfc00fc00, (int)0xfc00fc00, (int)0xfc00fc00, (int)0xfc00fc00};
        return r;
    }
};
template <> struct Pack<bf16_t> {
    static __device__ __forceinline__ void unpack(v4i r, float (&o)[8]) {
        const int w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[2 * j] = __int_as_float(w[j] << 16);
            o[2 * j + 1] = __int_as_float(w[j] & (int)0xffff0000);
        }
    }
    static __device__ __forceinline__ v4i pack(const float (&i)[8]) {
        int w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            unsigned lo = Elem<bf16_t>::from_f32(i[2 * j]).v, hi = Elem<bf16_t>::from_f32(i[2 * j + 1]).v;
            w[j] = (int)(lo | (hi << 16));
        }
        v4i r = {w[0], w[1], w[2], w[3]};
        return r;
    }
    static __device__ __forceinline__ v4i neg_inf() {
        v4i r = {(int)0xff80ff80, (int)0xff80ff80, (int)0xff80ff80, (int)0xff80ff80};
        return r;
    }
};
template <> struct Pack<double> {
    static __device__ __forceinline__ void unpack(v4i r, float (&o)[2]) {
        o[0] = (float)__hiloint2double(r.y, r.x);
        o[1] = (float)__hiloint2double(r.w, r.z);
    }
    static __device__ __forceinline__ v4i pack(const float (&i)[2]) {
        double a = (double)i[0], b = (double)i[1];
        v4i r = {__double2loint(a), __double2hiint(a), __double2loint(b), __double2hiint(b)};
        return r;
    }
    static __device__ __forceinline__ v4i neg_inf() {
        v4i r = {0, (int)0xfff00000, 0, (int)0xfff00000};
        return r;
    }
};

// position of column `col` inside a row that LPR lanes hold as K packs of VEC
template <int VEC, int LPR>
struct ColPos {
    int k, lane, c;
    __device__ __forceinline__ explicit ColPos(int col) {
        int pack = col / VEC;
        c = col - pack * VEC;
        k = pack / LPR;
        lane = pack - k * LPR;
    }
};

// ---------------------------------------------------------------------------------------------
// gather, fused log-softmax: lse[r], lp[cell] = (x[r,blank]-lse, x[r,label]-lse)
// ---------------------------------------------------------------------------------------------
// A row held by a lane group as K packs = K*VEC fp32 values in one register vector, so that an
// entry at a wave-uniform position can be read or written with indexed register access
// (s_set_gpr_idx) instead of a chain of selects.
template <int N> struct RegVec { typedef float type __attribute__((ext_vector_type(N))); };

// value of row scalar `v` held by lane `i`; i is wave-uniform when a wave works on one row at a time
template <int LPR> __device__ __forceinline__ int lane_get(int v, int i) {
    return LPR == 64 ? __builtin_amdgcn_readlane(v, i) : __shfl(v, i);
}
template <int LPR> __device__ __forceinline__ float lane_get(float v, int i) {
    return __int_as_float(lane_get<LPR>(__float_as_int(v), i));
}

// One pass: the LPR lanes of a group hold one row as K packs; all lanes of the group return the
// row's log-sum-exp and its blank / label entries.
template <typename T, int LPR, int K, bool EXTRACT = true>
__device__ __forceinline__ void gather_pass(const v4i (&raw)[K], const int g, const ColPos<Elem<T>::VEC, LPR>& pb,
                                            const int lab, Lse& lse, float& xb, float& xl) {
    constexpr int VEC = Elem<T>::VEC;
    typename RegVec<K * VEC>::type xv;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float t[VEC];
        Pack<T>::unpack(raw[k], t);
#pragma unroll
        for (int c = 0; c < VEC; ++c) xv[k * VEC + c] = t[c];
    }
    float m = xv[0];
#pragma unroll
    for (int j = 1; j < K * VEC; ++j) m = fmaxf(m, xv[j]);
    {
        m = group_allreduce<LPR, OpMax>(m);
        const float ms = m * kLog2e;
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < K * VEC; ++j) s += fast_exp2(fmaf(xv[j], kLog2e, -ms));
        s = group_allreduce<LPR, OpSum>(s);
        lse.m = m;
        // every exponent above is off by what ms lost to rounding (up to half an ulp of m log2 e,
        // 2e-6 for m = 25): the fma below recovers it exactly
        lse.l2s = log2_of_sum(s) - fmaf(m, kLog2e, -ms);
    }
    if (!EXTRACT) return;
    // pick the blank and label entries out of the registers
    const ColPos<VEC, LPR> pl(lab < 0 ? 0 : lab);
    float cb, cl;
    if (LPR == 64) {
        cb = xv[pb.k * VEC + pb.c];  // uniform positions
        cl = xv[pl.k * VEC + pl.c];
        xb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cb), pb.lane));
        xl = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cl), pl.lane));
    } else {
        // the blank sits in the same register and the same lane of every group: scalar reads
        cb = xv[pb.k * VEC + pb.c];
        xb = 0.f;
#pragma unroll
        for (int gg = 0; gg < 64 / LPR; ++gg) {
            const float v = readlane_f32(cb, gg * LPR + pb.lane);
            xb = gg == g ? v : xb;
        }
        if (K == 1) {  // the label's place differs between the groups: select, then one cross-lane read
            cl = xv[0];
#pragma unroll
            for (int c = 1; c < VEC; ++c) cl = c == pl.c ? xv[c] : cl;
            xl = __shfl(cl, g * LPR + pl.lane);
        } else {  // group by group, each with wave-uniform positions
            xl = 0.f;
#pragma unroll
            for (int gg = 0; gg < 64 / LPR; ++gg) {
                const int lab_g = __builtin_amdgcn_readlane(lab, gg * LPR);
                const ColPos<VEC, LPR> pg(lab_g < 0 ? 0 : lab_g);
                const float v = readlane_f32(xv[pg.k * VEC + pg.c], gg * LPR + pg.lane);
                xl = gg == g ? v : xl;
            }
        }
    }
}

// Workgroups are handed to the 8 XCDs round-robin.  With XCD_CONTIGUOUS the grid (a multiple of 8
// workgroups) is renumbered so that each XCD walks its own contiguous eighth of the rows: the
// small per-row outputs of neighbouring rows then meet in ONE L2 and leave it as full lines,
// instead of as eight partial lines from eight L2s.
template <bool XCD_CONTIGUOUS>
__device__ __forceinline__ i64 logical_block() {
    if (!XCD_CONTIGUOUS) return blockIdx.x;
    const unsigned per_xcd = gridDim.x >> 3;
    return (i64)(blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
}

// first row of this wave; wave-uniform by construction, and told so to the compiler so that the
// row decode of a one-row wave runs on the scalar unit
template <bool XCD_CONTIGUOUS = false>
__device__ __forceinline__ i64 wave_first_row(int rows_per_wave) {
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    return (logical_block<XCD_CONTIGUOUS>() * kWavesPerBlock + w) * rows_per_wave;
}

// Rows of at least 4 KiB (a whole wave per row, K >= 4 packs per lane): one row per wave.  The
// row is wave-uniform, so its decode runs on the scalar unit beside the vector work.
template <typename T, int K, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_row(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    constexpr int VEC = Elem<T>::VEC;
    // beyond 32 values per lane the register vector would be indexed through scratch memory:
    // the two entries are then read back from the row itself (it has just been fetched)
    constexpr bool kFromRegs = K * VEC <= 32;
    const int lane = threadIdx.x & 63;
    const i64 r = wave_first_row<true>(1);
    if (r >= R) return;
    const int NV = V / VEC;

    // loads first (a lane without a pack reads the row's first one and discards it) ...
    const T* row = x + r * (i64)V;
    v4i raw[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = lane + k * 64;
        raw[k] = load_raw<NT>(row + (i64)(j < NV ? j : 0) * VEC);
    }
    // ... then the row's place in the batch, while they are in flight
    int lab = -1;
    i64 dst = -1;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    if (pad >= 0) {
        lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
    }
    float xb = 0.f, xl = 0.f;
    if (!kFromRegs) {
        xb = Elem<T>::to_f32(row[blank]);
        xl = Elem<T>::to_f32(row[lab < 0 ? 0 : lab]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (lane + k * 64 >= NV) raw[k] = Pack<T>::neg_inf();
    const ColPos<VEC, 64> pb(blank);
    Lse lse;
    float rb, rl;
    gather_pass<T, 64, K, kFromRegs>(raw, 0, pb, lab, lse, rb, rl);
    if (kFromRegs) { xb = rb; xl = rl; }
    if (lane == 0) {
        lse_out[r] = lse.value();
        rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
        if (dst >= 0) lp[dst] = make_lp(xb, xl, lse, lab, seqmode + ri.n);
        else if (grads_skipped) grads_skipped[r] = make_float2(0.f, 0.f);
    }
}

// The per-sequence tables of a batch of at most 64 sequences, sequence l in lane l, so that a
// lane can look its row's sequence up with cross-lane reads instead of dependent memory loads.
struct SeqTables {
    i64 off, pad, lab;
    int T, U;
};

__device__ __forceinline__ i64 shfl_i64(i64 v, int src) {
    int lo = __shfl((int)(v & 0xffffffffLL), src), hi = __shfl((int)(v >> 32), src);
    return ((i64)hi << 32) | (i64)(unsigned)lo;
}

// Smaller rows: a wave takes NP passes of 64/LPR rows (4 to 8 KiB in all), issues every load up
// front, and decodes the rows meanwhile, one row per lane.
template <typename T, int LPR, int K, int NP, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_rows(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int RP = 64 / LPR;   // rows per pass
    constexpr int ROWS = RP * NP;  // rows per wave
    static_assert(ROWS <= 64 && K * VEC <= 32, "shape not meant for this kernel");
    const int lane = threadIdx.x & 63;
    const i64 r0 = wave_first_row<true>(ROWS);
    if (r0 >= R) return;
    const int NV = V / VEC;
    const int g = lane / LPR, lir = lane % LPR;

    v4i raw[NP][K];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const i64 r = r0 + p * RP + g;
        const T* row = x + (r < R ? r : r0) * (i64)V;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = lir + k * LPR;
            raw[p][k] = load_raw<NT>(row + (i64)(j < NV ? j : 0) * VEC);
        }
    }

    // Lane p of group g decodes the row that group g reduces in pass p, and keeps its results: no
    // value has to travel between lanes afterwards.
    static_assert(NP <= LPR && NP <= 16, "one lane of a group per pass");
    const i64 r = r0 + (i64)lir * RP + g;
    const bool mine = lir < NP && r < R;
    RowInfo ri;
    ri.n = -1; ri.t = 0; ri.u = 0; ri.T = 0; ri.U = 0; ri.off = 0;
    i64 pad = -1, labbase = 0;
    if (N <= 64) {
        SeqTables tb;
        tb.off = 0x7fffffffffffffffLL; tb.pad = -1; tb.lab = 0; tb.T = 0; tb.U = 0;
        if (lane < N) {
            tb.off = row_off[lane]; tb.pad = pad_off[lane]; tb.lab = lab_off[lane];
            tb.T = lx[lane]; tb.U = ly[lane];
        }
        const unsigned long long m = __ballot(tb.off <= r0);
        int n = m ? 63 - __clzll((long long)m) : 0;  // sequence of r0; later rows step over boundaries
        const i64 r_last = r0 + ROWS - 1;
        for (int j = n + 1; j < N; ++j) {
            const i64 oj = shfl_i64(tb.off, j);
            if (oj > r_last) break;
            n += (mine && oj <= r) ? 1 : 0;
        }
        const i64 off = shfl_i64(tb.off, n);
        pad = shfl_i64(tb.pad, n);
        labbase = shfl_i64(tb.lab, n);
        const int T_ = __shfl(tb.T, n), U_ = __shfl(tb.U, n);
        const i64 rem = r - off;
        if (mine && T_ > 0 && U_ >= 0 && rem >= 0 && rem < (i64)T_ * (U_ + 1)) {
            ri.n = n; ri.T = T_; ri.U = U_; ri.off = off;
            if ((i64)T_ * (U_ + 1) < 0x7fffffffLL) {
                const unsigned q = (unsigned)rem / (unsigned)(U_ + 1);
                ri.t = (int)q;
                ri.u = (int)((unsigned)rem - q * (unsigned)(U_ + 1));
            } else {
                ri.t = (int)(rem / (U_ + 1));
                ri.u = (int)(rem - (i64)ri.t * (U_ + 1));
            }
        }
    } else {
        // more sequences than lanes: the wave's first row is placed by a search on the scalar unit
        // and the lanes step on from there (the offsets they step over are wave-uniform loads)
        int lo = 0, hi = N - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (row_off[mid] <= r0) lo = mid; else hi = mid - 1;
        }
        int n = lo;
        const i64 r_last = r0 + ROWS - 1;
        for (int j = lo + 1; j < N; ++j) {
            const i64 oj = row_off[j];
            if (oj > r_last) break;
            n += (mine && oj <= r) ? 1 : 0;
        }
        if (mine) {
            ri = place_row(r, n, R, row_off, lx, ly);
            if (ri.n >= 0) { pad = pad_off[n]; labbase = lab_off[n]; }
        }
    }
    int my_lab = -1;
    i64 my_dst = -1;
    if (ri.n >= 0 && pad >= 0) {
        if (ri.u < ri.U) {
            const i64 at = (y_stride >= 0 ? (i64)ri.n * y_stride : labbase) + ri.u;
            const int l = (at >= 0 && at < y_len && (y_stride < 0 || ri.u < y_stride)) ? y[at] : -1;
            if (l < 0 || l >= V) { raise_flag(status, CWR_FLAG_BAD_LABEL); my_lab = kBadLabel; } else my_lab = l;
        }
        my_dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
    }

    // The two entries the loss wants of each row are picked out of LDS: every pass parks its packs
    // there as loaded (a wave's LDS accesses are served in order, so no barrier is needed for its
    // own region) and each lane reads its row's blank and label entry back.  Picking them out of
    // the registers instead takes a chain of selects and cross-lane reads per row, which is what
    // this kernel, bound by its vector instructions on rows this short, can least afford.
    __shared__ __attribute__((aligned(16))) v4i s_stage[kWavesPerBlock][RP * (LPR * K + 1)];
    v4i* stage = s_stage[__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))] + g * (LPR * K + 1);
    const ColPos<VEC, LPR> pb(blank);
    Lse res_lse = {0.f, 0.f};
    float res_b = 0.f, res_l = 0.f;  // results of the lane's own row
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const bool ok = r0 + p * RP + g < R;
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (!(ok && lir + k * LPR < NV)) raw[p][k] = Pack<T>::neg_inf();
#pragma unroll
        for (int k = 0; k < K; ++k) stage[lir + k * LPR] = raw[p][k];
        // the label of the row of this pass, from the lane that decoded it
        int lab;
        if (RP <= 2) {
            lab = __builtin_amdgcn_readlane(my_lab, p);
            if (RP == 2) lab = g == 0 ? lab : __builtin_amdgcn_readlane(my_lab, LPR + p);
        } else {
            lab = __shfl(my_lab, g * LPR + p);
        }
        const T* staged = reinterpret_cast<const T*>(stage);
        const float xb = Elem<T>::to_f32(staged[blank]);
        const float xl = Elem<T>::to_f32(staged[lab < 0 ? 0 : lab]);
        Lse lse;
        float unused_b, unused_l;
        gather_pass<T, LPR, K, false>(raw[p], g, pb, lab, lse, unused_b, unused_l);
        const bool here = lir == p;
        res_lse.m = here ? lse.m : res_lse.m;
        res_lse.l2s = here ? lse.l2s : res_lse.l2s;
        res_b = here ? xb : res_b;
        res_l = here ? xl : res_l;
    }
    if (mine) {
        lse_out[r] = res_lse.value();
        rowinfo[r] = make_int2(my_lab < 0 ? -1 : my_lab, ri.n);
        if (my_dst >= 0) lp[my_dst] = make_lp(res_b, res_l, res_lse, my_lab, seqmode + ri.n);
        else if (grads_skipped) grads_skipped[r] = make_float2(0.f, 0.f);
    }
}

// Long rows, and rows that do not start on a 16-byte boundary (V not a multiple of VEC): one wave
// per row, walking the 16-byte packs that cover it in chunks of 64*KC, the next chunk's loads in
// flight while the current one is reduced.  Every lane keeps a running (max, sum of exponentials)
// of its own elements, rescaled once per chunk, and the lanes are merged once at the end.  The
// packs at either end of an unaligned row also hold elements of the neighbouring rows: those are
// masked.  The tensor's first and last pack are whole (its base is 16-byte aligned and only packs
// that lie inside it are read: a ragged tail is read element by element).
template <typename T, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_long(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int KC = 4;
    const int lane = threadIdx.x & 63;
    const i64 r = wave_first_row<true>(1);
    if (r >= R) return;
    const i64 e0 = r * (i64)V, e1 = e0 + V;        // the row's elements in the flat tensor
    const i64 total = R * (i64)V;
    const i64 p0 = e0 / VEC;                       // first pack that holds any of them
    const i64 p_end = (e1 + VEC - 1) / VEC;        // one past the last
    const i64 p_whole = total / VEC;               // packs that lie inside the tensor
    const int P = (int)(p_end - p0);
    const T* row = x + e0;

    auto fetch = [&](int chunk, v4i (&raw)[KC]) {
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const i64 p = p0 + (i64)chunk * (64 * KC) + k * 64 + lane;
            raw[k] = load_raw<NT>(x + (p < p_end && p < p_whole ? p : p0) * VEC);
        }
    };
    v4i buf_a[KC], buf_b[KC];
    fetch(0, buf_a);
    // the row's place in the batch, while the first loads are in flight
    int lab = -1;
    i64 dst = -1;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    if (pad >= 0) {
        lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
    }
    const float xb = Elem<T>::to_f32(row[blank]);
    const float xl = Elem<T>::to_f32(row[lab < 0 ? 0 : lab]);

    float m = -INFINITY, s = 0.f;  // this lane's running maximum and sum of 2^((x - m) log2 e)
    auto reduce = [&](int ch, const v4i (&raw)[KC]) {
        float xv[KC][VEC];
        float cm = -INFINITY;
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const i64 p = p0 + (i64)ch * (64 * KC) + k * 64 + lane;
            Pack<T>::unpack(raw[k], xv[k]);
            // components [lo, hi) of this pack belong to the row: all of them, except in the packs at
            // its two ends, and none in a pack beyond it
            int lo = 0, hi = (p < p_end && p < p_whole) ? VEC : 0;
            if (p == p0) lo = (int)(e0 - p * VEC);
            if (p + 1 >= p_end && hi) hi = (int)(e1 - p * VEC) < VEC ? (int)(e1 - p * VEC) : VEC;
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                xv[k][c] = (c >= lo && c < hi) ? xv[k][c] : -INFINITY;
                cm = fmaxf(cm, xv[k][c]);
            }
        }
        if (cm > m) {  // rescale what has been summed so far (m = -inf: s = 0 stays 0)
            s *= fast_exp2((m - cm) * kLog2e);
            m = cm;
        }
        if (m > -INFINITY) {
            const float ms = m * kLog2e;
            float cs = 0.f;
#pragma unroll
            for (int k = 0; k < KC; ++k)
#pragma unroll
                for (int c = 0; c < VEC; ++c) cs += fast_exp2(fmaf(xv[k][c], kLog2e, -ms));
            // the exponents are off by what ms lost to rounding, the same for the whole chunk: the
            // fma recovers it exactly and the chunk's sum is brought back to the scale of m
            s = fmaf(cs, fmaf(-fmaf(m, kLog2e, -ms), kLn2, 1.f), s);
        }
    };
    // two buffers taking turns, so that no register with a load in flight is ever copied
    const int chunks = (P + 64 * KC - 1) / (64 * KC);
    for (int ch = 0; ch < chunks; ch += 2) {
        if (ch + 1 < chunks) fetch(ch + 1, buf_b);
        reduce(ch, buf_a);
        if (ch + 1 < chunks) {
            if (ch + 2 < chunks) fetch(ch + 2, buf_a);
            reduce(ch + 1, buf_b);
        }
    }
    // a ragged end of the tensor (its last, partial pack) belongs to the last row: element by element
    if (p_end > p_whole && lane == 0) {
        for (i64 e = p_whole * VEC < e0 ? e0 : p_whole * VEC; e < e1; ++e) {
            const float v = Elem<T>::to_f32(x[e]);
            if (v > m) { s *= fast_exp2((m - v) * kLog2e); m = v; }
            s += fast_exp2((v - m) * kLog2e);
        }
    }
    const float M = group_allreduce<64, OpMax>(m);
    const float S = group_allreduce<64, OpSum>(m > -INFINITY ? s * fast_exp2((m - M) * kLog2e) : 0.f);
    const Lse lse = {M, log2_of_sum(S)};
    if (lane == 0) {
        lse_out[r] = lse.value();
        rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
        if (dst >= 0) lp[dst] = make_lp(xb, xl, lse, lab, seqmode + ri.n);
        else if (grads_skipped) grads_skipped[r] = make_float2(0.f, 0.f);
    }
}

// Short rows of any length and alignment (V below 64 packs, where the packed kernels do not
// apply: V not a multiple of the pack, or an unaligned tensor): LPR lanes per row, element-wise
// loads all issued up front, 64/LPR rows per wave.
template <typename T, int LPR, int KMAX>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_small(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    constexpr int RP = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int g = lane / LPR, j = lane - g * LPR;
    const i64 r = wave_first_row(RP) + g;
    const bool live = r < R;
    const T* row = x + (live ? r : 0) * (i64)V;
    float xv[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const int v = j + k * LPR;
        xv[k] = (live && v < V) ? Elem<T>::to_f32(row[v]) : -INFINITY;
    }
    float m = xv[0];
#pragma unroll
    for (int k = 1; k < KMAX; ++k) m = fmaxf(m, xv[k]);
    m = group_allreduce<LPR, OpMax>(m);
    const float ms = m * kLog2e;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) s += fast_exp2(fmaf(xv[k], kLog2e, -ms));
    s = group_allreduce<LPR, OpSum>(s);
    const Lse lse = {m, log2_of_sum(s) - fmaf(m, kLog2e, -ms)};  // minus what ms lost to rounding
    if (live && j == 0) {
        lse_out[r] = lse.value();
        const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
        const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
        int lab = -1;
        if (pad >= 0) {
            lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
            const i64 dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
            const float xb = Elem<T>::to_f32(row[blank]);
            const float xl = lab >= 0 ? Elem<T>::to_f32(row[lab]) : 0.f;
            lp[dst] = make_lp(xb, xl, lse, lab, seqmode + ri.n);
        } else if (grads_skipped) {
            grads_skipped[r] = make_float2(0.f, 0.f);
        }
        rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
    }
}

// Any V, any alignment: one wave per row, scalar accesses.
template <typename T>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_fused_generic(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, float* __restrict__ lse_out, int2* __restrict__ rowinfo,
    float2* __restrict__ grads_skipped, int* __restrict__ seqmode, int* __restrict__ status) {
    const int lane = threadIdx.x & 63;
    const i64 r = wave_first_row(1);
    if (r >= R) return;
    const T* row = x + r * (i64)V;
    float m = -INFINITY;
    for (int v = lane; v < V; v += 64) m = fmaxf(m, Elem<T>::to_f32(row[v]));
    m = group_allreduce<64, OpMax>(m);
    const float ms = m * kLog2e;
    float s = 0.f;
    for (int v = lane; v < V; v += 64) s += fast_exp2(fmaf(Elem<T>::to_f32(row[v]), kLog2e, -ms));
    s = group_allreduce<64, OpSum>(s);
    const Lse lse = {m, log2_of_sum(s) - fmaf(m, kLog2e, -ms)};  // minus what ms lost to rounding
    if (lane == 0) {
        lse_out[r] = lse.value();
        const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
        const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
        int lab = -1;
        if (pad >= 0) {
            lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
            const i64 dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
            const float xb = Elem<T>::to_f32(row[blank]);
            const float xl = lab >= 0 ? Elem<T>::to_f32(row[lab]) : 0.f;
            lp[dst] = make_lp(xb, xl, lse, lab, seqmode + ri.n);
        } else if (grads_skipped) {
            grads_skipped[r] = make_float2(0.f, 0.f);
        }
        rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
    }
}

// x already holds log-probabilities: plain pick of two entries per row.
template <typename T>
__global__ __launch_bounds__(256) void k_gather_logprob(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    LpStore lp, int2* __restrict__ rowinfo, float2* __restrict__ grads_skipped,
    int* __restrict__ seqmode, int* __restrict__ status) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    int lab = -1;
    if (pad >= 0) {
        lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
        const i64 dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
        const T* row = x + r * (i64)V;
        const float xb = Elem<T>::to_f32(row[blank]);
        const float xl = lab >= 0 ? Elem<T>::to_f32(row[lab]) : 0.f;
        lp[dst] = make_lp(xb, xl, Lse{0.f, 0.f}, lab, seqmode + ri.n);
    } else if (grads_skipped) {
        grads_skipped[r] = make_float2(0.f, 0.f);
    }
    rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
}

// ---------------------------------------------------------------------------------------------
// gradient pass
// ---------------------------------------------------------------------------------------------
// Per-row coefficients of  grad[r,v] = softmax(x_r)[v]*cg + [v==blank]*cb + [v==label]*cl  (fused)
// or                       grad[r,v] = 0, [blank] <- cb, [label] <- cl                       (log-prob)
struct RowCoef {
    float cg, cb, cl;
    float nls;  // -lse * log2(e)
    int lab;
};

template <bool FUSED>
__device__ __forceinline__ RowCoef row_coef(i64 r, int N, const int2* __restrict__ rowinfo,
                                            const float2* __restrict__ grads, const float* __restrict__ lse,
                                            const GradOut grad_costs) {
    RowCoef rc;
    rc.cg = 0.f; rc.cb = 0.f; rc.cl = 0.f; rc.nls = 0.f; rc.lab = -1;
    const int2 info = rowinfo[r];
    if (info.y < 0 || info.y >= N) return rc;  // the row belongs to no usable sequence
    rc.lab = info.x;
    const float go = grad_costs.p[(i64)info.y * grad_costs.stride] * grad_costs.scale;
    const float2 g = grads[r];
    rc.cb = g.x * go;
    rc.cl = rc.lab >= 0 ? g.y * go : 0.f;
    if (FUSED) {
        rc.cg = -(g.x + (rc.lab >= 0 ? g.y : 0.f)) * go;
        rc.nls = -lse[r] * kLog2e;
    }
    return rc;
}

// One 16-byte pack of the gradient row; `pack` is its index inside the row.
template <typename T, bool FUSED>
__device__ __forceinline__ v4i grad_pack(v4i in, const RowCoef& rc, int pack, int blank, int V) {
    constexpr int VEC = Elem<T>::VEC;
    float xv[VEC], o[VEC];
    if (FUSED) Pack<T>::unpack(in, xv);
    const int cb_at = blank - pack * VEC;                      // component of the blank column, if 0..VEC-1
    const int cl_at = rc.lab >= 0 ? rc.lab - pack * VEC : -1;  // same for the label column
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
        float v = FUSED ? fast_exp2(fmaf(xv[c], kLog2e, rc.nls)) * rc.cg : 0.f;
        if (FUSED) {
            v += c == cb_at ? rc.cb : 0.f;
            v += c == cl_at ? rc.cl : 0.f;
        } else {
            v = c == cb_at ? rc.cb : v;
            v = c == cl_at ? rc.cl : v;  // label after blank, as the reference's scatter
        }
        o[c] = v;
    }
    return Pack<T>::pack(o);
}

// The VEC gradient values of a pack whose first element is column v0 of a row with coefficients rc
// (v0 may be negative or beyond V for the part of a pack that belongs to a neighbouring row: the
// blank / label positions then simply do not occur in it).
template <typename T, bool FUSED>
__device__ __forceinline__ void grad_elems(const float (&xv)[Elem<T>::VEC], const RowCoef& rc, int v0, int blank,
                                           float (&o)[Elem<T>::VEC]) {
    constexpr int VEC = Elem<T>::VEC;
    const int cb_at = blank - v0;
    const int cl_at = rc.lab >= 0 ? rc.lab - v0 : -1;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
        float v = FUSED ? fast_exp2(fmaf(xv[c], kLog2e, rc.nls)) * rc.cg : 0.f;
        if (FUSED) {
            v += c == cb_at ? rc.cb : 0.f;
            v += c == cl_at ? rc.cl : 0.f;
        } else {
            v = c == cb_at ? rc.cb : v;
            v = c == cl_at ? rc.cl : v;  // label after blank, as the reference's scatter
        }
        o[c] = v;
    }
}

// Any V of at least 64*VEC, aligned or not: the (R,V) tensor is walked as one flat array of 16-byte
// packs, 64 per wave, whatever the rows do.  A wave then touches at most two rows (their
// coefficients come through the scalar unit) and at most one of its packs straddles them.
template <typename T, bool FUSED, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_any(
    const T* __restrict__ x, i64 R, int V, int N, int blank, const int2* __restrict__ rowinfo,
    const float2* __restrict__ grads, const float* __restrict__ lse, const GradOut grad_costs,
    T* __restrict__ gx) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const i64 wave = wave_first_row<true>(1);  // global wave index
    const i64 total = R * (i64)V;
    const i64 E0 = wave * (64 * VEC);
    if (E0 >= total) return;
    const i64 ra = E0 / V;
    const i64 a_start = ra * V, b_start = a_start + V;  // row ra, and the row after it
    const bool two = b_start < E0 + 64 * VEC && ra + 1 < R;
    const RowCoef ca = row_coef<FUSED>(ra, N, rowinfo, grads, lse, grad_costs);
    const RowCoef cb = two ? row_coef<FUSED>(ra + 1, N, rowinfo, grads, lse, grad_costs) : ca;
    const i64 e = E0 + (i64)lane * VEC;
    if (e >= total) return;
    float xv[VEC], o[VEC];
    if (e + VEC <= total) {
        if (FUSED) Pack<T>::unpack(load_raw<NT>(x + e), xv);
        const bool in_b = e >= b_start;
        const bool straddle = !in_b && e + VEC > b_start;
        RowCoef rc;
        rc.cg = in_b ? cb.cg : ca.cg; rc.cb = in_b ? cb.cb : ca.cb; rc.cl = in_b ? cb.cl : ca.cl;
        rc.nls = in_b ? cb.nls : ca.nls; rc.lab = in_b ? cb.lab : ca.lab;
        grad_elems<T, FUSED>(xv, rc, (int)(e - (in_b ? b_start : a_start)), blank, o);
        if (straddle) {
            float ob[VEC];
            grad_elems<T, FUSED>(xv, cb, (int)(e - b_start), blank, ob);
            const int split = (int)(b_start - e);
#pragma unroll
            for (int c = 0; c < VEC; ++c) o[c] = c >= split ? ob[c] : o[c];
        }
        store_raw<NT>(gx + e, Pack<T>::pack(o));
    } else {
        // the tensor's ragged tail (fewer than VEC elements): element by element
        for (i64 g = e; g < total; ++g) {
            const bool in_b = g >= b_start;
            const RowCoef& rc = in_b ? cb : ca;
            const int v = (int)(g - (in_b ? b_start : a_start));
            float val = FUSED ? fast_exp2(fmaf(Elem<T>::to_f32(x[g]), kLog2e, rc.nls)) * rc.cg : 0.f;
            if (FUSED) {
                val += v == blank ? rc.cb : 0.f;
                val += v == rc.lab ? rc.cl : 0.f;
            } else {
                val = v == blank ? rc.cb : val;
                val = v == rc.lab ? rc.cl : val;
            }
            gx[g] = Elem<T>::from_f32(val);
        }
    }
}

// Short rows (VEC <= V < 64 packs) of any length: the same flat walk, but a wave now covers many
// rows, so every lane finds the (at most two) rows of its pack and fetches their coefficients
// itself.
template <typename T, bool FUSED, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_small(
    const T* __restrict__ x, i64 R, int V, int N, int blank, const int2* __restrict__ rowinfo,
    const float2* __restrict__ grads, const float* __restrict__ lse, const GradOut grad_costs,
    T* __restrict__ gx) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const i64 wave = wave_first_row<true>(1);
    const i64 total = R * (i64)V;
    const i64 E0 = wave * (64 * VEC);
    if (E0 >= total) return;
    const i64 r0 = E0 / V;                                  // wave-uniform: one 64-bit division per wave
    const unsigned in0 = (unsigned)(E0 - r0 * V) + (unsigned)lane * VEC;
    const unsigned dr = in0 / (unsigned)V;
    const i64 ra = r0 + dr;
    const int v0 = (int)(in0 - dr * (unsigned)V);           // column of the pack's first element in row ra
    const i64 e = E0 + (i64)lane * VEC;
    if (e >= total) return;
    const bool two = v0 + VEC > V && ra + 1 < R;            // V >= VEC: a pack meets at most two rows
    float xv[VEC], o[VEC];
    const bool whole = e + VEC <= total;
    if (FUSED && whole) Pack<T>::unpack(load_raw<NT>(x + e), xv);
    // both rows' coefficients are fetched by every lane (neighbouring lanes share them, and a
    // branch around the second fetch would put its latency behind the first one's)
    const RowCoef ca = row_coef<FUSED>(ra, N, rowinfo, grads, lse, grad_costs);
    const RowCoef cb = row_coef<FUSED>(ra + 1 < R ? ra + 1 : ra, N, rowinfo, grads, lse, grad_costs);
    if (whole) {
        grad_elems<T, FUSED>(xv, ca, v0, blank, o);
        if (two) {
            float ob[VEC];
            grad_elems<T, FUSED>(xv, cb, v0 - V, blank, ob);
            const int split = V - v0;
#pragma unroll
            for (int c = 0; c < VEC; ++c) o[c] = c >= split ? ob[c] : o[c];
        }
        store_raw<NT>(gx + e, Pack<T>::pack(o));
    } else {
        for (i64 g = e; g < total; ++g) {  // the tensor's ragged tail
            const i64 rr = g / V;
            const int v = (int)(g - rr * V);
            const RowCoef rc = row_coef<FUSED>(rr, N, rowinfo, grads, lse, grad_costs);
            float val = FUSED ? fast_exp2(fmaf(Elem<T>::to_f32(x[g]), kLog2e, rc.nls)) * rc.cg : 0.f;
            if (FUSED) {
                val += v == blank ? rc.cb : 0.f;
                val += v == rc.lab ? rc.cl : 0.f;
            } else {
                val = v == blank ? rc.cb : val;
                val = v == rc.lab ? rc.cl : val;
            }
            gx[g] = Elem<T>::from_f32(val);
        }
    }
}

// Rows of NV = 64*CH packs: a wave moves 64 consecutive packs of one row, one per lane.  The row
// is wave-uniform, so its coefficients come through the scalar unit.
template <typename T, bool FUSED, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_flat(
    const T* __restrict__ x, i64 R, int V, int N, int blank, int chunks_per_row,
    const int2* __restrict__ rowinfo, const float2* __restrict__ grads, const float* __restrict__ lse,
    const GradOut grad_costs, T* __restrict__ gx) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    // global wave index = chunk of 64 packs in the flat tensor; the host keeps their number below 2^31
    const unsigned wave = (unsigned)wave_first_row<true>(1);
    if ((i64)wave >= R * chunks_per_row) return;
    // rows are whole numbers of chunks, so the address needs no row: the load goes out first and the
    // (32-bit, branch-free) division that finds the row runs under it
    const i64 at = ((i64)wave * 64 + lane) * VEC;
    v4i in = {0, 0, 0, 0};
    if (FUSED) in = load_raw<NT>(x + at);
    const unsigned ur = wave / (unsigned)chunks_per_row;
    const i64 r = ur;
    const int pack = (int)(wave - ur * (unsigned)chunks_per_row) * 64 + lane;
    const RowCoef rc = row_coef<FUSED>(r, N, rowinfo, grads, lse, grad_costs);
    store_raw<NT>(gx + at, grad_pack<T, FUSED>(in, rc, pack, blank, V));
}

// Rows of 64/RP packs, RP = 2 or 4: a wave moves RP whole rows, one pack per lane, as one run of 64
// consecutive packs.  The rows are wave-uniform, so their coefficients come through the scalar
// unit and each lane selects its row's; per-lane loads of the row records (three more vector
// loads per lane, most lanes asking for the same address) cost 5 % of the pass on 512-byte rows.
template <typename T, bool FUSED, int RP, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_rows(
    const T* __restrict__ x, i64 R, int V, int N, int blank, const int2* __restrict__ rowinfo,
    const float2* __restrict__ grads, const float* __restrict__ lse, const GradOut grad_costs,
    T* __restrict__ gx) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int LPR = 64 / RP;
    const int lane = threadIdx.x & 63;
    const i64 r0 = wave_first_row<true>(RP);
    if (r0 >= R) return;
    const int g = lane / LPR;
    const bool ok = r0 + g < R;
    const i64 at = (r0 * LPR + (ok ? lane : lane % LPR)) * VEC;  // rows beyond the tensor re-read the wave's first
    v4i in = {0, 0, 0, 0};
    if (FUSED) in = load_raw<NT>(x + at);
    RowCoef rc = row_coef<FUSED>(r0, N, rowinfo, grads, lse, grad_costs);
#pragma unroll
    for (int j = 1; j < RP; ++j) {
        const RowCoef cj = row_coef<FUSED>(r0 + j < R ? r0 + j : r0, N, rowinfo, grads, lse, grad_costs);
        const bool mine = g == j;
        rc.cg = mine ? cj.cg : rc.cg; rc.cb = mine ? cj.cb : rc.cb; rc.cl = mine ? cj.cl : rc.cl;
        rc.nls = mine ? cj.nls : rc.nls; rc.lab = mine ? cj.lab : rc.lab;
    }
    const v4i o = grad_pack<T, FUSED>(in, rc, lane % LPR, blank, V);
    if (ok) store_raw<NT>(gx + at, o);
}

// Other packed shapes: LPR lanes per row, K packs per lane, 64/LPR rows per wave.
template <typename T, bool FUSED, int LPR, int K, bool NT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad(
    const T* __restrict__ x, i64 R, int V, int N, int blank, const int2* __restrict__ rowinfo,
    const float2* __restrict__ grads, const float* __restrict__ lse,
    const GradOut grad_costs, T* __restrict__ gx) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int RP = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const i64 r0 = wave_first_row(RP);
    if (r0 >= R) return;
    const int NV = V / VEC;
    const int g = lane / LPR, lir = lane % LPR;
    const i64 r = r0 + g;
    const bool ok = r < R;
    const i64 rbase = (ok ? r : r0) * (i64)V;
    v4i in[K];
    if (FUSED) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = lir + k * LPR;
            in[k] = load_raw<NT>(x + rbase + (i64)(j < NV ? j : 0) * VEC);
        }
    }
    const RowCoef rc = row_coef<FUSED>(ok ? r : r0, N, rowinfo, grads, lse, grad_costs);
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = lir + k * LPR;
        const v4i o = grad_pack<T, FUSED>(in[k], rc, j, blank, V);
        if (ok && j < NV) store_raw<NT>(gx + rbase + (i64)j * VEC, o);
    }
}

template <typename T, bool FUSED>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_generic(
    const T* __restrict__ x, i64 R, int V, int N, int blank, const int2* __restrict__ rowinfo,
    const float2* __restrict__ grads, const float* __restrict__ lse,
    const GradOut grad_costs, T* __restrict__ gx) {
    const int lane = threadIdx.x & 63;
    const i64 r = wave_first_row(1);
    if (r >= R) return;
    const RowCoef rc = row_coef<FUSED>(r, N, rowinfo, grads, lse, grad_costs);
    const T* row = x + r * (i64)V;
    T* orow = gx + r * (i64)V;
    for (int v = lane; v < V; v += 64) {
        float o = FUSED ? fast_exp2(fmaf(Elem<T>::to_f32(row[v]), kLog2e, rc.nls)) * rc.cg : 0.f;
        if (FUSED) {
            if (v == blank) o += rc.cb;
            if (v == rc.lab) o += rc.cl;
        } else {
            if (v == blank) o = rc.cb;
            if (v == rc.lab) o = rc.cl;
        }
        orow[v] = Elem<T>::from_f32(o);
    }
}

// The per-row record of the backward pass, for callers that did not keep the one cwr_forward wrote.
__global__ __launch_bounds__(256) void k_rowinfo(const int* __restrict__ lx, const int* __restrict__ ly,
                                                 const int* __restrict__ y, i64 y_stride, i64 y_len,
                                                 const i64* __restrict__ row_off,
                                                 const i64* __restrict__ lab_off, int N, i64 R, int V,
                                                 int2* __restrict__ rowinfo) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const int lab = ri.n >= 0 ? fetch_label(ri, y, y_stride, y_len, lab_off, V, nullptr) : -1;
    rowinfo[r] = make_int2(lab < 0 ? -1 : lab, ri.n);
}

int launch_rowinfo(const Batch& b, int* rowinfo) {
    if (b.R == 0) return CWR_OK;
    CWR_LAUNCH(k_rowinfo, dim3((unsigned)((b.R + 255) / 256)), dim3(256), 0, b.stream, b.lx, b.ly,
                       b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, b.N, b.R, b.V,
                       reinterpret_cast<int2*>(rowinfo));
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// dispatch
// ---------------------------------------------------------------------------------------------
// Lanes per row and packs per lane for a row of NV packs; false if the packed path cannot take it.
static bool pick_shape(int NV, int* lpr, int* k) {
    if (NV < 8) return false;
    if (NV <= 8) { *lpr = 8; *k = 1; return true; }
    if (NV <= 16) { *lpr = 16; *k = 1; return true; }
    if (NV <= 32) { *lpr = 32; *k = 1; return true; }
    *lpr = 64;
    for (int kk = 1; kk <= 16; kk *= 2)
        if (NV <= 64 * kk) { *k = kk; return true; }
    return false;
}

// The same for the gather pass.  Rows below 4 KiB share a wave: few lanes per row with 4 packs each
// keep the cross-lane part of the reduction short, and 8 KiB of loads in flight per wave (4 KiB
// for the shortest rows, whose per-row outputs weigh as much as the row) measured best.
static bool pick_gather_shape(int NV, int* lpr, int* k) {
    if (NV < 8) return false;
    if (NV <= 8) { *lpr = 8; *k = 1; return true; }
    if (NV <= 16) { *lpr = 16; *k = 1; return true; }
    if (NV <= 32) { *lpr = 8; *k = 4; return true; }
    if (NV <= 64) { *lpr = 16; *k = 4; return true; }
    if (NV <= 128) { *lpr = 32; *k = 4; return true; }
    return pick_shape(NV, lpr, k);
}

static bool base_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T>
static bool packed_ok(const void* p, int V) {
    return V % Elem<T>::VEC == 0 && (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

#define CWR_SHAPES(M)                                                                     \
    M(8, 1) M(16, 1) M(32, 1) M(64, 1) M(64, 2) M(64, 4) M(64, 8) M(64, 16)

// streaming (non-temporal) accesses for the (R,V) tensors
constexpr bool kGatherNT = true;
constexpr bool kGradNT = true;

static unsigned blocks_for_waves(i64 waves) { return (unsigned)((waves + kWavesPerBlock - 1) / kWavesPerBlock); }

template <typename T>
static int gather_typed(const Batch& b, const Workspace& ws, float* lse, int* rowinfo, float* grads) {
    const T* x = static_cast<const T*>(b.x);
    int2* ri = reinterpret_cast<int2*>(rowinfo);
    float2* gz = reinterpret_cast<float2*>(grads);  // rows of skipped sequences get a zero record here
    if (b.R == 0) return CWR_OK;
    if (b.mode == CWR_MODE_LOGPROB) {
        unsigned blocks = (unsigned)((b.R + 255) / 256);
        CWR_LAUNCH((k_gather_logprob<T>), dim3(blocks), dim3(256), 0, b.stream, x, b.R, b.V, b.lx,
                           b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank,
                           ws.lp, ri, gz, ws.seqmode, b.status);
        return check_launch();
    }
    int lpr = 0, k = 0;
    if (packed_ok<T>(b.x, b.V) && pick_gather_shape(b.V / Elem<T>::VEC, &lpr, &k)) {
#define CWR_ARGS x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N,   \
                 b.blank, ws.lp, lse, ri, gz, ws.seqmode, b.status
        // grids are multiples of 8 workgroups, see logical_block
#define CWR_ROW(KK)                                                                                  \
    if (lpr == 64 && k == KK) {                                                                      \
        CWR_LAUNCH((k_gather_row<T, KK, kGatherNT>), dim3((blocks_for_waves(b.R) + 7u) & ~7u), \
                           dim3(kWavesPerBlock * 64), 0, b.stream, CWR_ARGS);                        \
        return check_launch();                                                                       \
    }
#define CWR_ROWS(L, KK, NP)                                                                          \
    if (lpr == L && k == KK) {                                                                       \
        const int rows = (64 / L) * NP;                                                              \
        CWR_LAUNCH((k_gather_rows<T, L, KK, NP, kGatherNT>),                                 \
                           dim3((blocks_for_waves((b.R + rows - 1) / rows) + 7u) & ~7u),             \
                           dim3(kWavesPerBlock * 64), 0, b.stream, CWR_ARGS);                        \
        return check_launch();                                                                       \
    }
        CWR_ROW(4) CWR_ROW(8) CWR_ROW(16)
        CWR_ROWS(8, 1, 8) CWR_ROWS(16, 1, 8) CWR_ROWS(8, 4, 2) CWR_ROWS(16, 4, 2) CWR_ROWS(32, 4, 2)
#undef CWR_ROW
#undef CWR_ROWS
#undef CWR_ARGS
    }
    if (base_aligned(b.x) && b.V >= 64 * Elem<T>::VEC) {  // long rows, or rows off the 16-byte grid
        CWR_LAUNCH((k_gather_long<T, kGatherNT>), dim3((blocks_for_waves(b.R) + 7u) & ~7u),
                           dim3(kWavesPerBlock * 64), 0, b.stream, x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride,
                           b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, ws.lp, lse, ri, gz, ws.seqmode,
                           b.status);
        return check_launch();
    }
    if (b.V < 64 * Elem<T>::VEC) {  // short rows off the packed paths
#define CWR_SMALL(L, KM)                                                                             \
    if (b.V <= L * KM) {                                                                             \
        CWR_LAUNCH((k_gather_small<T, L, KM>), dim3(blocks_for_waves((b.R + 64 / L - 1) / (64 / L))), \
                           dim3(kWavesPerBlock * 64), 0, b.stream, x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, \
                           b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, ws.lp, lse, ri, gz,     \
                           ws.seqmode, b.status);                                                    \
        return check_launch();                                                                       \
    }
        CWR_SMALL(8, 4) CWR_SMALL(8, 8) CWR_SMALL(16, 8) CWR_SMALL(32, 8) CWR_SMALL(64, 8)
#undef CWR_SMALL
    }
    CWR_LAUNCH((k_gather_fused_generic<T>), dim3(blocks_for_waves(b.R)), dim3(kWavesPerBlock * 64),
                       0, b.stream, x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off,
                       ws.pad_off, b.N, b.blank, ws.lp, lse, ri, gz, ws.seqmode, b.status);
    return check_launch();
}

template <typename T, bool FUSED>
static int grad_typed(const Batch& b, const int* rowinfo, const float* grads, const float* lse,
                      const GradOut grad_costs, void* grad_x) {
    const T* x = static_cast<const T*>(b.x);
    T* gx = static_cast<T*>(grad_x);
    const float2* g2 = reinterpret_cast<const float2*>(grads);
    const int2* ri = reinterpret_cast<const int2*>(rowinfo);
    if (b.R == 0) return CWR_OK;
    int lpr = 0, k = 0;
    if (packed_ok<T>(grad_x, b.V) && (!FUSED || packed_ok<T>(b.x, b.V))) {
        const int NV = b.V / Elem<T>::VEC;
        if (NV % 64 == 0 && b.R * (i64)(NV / 64) < 0x7fffffffLL) {  // (2^31 chunks of 1 KiB would be 2 TiB)
            const int ch = NV / 64;
            CWR_LAUNCH((k_grad_flat<T, FUSED, kGradNT>), dim3((blocks_for_waves(b.R * ch) + 7u) & ~7u),
                               dim3(kWavesPerBlock * 64), 0, b.stream, x, b.R, b.V, b.N, b.blank, ch, ri, g2,
                               lse, grad_costs, gx);
            return check_launch();
        }
        if ((NV == 32 || NV == 16) && (b.R + 1) / 2 < 0x7fffffffLL) {
            const int rp = 64 / NV;
            const unsigned blocks = (blocks_for_waves((b.R + rp - 1) / rp) + 7u) & ~7u;
            if (rp == 2)
                CWR_LAUNCH((k_grad_rows<T, FUSED, 2, kGradNT>), dim3(blocks), dim3(kWavesPerBlock * 64), 0, b.stream, x,
                           b.R, b.V, b.N, b.blank, ri, g2, lse, grad_costs, gx);
            else
                CWR_LAUNCH((k_grad_rows<T, FUSED, 4, kGradNT>), dim3(blocks), dim3(kWavesPerBlock * 64), 0, b.stream, x,
                           b.R, b.V, b.N, b.blank, ri, g2, lse, grad_costs, gx);
            return check_launch();
        }
        if (pick_shape(NV, &lpr, &k)) {
            const int rp = 64 / lpr;
            unsigned blocks = blocks_for_waves((b.R + rp - 1) / rp);
#define CWR_CASE(L, KK)                                                                              \
    if (lpr == L && k == KK) {                                                                       \
        CWR_LAUNCH((k_grad<T, FUSED, L, KK, kGradNT>), dim3(blocks), dim3(kWavesPerBlock * 64), \
                           0, b.stream, x, b.R, b.V, b.N, b.blank, ri, g2, lse, grad_costs, gx);     \
        return check_launch();                                                                       \
    }
            CWR_SHAPES(CWR_CASE)
#undef CWR_CASE
        }
    }
    if (base_aligned(grad_x) && (!FUSED || base_aligned(b.x)) && b.V >= 64 * Elem<T>::VEC) {
        const i64 per_wave = 64 * Elem<T>::VEC;
        const i64 waves = (b.R * (i64)b.V + per_wave - 1) / per_wave;
        CWR_LAUNCH((k_grad_any<T, FUSED, kGradNT>), dim3((blocks_for_waves(waves) + 7u) & ~7u),
                           dim3(kWavesPerBlock * 64), 0, b.stream, x, b.R, b.V, b.N, b.blank, ri, g2, lse,
                           grad_costs, gx);
        return check_launch();
    }
    if (base_aligned(grad_x) && (!FUSED || base_aligned(b.x)) && b.V >= Elem<T>::VEC) {
        const i64 per_wave = 64 * Elem<T>::VEC;
        const i64 waves = (b.R * (i64)b.V + per_wave - 1) / per_wave;
        CWR_LAUNCH((k_grad_small<T, FUSED, kGradNT>), dim3((blocks_for_waves(waves) + 7u) & ~7u),
                           dim3(kWavesPerBlock * 64), 0, b.stream, x, b.R, b.V, b.N, b.blank, ri, g2, lse,
                           grad_costs, gx);
        return check_launch();
    }
    CWR_LAUNCH((k_grad_generic<T, FUSED>), dim3(blocks_for_waves(b.R)), dim3(kWavesPerBlock * 64), 0,
                       b.stream, x, b.R, b.V, b.N, b.blank, ri, g2, lse, grad_costs, gx);
    return check_launch();
}

int launch_gather(const Batch& b, const Workspace& ws, float* lse, int* rowinfo, float* grads) {
    switch (b.dtype) {
        case CWR_F32: return gather_typed<float>(b, ws, lse, rowinfo, grads);
        case CWR_F16: return gather_typed<__half>(b, ws, lse, rowinfo, grads);
        case CWR_BF16: return gather_typed<bf16_t>(b, ws, lse, rowinfo, grads);
        case CWR_F64: return gather_typed<double>(b, ws, lse, rowinfo, grads);
    }
    return CWR_ERR_DTYPE;
}

int launch_grad(const Batch& b, const int* rowinfo, const float* grads, const float* lse,
                const GradOut grad_costs, void* grad_x) {
    const bool fused = b.mode == CWR_MODE_FUSED;
    switch (b.dtype) {
        case CWR_F32:
            return fused ? grad_typed<float, true>(b, rowinfo, grads, lse, grad_costs, grad_x)
                         : grad_typed<float, false>(b, rowinfo, grads, lse, grad_costs, grad_x);
        case CWR_F16:
            return fused ? grad_typed<__half, true>(b, rowinfo, grads, lse, grad_costs, grad_x)
                         : grad_typed<__half, false>(b, rowinfo, grads, lse, grad_costs, grad_x);
        case CWR_BF16:
            return fused ? grad_typed<bf16_t, true>(b, rowinfo, grads, lse, grad_costs, grad_x)
                         : grad_typed<bf16_t, false>(b, rowinfo, grads, lse, grad_costs, grad_x);
        case CWR_F64:
            return fused ? grad_typed<double, true>(b, rowinfo, grads, lse, grad_costs, grad_x)
                         : grad_typed<double, false>(b, rowinfo, grads, lse, grad_costs, grad_x);
    }
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
