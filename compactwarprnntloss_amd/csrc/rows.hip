// The two passes that stream the (R,V) tensors: the gather pass (forward) and the gradient pass
// (backward).  These carry all the HBM traffic of the loss.
//
// Replaces, for gfx950 (wave64):
//   cwarp_cuda_gather_kernel.cu:19-43   gather_cuda_kernel        -> k_gather_*
//   cwarp_cuda_gather_kernel.cu:52-74   scatter_grad_cuda_kernel  \
//   cwarp_cuda.cpp:134 (zeros(R,V))                                > k_grad_*
//   cwarp_cuda_rnnt_kernel.cu:512-521   cwarp_cuda_backward_      /
//
// Work split: a wave owns 64 consecutive rows.  In a preamble lane i decodes row r0+i (owning
// sequence, label, per-row scalars); the main loop then walks the rows, LPR lanes per row, each
// lane moving K 16-byte packs, and fetches the row's scalars from lane i with a wave permute.
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

constexpr int kWavesPerBlock = 4;
constexpr int kRowsPerWave = 64;

// What the lattice walk consumes: (blank, label) log-probabilities as base-2 logarithms in fp64,
// floored so that -inf logits stay finite.
__device__ __forceinline__ double2 make_lp(float xb, float xl, float lse) {
    const double b = ((double)fmaxf(xb, kLpFloor) - (double)lse) * 1.4426950408889634;
    const double l = ((double)fmaxf(xl, kLpFloor) - (double)lse) * 1.4426950408889634;
    return make_double2(b, l);
}

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
template <typename T, int LPR, int K>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_fused(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    double2* __restrict__ lp,
    float* __restrict__ lse_out, int* __restrict__ status) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int RP = 64 / LPR;  // rows per pass
    const int lane = threadIdx.x & 63;
    const i64 r0 = ((i64)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * kRowsPerWave;
    if (r0 >= R) return;

    // preamble: lane i looks after row r0+i
    int my_lab = -1;
    i64 my_dst = -1;
    {
        const i64 r = r0 + lane;
        if (r < R) {
            const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
            const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
            if (pad >= 0) {
                my_lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
                my_dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
            }
        }
    }

    const int NV = V / VEC;
    const int g = lane / LPR, lir = lane % LPR;
    const ColPos<VEC, LPR> pb(blank);
#pragma unroll 1
    for (int p = 0; p < kRowsPerWave / RP; ++p) {
        if (r0 + (i64)p * RP >= R) break;
        const int i = p * RP + g;
        const i64 r = r0 + i;
        const bool ok = r < R;
        const int lab = __shfl(my_lab, i);
        const i64 dst = __shfl(my_dst, i);
        const T* row = x + r * (i64)V;

        float xv[K][VEC];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = lir + k * LPR;
            if (ok && j < NV) {
                load_pack<T, VEC>(row + (i64)j * VEC, xv[k]);
            } else {
#pragma unroll
                for (int c = 0; c < VEC; ++c) xv[k][c] = -INFINITY;
            }
        }
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int c = 0; c < VEC; ++c) m = fmaxf(m, xv[k][c]);
        m = group_allreduce<LPR, OpMax>(m);
        const float ms = m * kLog2e;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int c = 0; c < VEC; ++c) s += fast_exp2(fmaf(xv[k][c], kLog2e, -ms));
        s = group_allreduce<LPR, OpSum>(s);
        const float lse = fmaf(fast_log2(s), kLn2, m);

        // pick the blank and label entries out of the registers
        const ColPos<VEC, LPR> pl(lab < 0 ? 0 : lab);
        float cb = 0.f, cl = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                if (k == pb.k && c == pb.c) cb = xv[k][c];
                if (k == pl.k && c == pl.c) cl = xv[k][c];
            }
        }
        const float xb = __shfl(cb, g * LPR + pb.lane);
        const float xl = __shfl(cl, g * LPR + pl.lane);
        if (ok && lir == 0) {
            lse_out[r] = lse;
            if (dst >= 0) lp[dst] = make_lp(xb, lab >= 0 ? xl : lse, lse);
        }
    }
}

// Any V, any alignment: one wave per row, scalar accesses.
template <typename T>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_gather_fused_generic(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    double2* __restrict__ lp,
    float* __restrict__ lse_out, int* __restrict__ status) {
    const int lane = threadIdx.x & 63;
    const i64 r = (i64)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (r >= R) return;
    const T* row = x + r * (i64)V;
    float m = -INFINITY;
    for (int v = lane; v < V; v += 64) m = fmaxf(m, Elem<T>::to_f32(row[v]));
    m = group_allreduce<64, OpMax>(m);
    const float ms = m * kLog2e;
    float s = 0.f;
    for (int v = lane; v < V; v += 64) s += fast_exp2(fmaf(Elem<T>::to_f32(row[v]), kLog2e, -ms));
    s = group_allreduce<64, OpSum>(s);
    const float lse = fmaf(fast_log2(s), kLn2, m);
    if (lane == 0) {
        lse_out[r] = lse;
        const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
        const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
        if (pad >= 0) {
            const int lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
            const i64 dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
            const float xb = Elem<T>::to_f32(row[blank]);
            const float xl = lab >= 0 ? Elem<T>::to_f32(row[lab]) : lse;
            lp[dst] = make_lp(xb, xl, lse);
        }
    }
}

// x already holds log-probabilities: plain pick of two entries per row.
template <typename T>
__global__ __launch_bounds__(256) void k_gather_logprob(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, const i64* __restrict__ pad_off, int N, int blank,
    double2* __restrict__ lp,
    int* __restrict__ status) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    if (pad < 0) return;
    const int lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
    const i64 dst = pad + lattice_slot(ri.t, ri.u, ri.T, (i64)ri.U + 1);
    const T* row = x + r * (i64)V;
    const float xb = Elem<T>::to_f32(row[blank]);
    const float xl = lab >= 0 ? Elem<T>::to_f32(row[lab]) : 0.f;
    lp[dst] = make_lp(xb, xl, 0.f);
}

// ---------------------------------------------------------------------------------------------
// gradient pass
// ---------------------------------------------------------------------------------------------
struct RowCoef {
    float cg;   // factor of softmax(x)            (fused mode)
    float cb;   // value added / written at blank
    float cl;   // value added / written at label
    float nls;  // -lse * log2(e)
    int lab;
};

template <bool FUSED>
__device__ __forceinline__ RowCoef row_coef(i64 r, i64 R, const int* lx, const int* ly, const int* y,
                                            i64 y_stride, i64 y_len, const i64* row_off,
                                            const i64* lab_off, int N, int V, const float2* grads,
                                            const float* lse, const float* grad_costs, int* status) {
    RowCoef rc;
    rc.cg = 0.f; rc.cb = 0.f; rc.cl = 0.f; rc.nls = 0.f; rc.lab = -1;
    if (r >= R) return rc;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    if (ri.n < 0) return rc;
    rc.lab = fetch_label(ri, y, y_stride, y_len, lab_off, V, status);
    const float go = grad_costs[ri.n];
    const float2 g = grads[r];
    rc.cb = g.x * go;
    rc.cl = rc.lab >= 0 ? g.y * go : 0.f;
    if (FUSED) {
        rc.cg = -(g.x + (rc.lab >= 0 ? g.y : 0.f)) * go;
        rc.nls = -lse[r] * kLog2e;
    }
    return rc;
}

template <typename T, bool FUSED, int LPR, int K>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, int N, int blank, const float2* __restrict__ grads,
    const float* __restrict__ lse, const float* __restrict__ grad_costs, T* __restrict__ gx,
    int* __restrict__ status) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int RP = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const i64 r0 = ((i64)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * kRowsPerWave;
    if (r0 >= R) return;
    const RowCoef mine = row_coef<FUSED>(r0 + lane, R, lx, ly, y, y_stride, y_len, row_off, lab_off, N, V,
                                         grads, lse, grad_costs, status);
    const int NV = V / VEC;
    const int g = lane / LPR, lir = lane % LPR;
    const ColPos<VEC, LPR> pb(blank);
#pragma unroll 1
    for (int p = 0; p < kRowsPerWave / RP; ++p) {
        if (r0 + (i64)p * RP >= R) break;
        const int i = p * RP + g;
        const i64 r = r0 + i;
        const bool ok = r < R;
        const float cg = __shfl(mine.cg, i);
        const float cb = __shfl(mine.cb, i);
        const float cl = __shfl(mine.cl, i);
        const float nls = __shfl(mine.nls, i);
        const int lab = __shfl(mine.lab, i);
        const ColPos<VEC, LPR> pl(lab < 0 ? 0 : lab);
        const bool own_b = lir == pb.lane;
        const bool own_l = lab >= 0 && lir == pl.lane;

        float xv[K][VEC];
        if (FUSED) {
            const T* row = x + r * (i64)V;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int j = lir + k * LPR;
                if (ok && j < NV) {
                    load_pack<T, VEC>(row + (i64)j * VEC, xv[k]);
                } else {
#pragma unroll
                    for (int c = 0; c < VEC; ++c) xv[k][c] = 0.f;
                }
            }
        }
        T* orow = gx + r * (i64)V;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float o[VEC];
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                float v = FUSED ? fast_exp2(fmaf(xv[k][c], kLog2e, nls)) * cg : 0.f;
                if (FUSED) {
                    if (own_b && k == pb.k && c == pb.c) v += cb;
                    if (own_l && k == pl.k && c == pl.c) v += cl;
                } else {
                    if (own_b && k == pb.k && c == pb.c) v = cb;
                    if (own_l && k == pl.k && c == pl.c) v = cl;  // label after blank
                }
                o[c] = v;
            }
            const int j = lir + k * LPR;
            if (ok && j < NV) store_pack<T, VEC>(orow + (i64)j * VEC, o);
        }
    }
}

template <typename T, bool FUSED>
__global__ __launch_bounds__(kWavesPerBlock * 64) void k_grad_generic(
    const T* __restrict__ x, i64 R, int V, const int* __restrict__ lx, const int* __restrict__ ly,
    const int* __restrict__ y, i64 y_stride, i64 y_len, const i64* __restrict__ row_off,
    const i64* __restrict__ lab_off, int N, int blank, const float2* __restrict__ grads,
    const float* __restrict__ lse, const float* __restrict__ grad_costs, T* __restrict__ gx,
    int* __restrict__ status) {
    const int lane = threadIdx.x & 63;
    const i64 r = (i64)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (r >= R) return;
    RowCoef rc;
    if (lane == 0)
        rc = row_coef<FUSED>(r, R, lx, ly, y, y_stride, y_len, row_off, lab_off, N, V, grads, lse,
                             grad_costs, status);
    rc.cg = __shfl(rc.cg, 0); rc.cb = __shfl(rc.cb, 0); rc.cl = __shfl(rc.cl, 0);
    rc.nls = __shfl(rc.nls, 0); rc.lab = __shfl(rc.lab, 0);
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

template <typename T>
static bool packed_ok(const void* p, int V) {
    return V % Elem<T>::VEC == 0 && (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

#define CWR_SHAPES(M)                                                                     \
    M(8, 1) M(16, 1) M(32, 1) M(64, 1) M(64, 2) M(64, 4) M(64, 8) M(64, 16)

template <typename T>
static int gather_typed(const Batch& b, const Workspace& ws, float* lse) {
    const T* x = static_cast<const T*>(b.x);
    if (b.R == 0) return CWR_OK;
    if (b.mode == CWR_MODE_LOGPROB) {
        unsigned blocks = (unsigned)((b.R + 255) / 256);
        hipLaunchKernelGGL((k_gather_logprob<T>), dim3(blocks), dim3(256), 0, b.stream, x, b.R, b.V, b.lx,
                           b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off, b.N, b.blank, ws.lp,
                           b.status);
        return check_launch();
    }
    int lpr = 0, k = 0;
    if (packed_ok<T>(b.x, b.V) && pick_shape(b.V / Elem<T>::VEC, &lpr, &k)) {
        const i64 rows_per_block = (i64)kWavesPerBlock * kRowsPerWave;
        unsigned blocks = (unsigned)((b.R + rows_per_block - 1) / rows_per_block);
#define CWR_CASE(L, KK)                                                                              \
    if (lpr == L && k == KK) {                                                                       \
        hipLaunchKernelGGL((k_gather_fused<T, L, KK>), dim3(blocks), dim3(kWavesPerBlock * 64), 0,   \
                           b.stream, x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off,   \
                           b.lab_off, ws.pad_off, b.N, b.blank, ws.lp, lse, b.status);                           \
        return check_launch();                                                                       \
    }
        CWR_SHAPES(CWR_CASE)
#undef CWR_CASE
    }
    unsigned blocks = (unsigned)((b.R + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL((k_gather_fused_generic<T>), dim3(blocks), dim3(kWavesPerBlock * 64), 0, b.stream,
                       x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, ws.pad_off,
                       b.N, b.blank, ws.lp, lse, b.status);
    return check_launch();
}

template <typename T, bool FUSED>
static int grad_typed(const Batch& b, const float* grads, const float* lse, const float* grad_costs,
                      void* grad_x) {
    const T* x = static_cast<const T*>(b.x);
    T* gx = static_cast<T*>(grad_x);
    const float2* g2 = reinterpret_cast<const float2*>(grads);
    if (b.R == 0) return CWR_OK;
    int lpr = 0, k = 0;
    if (packed_ok<T>(grad_x, b.V) && (!FUSED || packed_ok<T>(b.x, b.V)) &&
        pick_shape(b.V / Elem<T>::VEC, &lpr, &k)) {
        const i64 rows_per_block = (i64)kWavesPerBlock * kRowsPerWave;
        unsigned blocks = (unsigned)((b.R + rows_per_block - 1) / rows_per_block);
#define CWR_CASE(L, KK)                                                                              \
    if (lpr == L && k == KK) {                                                                       \
        hipLaunchKernelGGL((k_grad<T, FUSED, L, KK>), dim3(blocks), dim3(kWavesPerBlock * 64), 0,    \
                           b.stream, x, b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off,   \
                           b.lab_off, b.N, b.blank, g2, lse, grad_costs, gx, b.status);              \
        return check_launch();                                                                       \
    }
        CWR_SHAPES(CWR_CASE)
#undef CWR_CASE
    }
    unsigned blocks = (unsigned)((b.R + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL((k_grad_generic<T, FUSED>), dim3(blocks), dim3(kWavesPerBlock * 64), 0, b.stream, x,
                       b.R, b.V, b.lx, b.ly, b.y, b.y_stride, b.y_len, b.row_off, b.lab_off, b.N, b.blank,
                       g2, lse, grad_costs, gx, b.status);
    return check_launch();
}

int launch_gather(const Batch& b, const Workspace& ws, float* lse) {
    switch (b.dtype) {
        case CWR_F32: return gather_typed<float>(b, ws, lse);
        case CWR_F16: return gather_typed<__half>(b, ws, lse);
        case CWR_BF16: return gather_typed<bf16_t>(b, ws, lse);
        case CWR_F64: return gather_typed<double>(b, ws, lse);
    }
    return CWR_ERR_DTYPE;
}

int launch_grad(const Batch& b, const float* grads, const float* lse, const float* grad_costs,
                void* grad_x) {
    const bool fused = b.mode == CWR_MODE_FUSED;
    switch (b.dtype) {
        case CWR_F32:
            return fused ? grad_typed<float, true>(b, grads, lse, grad_costs, grad_x)
                         : grad_typed<float, false>(b, grads, lse, grad_costs, grad_x);
        case CWR_F16:
            return fused ? grad_typed<__half, true>(b, grads, lse, grad_costs, grad_x)
                         : grad_typed<__half, false>(b, grads, lse, grad_costs, grad_x);
        case CWR_BF16:
            return fused ? grad_typed<bf16_t, true>(b, grads, lse, grad_costs, grad_x)
                         : grad_typed<bf16_t, false>(b, grads, lse, grad_costs, grad_x);
        case CWR_F64:
            return fused ? grad_typed<double, true>(b, grads, lse, grad_costs, grad_x)
                         : grad_typed<double, false>(b, grads, lse, grad_costs, grad_x);
    }
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
