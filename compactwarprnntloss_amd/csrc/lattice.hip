// Offsets prefix scan, alpha/beta anti-diagonal recursions, and the per-row gradient / cost fill.
//
// Replaces, for gfx950 (wave64):
//   cwarp_cuda.cpp:72-77                      -> k_offsets
//   cwarp_cuda_rnnt_kernel.cu:31-273          -> k_lattice  (cal_alphas_kernel, cal_betas_kernel)
//   cwarp_cuda_rnnt_kernel.cu:275-367         -> k_fill     (fill_grad_blank/label, fill_cost)
//   cwarp_cuda_rnnt_kernel.cu:575             -> k_cost_from_beta
//
// Design: one wave owns a strip of 64 label positions of one sequence and walks it along the
// anti-diagonals; lane l holds cell (t = q - l, u = 64 s + l) at step q.  The neighbour in u is
// the adjacent lane (one DPP wave shift), the neighbour in t is the lane's own previous value, so
// a step is a handful of VALU instructions with no LDS traffic and no barrier.  Strips hand the
// values of their last column to the next strip through a small boundary stream.  Log-probs,
// alpha and beta are stored in anti-diagonal order so that every step's global access is one
// contiguous segment; a register ring prefetches the log-probs PF steps ahead.
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

// ---------------------------------------------------------------------------------------------
// offsets
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void k_offsets(const int* __restrict__ lx, const int* __restrict__ ly,
                                                i64 N, i64 R, i64* __restrict__ row_off,
                                                i64* __restrict__ lab_off, int* __restrict__ status,
                                                float* __restrict__ costs) {
    const int lane = threadIdx.x;
    i64 carry_r = 0, carry_l = 0;
    int bad = 0;
    for (i64 base = 0; base < N; base += 64) {
        i64 i = base + lane;
        i64 rows = 0, labs = 0;
        if (i < N) {
            int T = lx[i], U = ly[i];
            if (T <= 0 || U < 0) {
                bad = 1;
                if (costs) costs[i] = __int_as_float(0x7fc00000);
            } else {
                rows = (i64)T * (i64)(U + 1);
                labs = U;
            }
        }
        i64 inc_r = wave_inclusive_scan(rows);
        i64 inc_l = wave_inclusive_scan(labs);
        if (i < N) {
            i64 start = carry_r + inc_r - rows;
            row_off[i] = start;
            lab_off[i] = carry_l + inc_l - labs;
            // a sequence whose rows do not fit below R is skipped by every kernel
            if (costs && R >= 0 && rows > 0 && start + rows > R) costs[i] = __int_as_float(0x7fc00000);
        }
        carry_r += __shfl(inc_r, 63);
        carry_l += __shfl(inc_l, 63);
    }
    int any_bad = __any(bad);
    if (lane == 0) {
        row_off[N] = carry_r;
        lab_off[N] = carry_l;
        int f = 0;
        if (any_bad) f |= CWR_FLAG_BAD_LENGTH;
        if (R >= 0 && carry_r != R) f |= CWR_FLAG_ROWS_MISMATCH;
        status[0] = f;
        status[1] = 0;
        status[2] = 0;
        status[3] = 0;
    }
}

int launch_offsets(const int* lx, const int* ly, i64 N, i64 R, i64* row_off, i64* lab_off,
                   int* status, float* costs, hipStream_t stream) {
    hipLaunchKernelGGL(k_offsets, dim3(1), dim3(64), 0, stream, lx, ly, N, R, row_off, lab_off,
                       status, costs);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// lattice
// ---------------------------------------------------------------------------------------------
// Uniform (scalar) cursor over the anti-diagonals of one T x (U+1) lattice.
struct DiagCursor {
    int k;
    i64 start;
    int T, U;
    __device__ __forceinline__ void init(int k0, int T_, int U_) {
        k = k0; T = T_; U = U_;
        start = diag_start(k0, T_, (i64)U_ + 1);
    }
    __device__ __forceinline__ int umin() const { return k - (T - 1) > 0 ? k - (T - 1) : 0; }
    __device__ __forceinline__ int count() const { return (k < U ? k : U) - umin() + 1; }
    __device__ __forceinline__ void up() { start += count(); ++k; }
    __device__ __forceinline__ void down() { --k; start -= count(); }
};

// Walk one strip.  PF = prefetch depth (steps) of the log-prob register ring.
//   alpha: r = lse(own, nbr); own' = r + B; nbr' = r + L         (parents' log-probs)
//   beta : r = lse(own + B, nbr + L); own' = nbr' = r            (the cell's own log-probs)
template <bool BETA, int PF>
__device__ __forceinline__ void sweep_strip(const int T, const int U, const i64 off, const int u_base,
                                            const int nl, const bool has_in, const bool has_out,
                                            const float2* __restrict__ lp, double* __restrict__ out,
                                            const double* bnd_in, double* bnd_out) {
    const int lane = threadIdx.x & 63;
    const int u = u_base + lane;
    const bool lane_ok = lane < nl;
    const int e = BETA ? (nl - 1 - lane) : lane;  // step at which this lane meets its first cell
    const int Q = T + nl - 1;
    const int out_lane = BETA ? 0 : nl - 1;

    DiagCursor cur, pf;
    cur.init(BETA ? (T - 1 + u_base + nl - 1) : u_base, T, U);
    pf = cur;

    auto fetch = [&](const DiagCursor& c, int q) -> float2 {
        int tt = q - e;
        float2 v = make_float2(0.f, 0.f);
        if (q < Q && lane_ok && tt >= 0 && tt < T) v = lp[off + c.start + (u - c.umin())];
        return v;
    };
    auto fetch_bnd = [&](int q) -> double {
        double v = kNeg;
        if (has_in && lane < PF && q + lane < T) v = bnd_in[q + lane];
        return v;
    };

    float2 ring[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
        ring[j] = fetch(pf, j);
        if (BETA) pf.down(); else pf.up();
    }
    double own = kNeg, pass = kNeg;
    double bv = fetch_bnd(0);

    for (int q0 = 0; q0 < Q; q0 += PF) {
        double bv_next = fetch_bnd(q0 + PF);
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            const int q = q0 + j;
            if (q < Q) {
                const int tt = q - e;
                const bool act = lane_ok && tt >= 0 && tt < T;
                const float2 c = ring[j];
                ring[j] = fetch(pf, q + PF);
                if (BETA) pf.down(); else pf.up();

                const double bj = readlane_f64(bv, j);
                const double nbr = BETA ? dpp_f64<DPP_WAVE_SHL1>(bj, pass) : dpp_f64<DPP_WAVE_SHR1>(bj, pass);
                double r;
                if (BETA) {
                    r = log_sum_exp(own + (double)c.x, nbr + (double)c.y);
                    if (u == U && tt == 0) r = (double)c.x;  // beta[T-1][U] = B(T-1,U)
                } else {
                    r = log_sum_exp(own, nbr);
                    if (u == 0 && tt == 0) r = 0.0;  // alpha[0][0] = 0
                }
                r = act ? r : kNeg;
                if (act) out[off + cur.start + (u - cur.umin())] = r;
                if (BETA) {
                    own = r;
                    pass = r;
                } else {
                    own = act ? r + (double)c.x : kNeg;
                    pass = act ? r + (double)c.y : kNeg;
                }
                if (has_out && act && lane == out_lane) bnd_out[tt] = pass;
                if (BETA) cur.down(); else cur.up();
            }
        }
        bv = bv_next;
    }
}

// One wave per (sequence, direction); strips of 64 label positions are walked one after the
// other, the boundary stream between them lives in global memory.
template <int PF>
__global__ __launch_bounds__(64) void k_lattice(const int* __restrict__ lx, const int* __restrict__ ly,
                                                const i64* __restrict__ row_off, i64 R,
                                                const float2* __restrict__ lp, double* __restrict__ alpha,
                                                double* __restrict__ beta, double* __restrict__ bnd_a,
                                                double* __restrict__ bnd_b, int beta_only) {
    const int n = blockIdx.x;
    const int dir = beta_only ? 1 : (int)blockIdx.y;
    const int T = lx[n], U = ly[n];
    const i64 off = row_off[n];
    if (T <= 0 || U < 0 || off + (i64)T * (i64)(U + 1) > R) return;
    const int Up = U + 1;
    const int S = (Up + 63) >> 6;
    double* bnd = (dir ? bnd_b : bnd_a) + (off >> 6);
    for (int p = 0; p < S; ++p) {
        const int s = dir ? S - 1 - p : p;
        const int u_base = s << 6;
        const int nl = (Up - u_base) < 64 ? (Up - u_base) : 64;
        const bool has_in = p > 0, has_out = p < S - 1;
        if (dir == 0) {
            // boundary j sits between strips j and j+1
            sweep_strip<false, PF>(T, U, off, u_base, nl, has_in, has_out, lp, alpha,
                                   bnd + (i64)(s - 1) * T, bnd + (i64)s * T);
        } else {
            sweep_strip<true, PF>(T, U, off, u_base, nl, has_in, has_out, lp, beta,
                                  bnd + (i64)s * T, bnd + (i64)(s - 1) * T);
        }
        __threadfence_block();
    }
}

int launch_lattice(const Batch& b, const Workspace& ws, bool beta_only) {
    if (b.N == 0) return CWR_OK;
    dim3 grid((unsigned)b.N, beta_only ? 1 : 2);
    hipLaunchKernelGGL((k_lattice<16>), grid, dim3(64), 0, b.stream, b.lx, b.ly, b.row_off, b.R, ws.lp,
                       ws.alpha, ws.beta, ws.bnd_a, ws.bnd_b, beta_only ? 1 : 0);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// per-row gradient w.r.t. the gathered log-probs, and the costs
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_fill(const int* __restrict__ lx, const int* __restrict__ ly,
                                               const i64* __restrict__ row_off, int N, i64 R,
                                               const float2* __restrict__ lp, const double* __restrict__ alpha,
                                               const double* __restrict__ beta, float2* __restrict__ grads,
                                               float* __restrict__ costs, int* __restrict__ status) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    if (ri.n < 0) {
        grads[r] = make_float2(0.f, 0.f);
        return;
    }
    const int T = ri.T, U = ri.U, t = ri.t, u = ri.u;
    const i64 Up = (i64)U + 1;
    const i64 k = (i64)t + u;
    const i64 base = ri.off;
    const i64 lo = k - (T - 1) > 0 ? k - (T - 1) : 0;
    const i64 idx = base + diag_start(k, T, Up) + (u - lo);
    const double a = alpha[idx];
    const float2 c = lp[idx];
    const double b00 = beta[base];
    // both successors, (t+1,u) and (t,u+1), sit side by side on diagonal k+1
    const i64 lo1 = k + 1 - (T - 1) > 0 ? k + 1 - (T - 1) : 0;
    const i64 nxt = base + diag_start(k + 1, T, Up) + (u - lo1);
    float gb = 0.f, gl = 0.f;
    if (t < T - 1) {
        gb = -fast_exp2((float)(a + beta[nxt] + (double)c.x - b00) * kLog2e);
    } else if (u == U) {
        gb = -fast_exp2((float)(a + (double)c.x - b00) * kLog2e);
    }
    if (u < U) gl = -fast_exp2((float)(a + beta[nxt + 1] + (double)c.y - b00) * kLog2e);
    grads[r] = make_float2(gb, gl);
    if (t == T - 1 && u == U) {
        // cwarp_cuda_rnnt_kernel.cu:353-366
        double fa = a + (double)c.x;
        double fb = b00;
        double ratio = fabs(fa - fb) / fabs(fmax(fa, fb));
        if (ratio > 1e-3) {
            atomicOr(status, CWR_FLAG_FB_MISMATCH);
            fb = (fa + fb) * 0.5;
        }
        costs[ri.n] = (float)(-fb);
    }
}

int launch_fill(const Batch& b, const Workspace& ws, float* grads, float* costs) {
    if (b.R == 0) return CWR_OK;
    unsigned blocks = (unsigned)((b.R + 255) / 256);
    hipLaunchKernelGGL(k_fill, dim3(blocks), dim3(256), 0, b.stream, b.lx, b.ly, b.row_off, b.N, b.R,
                       ws.lp, ws.alpha, ws.beta, reinterpret_cast<float2*>(grads), costs, b.status);
    return check_launch();
}

__global__ __launch_bounds__(64) void k_cost_from_beta(const int* __restrict__ lx, const int* __restrict__ ly,
                                                       const i64* __restrict__ row_off, int N, i64 R,
                                                       const double* __restrict__ beta,
                                                       float* __restrict__ costs) {
    const int n = blockIdx.x * 64 + threadIdx.x;
    if (n >= N) return;
    const int T = lx[n], U = ly[n];
    const i64 off = row_off[n];
    if (T <= 0 || U < 0 || off + (i64)T * (i64)(U + 1) > R) return;  // NaN already set by k_offsets
    costs[n] = (float)(-beta[off]);
}

int launch_cost_from_beta(const Batch& b, const Workspace& ws, float* costs) {
    if (b.N == 0) return CWR_OK;
    hipLaunchKernelGGL(k_cost_from_beta, dim3((unsigned)((b.N + 63) / 64)), dim3(64), 0, b.stream, b.lx,
                       b.ly, b.row_off, b.N, b.R, ws.beta, costs);
    return check_launch();
}

}  // namespace cwr
