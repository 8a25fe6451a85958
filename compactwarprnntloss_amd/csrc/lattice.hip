// Offsets prefix scan, alpha/beta anti-diagonal recursions, and the per-row gradient / cost fill.
//
// Replaces, for gfx950 (wave64):
//   cwarp_cuda.cpp:72-77                      -> k_offsets
//   cwarp_cuda_rnnt_kernel.cu:31-273          -> k_lattice  (cal_alphas_kernel, cal_betas_kernel)
//   cwarp_cuda_rnnt_kernel.cu:275-367         -> k_fill     (fill_grad_blank/label, fill_cost)
//   cwarp_cuda_rnnt_kernel.cu:575             -> k_cost_from_beta
//
// Lattice walk: one wave owns a strip of 64 label positions of one sequence and walks it along
// the anti-diagonals; at step q lane l holds cell (t = q - l, u = 64 s + l).  The neighbour in u
// is the adjacent lane (one DPP wave shift), the neighbour in t is the lane's own previous value,
// so a step needs no LDS and no barrier.  A lone wave issues one instruction every four cycles
// whatever its kind, so the step is written for the smallest instruction count:
//   - the strip layout (see lattice_slot) makes every step's access one row at a constant pitch:
//     buffer instructions with a per-lane constant offset and a scalar row offset, no address
//     arithmetic on the vector unit;
//   - no lane is ever predicated: lanes that hold no cell read and write padding slots, and the
//     recursion keeps them at the "no path" marker by itself (see sweep_strip);
//   - values are base-2 logarithms, so log-sum-exp is v_exp_f32 / v_log_f32 without scaling.
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kOob = (int)0x80000000;  // per-lane offset that every buffer range check rejects
constexpr int kMaxFrames = 1 << 20;    // keeps a strip below the 2 GiB a buffer descriptor spans

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, i64 bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ double2 buf_load_d2(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
    return make_double2(__hiloint2double(v.y, v.x), __hiloint2double(v.w, v.z));
}
__device__ __forceinline__ double buf_load_d(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    v2i v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    return __hiloint2double(v.y, v.x);
}
__device__ __forceinline__ void buf_store_d(__amdgpu_buffer_rsrc_t r, int voff, int soff, double x) {
    v2i v;
    v.x = __double2loint(x);
    v.y = __double2hiint(x);
    __builtin_amdgcn_raw_buffer_store_b64(v, r, voff, soff, 0);
}
__device__ __forceinline__ void buf_store_zero16(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    v4i z = {0, 0, 0, 0};
    __builtin_amdgcn_raw_buffer_store_b128(z, r, voff, soff, 0);
}

// ---------------------------------------------------------------------------------------------
// offsets
// ---------------------------------------------------------------------------------------------
// One wave.  Four exclusive scans over the sequences: compact rows, labels, lattice slots and
// boundary-stream entries.  A sequence the kernels cannot take (bad lengths, rows beyond R, more
// labels than max_u) gets pad_off = -1 and cost = NaN, and is skipped everywhere.
__global__ __launch_bounds__(64) void k_offsets(const int* __restrict__ lx, const int* __restrict__ ly,
                                                i64 N, i64 R, i64 max_u, i64 slot_cap, i64 bnd_cap,
                                                i64* __restrict__ row_off, i64* __restrict__ lab_off,
                                                i64* __restrict__ pad_off, i64* __restrict__ bnd_off,
                                                int* __restrict__ status, float* __restrict__ costs) {
    const int lane = threadIdx.x;
    i64 carry_r = 0, carry_l = 0, carry_p = 0, carry_b = 0;
    int flags = 0;
    for (i64 base = 0; base < N; base += 64) {
        const i64 i = base + lane;
        i64 rows = 0, labs = 0;
        int T = 0, U = 0;
        bool ok = false;
        if (i < N) {
            T = lx[i];
            U = ly[i];
            if (T <= 0 || U < 0) {
                flags |= CWR_FLAG_BAD_LENGTH;
            } else {
                ok = true;
                rows = (i64)T * (i64)(U + 1);
                labs = U;
            }
        }
        const i64 inc_r = wave_inclusive_scan(rows);
        const i64 inc_l = wave_inclusive_scan(labs);
        const i64 start = carry_r + inc_r - rows;
        if (ok && R >= 0 && start + rows > R) ok = false;  // ROWS_MISMATCH is flagged below
        if (ok && pad_off && (U > max_u || T > kMaxFrames)) {
            ok = false;
            flags |= CWR_FLAG_U_TOO_LARGE;
        }
        i64 slots = 0, bnd = 0;
        if (ok && pad_off) {
            slots = lattice_slots(T, (i64)U + 1);
            bnd = boundary_entries(T, (i64)U + 1);
        }
        const i64 inc_p = wave_inclusive_scan(slots);
        const i64 inc_b = wave_inclusive_scan(bnd);
        if (i < N) {
            row_off[i] = start;
            lab_off[i] = carry_l + inc_l - labs;
            if (pad_off) {
                const i64 ps = carry_p + inc_p - slots, bs = carry_b + inc_b - bnd;
                if (ok && (ps + slots > slot_cap || bs + bnd > bnd_cap)) {
                    ok = false;  // cannot happen when max_u is a true bound
                    flags |= CWR_FLAG_U_TOO_LARGE;
                }
                pad_off[i] = ok ? ps : -1;
                bnd_off[i] = bs;
            }
            if (costs && !ok) costs[i] = __int_as_float(0x7fc00000);
        }
        carry_r += __shfl(inc_r, 63);
        carry_l += __shfl(inc_l, 63);
        carry_p += __shfl(inc_p, 63);
        carry_b += __shfl(inc_b, 63);
    }
    flags |= __shfl_xor(flags, 1);
    flags |= __shfl_xor(flags, 2);
    flags |= __shfl_xor(flags, 4);
    flags |= __shfl_xor(flags, 8);
    flags |= __shfl_xor(flags, 16);
    flags |= __shfl_xor(flags, 32);
    if (lane == 0) {
        row_off[N] = carry_r;
        lab_off[N] = carry_l;
        if (pad_off) {
            pad_off[N] = carry_p;
            bnd_off[N] = carry_b;
        }
        if (R >= 0 && carry_r != R) flags |= CWR_FLAG_ROWS_MISMATCH;
        status[0] = flags;
        status[1] = 0;
        status[2] = 0;
        status[3] = 0;
    }
}

int launch_offsets(const int* lx, const int* ly, i64 N, i64 R, i64 max_u, i64 slot_cap, i64 bnd_cap,
                   i64* row_off, i64* lab_off, i64* pad_off, i64* bnd_off, int* status, float* costs,
                   hipStream_t stream) {
    hipLaunchKernelGGL(k_offsets, dim3(1), dim3(64), 0, stream, lx, ly, N, R, max_u, slot_cap, bnd_cap,
                       row_off, lab_off, pad_off, bnd_off, status, costs);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// lattice
// ---------------------------------------------------------------------------------------------
// Walk one strip of nl columns and T frames: rows q = 0 .. T+nl-2 (alpha) or back (beta).
//   alpha: r = lse(own, nbr);          own' = r + B;  nbr' = r + L     (the parents' log-probs)
//   beta : r = lse(own + B, nbr + L);  own' = nbr' = r                 (the cell's own log-probs)
// Lanes that hold no cell at a step are not masked:
//   - before its first cell a lane holds the "no path" marker (-1e30) in own and nbr'; it reads
//     zeros from the padding (cleared below), so the marker survives (1e30 absorbs any sum);
//   - the start cell is produced by seeding its lane's `own` with 0 (alpha[0][0] = lse(0, none) = 0,
//     beta[T-1][U] = lse(0 + B, none) = B);
//   - after its last cell a lane computes junk that no lane with a cell reads any more, and
//     stores it into padding slots;
//   - lanes >= nl use an offset every buffer range check rejects (loads give 0, stores vanish).
// The value a strip hands to the next one (alpha: r + L of its last column; beta: r of its first
// column) goes through a boundary stream indexed by row; the receiving edge lane loads it as the
// `old` operand of the DPP shift, so it lands in the lane that has no neighbour.
template <bool BETA, bool HAS_IN, bool HAS_OUT>
__device__ __forceinline__ void sweep_strip(const int T, const int nl, const bool seed,
                                            const double2* lp_strip, double* out_strip,
                                            const double* bnd_in, double* bnd_out) {
    const int lane = threadIdx.x & 63;
    const int Q = T + nl - 1;
    const i64 rows = strip_rows(T, nl);
    const __amdgpu_buffer_rsrc_t r_lp = make_rsrc(lp_strip, rows * nl * 16);
    const __amdgpu_buffer_rsrc_t r_out = make_rsrc(out_strip, rows * nl * 8);
    const __amdgpu_buffer_rsrc_t r_in = make_rsrc(bnd_in, HAS_IN ? ((i64)T + kBndPad) * 8 : 0);
    const __amdgpu_buffer_rsrc_t r_bo = make_rsrc(bnd_out, HAS_OUT ? ((i64)T + kBndPad) * 8 : 0);
    const int vo_lp = lane < nl ? lane * 16 : kOob;
    const int vo_out = lane < nl ? lane * 8 : kOob;
    const int vo_in = lane == (BETA ? 63 : 0) ? 0 : kOob;
    const int vo_bo = lane == (BETA ? 0 : 63) ? 0 : kOob;
    const int p16 = nl * 16, p8 = nl * 8;
    constexpr int dq = BETA ? -1 : 1;
    // index of the boundary entry relative to the row index (see kBndPad)
    constexpr int in_shift = BETA ? 1 : 63;
    constexpr int out_shift = BETA ? 64 : 0;

    // clear the triangle of padding slots this direction reads before a lane's first cell
    for (int j = 0; j < nl - 1; ++j) {
        const int row = (BETA ? T + j : j) + kRowShift;
        const bool mine = BETA ? lane <= j : (lane > j && lane < nl);
        buf_store_zero16(r_lp, mine ? lane * 16 : kOob, row * p16);
    }
    __threadfence_block();

    int qi = (BETA ? Q - 1 : 0) + kRowShift;  // current row
    double2 ring[kPF];
    double ering[kPF];
#pragma unroll
    for (int j = 0; j < kPF; ++j) {
        ring[j] = buf_load_d2(r_lp, vo_lp, (qi + dq * j) * p16);
        ering[j] = HAS_IN ? buf_load_d(r_in, vo_in, (qi + dq * j + in_shift) * 8) : kNeg;
    }
    double own = seed ? 0.0 : kNeg;
    double pass = kNeg;
    double nbr = kNeg;  // without an incoming stream the edge lane keeps this marker for good
    const int nblocks = (Q + kPF - 1) / kPF;
    for (int blk = 0; blk < nblocks; ++blk) {
#pragma unroll
        for (int j = 0; j < kPF; ++j) {
            const double2 c = ring[j];
            const double e = ering[j];
            ring[j] = buf_load_d2(r_lp, vo_lp, (qi + dq * kPF) * p16);
            if (HAS_IN) ering[j] = buf_load_d(r_in, vo_in, (qi + dq * kPF + in_shift) * 8);
            const double old = HAS_IN ? e : nbr;
            nbr = BETA ? dpp_f64<DPP_WAVE_SHL1>(old, pass) : dpp_f64<DPP_WAVE_SHR1>(old, pass);
            double r;
            if (BETA) {
                r = log2_sum_exp2(own + c.x, nbr + c.y);
                own = r;
                pass = r;
            } else {
                r = log2_sum_exp2(own, nbr);
                own = r + c.x;
                pass = r + c.y;
            }
            buf_store_d(r_out, vo_out, qi * p8, r);
            if (HAS_OUT) buf_store_d(r_bo, vo_bo, (qi + out_shift) * 8, pass);
            qi += dq;
        }
    }
}

// One wave per (sequence, direction); the strips of a sequence are walked one after the other,
// the boundary streams between them live in global memory.
__global__ __launch_bounds__(64) void k_lattice(const int* __restrict__ lx, const int* __restrict__ ly,
                                                const i64* __restrict__ pad_off,
                                                const i64* __restrict__ bnd_off, const double2* lp,
                                                double* alpha, double* beta, double* bnd_a, double* bnd_b,
                                                int beta_only) {
    const int n = blockIdx.x;
    const int dir = beta_only ? 1 : (int)blockIdx.y;
    const i64 pad = pad_off[n];
    if (pad < 0) return;
    const int T = lx[n], U = ly[n];
    const int Up = U + 1;
    const int S = (Up + 63) >> 6;
    const int lane = threadIdx.x & 63;
    const i64 full_strip = strip_rows(T, 64) * 64;
    double* bnd = (dir ? bnd_b : bnd_a) + bnd_off[n];
    double* out = dir ? beta : alpha;
    const i64 bstride = (i64)T + kBndPad;
    for (int p = 0; p < S; ++p) {
        const int s = dir ? S - 1 - p : p;
        const int nl = (Up - (s << 6)) < 64 ? (Up - (s << 6)) : 64;
        const i64 base = pad + (i64)s * full_strip;
        const bool has_in = p > 0, has_out = p < S - 1;
        // boundary j sits between strips j and j+1
        if (dir == 0) {
            const bool seed = s == 0 && lane == 0;
            const double* bi = bnd + (i64)(s > 0 ? s - 1 : 0) * bstride;
            double* bo = bnd + (i64)s * bstride;
            if (has_in && has_out) sweep_strip<false, true, true>(T, nl, seed, lp + base, out + base, bi, bo);
            else if (has_in) sweep_strip<false, true, false>(T, nl, seed, lp + base, out + base, bi, bo);
            else if (has_out) sweep_strip<false, false, true>(T, nl, seed, lp + base, out + base, bi, bo);
            else sweep_strip<false, false, false>(T, nl, seed, lp + base, out + base, bi, bo);
        } else {
            const bool seed = s == S - 1 && lane == nl - 1;
            const double* bi = bnd + (i64)s * bstride;
            double* bo = bnd + (i64)(s > 0 ? s - 1 : 0) * bstride;
            if (has_in && has_out) sweep_strip<true, true, true>(T, nl, seed, lp + base, out + base, bi, bo);
            else if (has_in) sweep_strip<true, true, false>(T, nl, seed, lp + base, out + base, bi, bo);
            else if (has_out) sweep_strip<true, false, true>(T, nl, seed, lp + base, out + base, bi, bo);
            else sweep_strip<true, false, false>(T, nl, seed, lp + base, out + base, bi, bo);
        }
        __threadfence_block();
    }
}

int launch_lattice(const Batch& b, const Workspace& ws, bool beta_only) {
    if (b.N == 0) return CWR_OK;
    dim3 grid((unsigned)b.N, beta_only ? 1 : 2);
    hipLaunchKernelGGL(k_lattice, grid, dim3(64), 0, b.stream, b.lx, b.ly, ws.pad_off, ws.bnd_off, ws.lp,
                       ws.alpha, ws.beta, ws.bnd_a, ws.bnd_b, beta_only ? 1 : 0);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// per-row gradient w.r.t. the gathered log-probs, and the costs
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_fill(const int* __restrict__ lx, const int* __restrict__ ly,
                                               const i64* __restrict__ row_off,
                                               const i64* __restrict__ pad_off, int N, i64 R,
                                               const double2* __restrict__ lp, const double* __restrict__ alpha,
                                               const double* __restrict__ beta, float2* __restrict__ grads,
                                               float* __restrict__ costs, int* __restrict__ status) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    const RowInfo ri = decode_row(r, R, row_off, lx, ly, N);
    const i64 pad = ri.n >= 0 ? pad_off[ri.n] : -1;
    if (pad < 0) {
        grads[r] = make_float2(0.f, 0.f);
        return;
    }
    const int T = ri.T, U = ri.U, t = ri.t, u = ri.u;
    const i64 Up = (i64)U + 1;
    const i64 idx = pad + lattice_slot(t, u, T, Up);
    const double a = alpha[idx];
    const double2 c = lp[idx];
    const double b00 = beta[pad + lattice_slot(0, 0, T, Up)];
    // all values are base-2 logarithms
    float gb = 0.f, gl = 0.f;
    if (t < T - 1) {
        gb = -fast_exp2((float)(a + beta[pad + lattice_slot(t + 1, u, T, Up)] + c.x - b00));
    } else if (u == U) {
        gb = -fast_exp2((float)(a + c.x - b00));
    }
    if (u < U) gl = -fast_exp2((float)(a + beta[pad + lattice_slot(t, u + 1, T, Up)] + c.y - b00));
    grads[r] = make_float2(gb, gl);
    if (t == T - 1 && u == U) {
        // cwarp_cuda_rnnt_kernel.cu:353-366
        double fa = a + c.x;
        double fb = b00;
        double ratio = fabs(fa - fb) / fabs(fmax(fa, fb));
        if (ratio > 1e-3) {
            atomicOr(status, CWR_FLAG_FB_MISMATCH);
            fb = (fa + fb) * 0.5;
        }
        costs[ri.n] = (float)(-fb * (double)kLn2);
    }
}

int launch_fill(const Batch& b, const Workspace& ws, float* grads, float* costs) {
    if (b.R == 0) return CWR_OK;
    unsigned blocks = (unsigned)((b.R + 255) / 256);
    hipLaunchKernelGGL(k_fill, dim3(blocks), dim3(256), 0, b.stream, b.lx, b.ly, b.row_off, ws.pad_off, b.N,
                       b.R, ws.lp, ws.alpha, ws.beta, reinterpret_cast<float2*>(grads), costs, b.status);
    return check_launch();
}

__global__ __launch_bounds__(64) void k_cost_from_beta(const int* __restrict__ lx, const int* __restrict__ ly,
                                                       const i64* __restrict__ pad_off, int N,
                                                       const double* __restrict__ beta,
                                                       float* __restrict__ costs) {
    const int n = blockIdx.x * 64 + threadIdx.x;
    if (n >= N) return;
    const i64 pad = pad_off[n];
    if (pad < 0) return;  // NaN already set by k_offsets
    costs[n] = (float)(-beta[pad + lattice_slot(0, 0, lx[n], (i64)ly[n] + 1)] * (double)kLn2);
}

int launch_cost_from_beta(const Batch& b, const Workspace& ws, float* costs) {
    if (b.N == 0) return CWR_OK;
    hipLaunchKernelGGL(k_cost_from_beta, dim3((unsigned)((b.N + 63) / 64)), dim3(64), 0, b.stream, b.lx,
                       b.ly, ws.pad_off, b.N, ws.beta, costs);
    return check_launch();
}

}  // namespace cwr
