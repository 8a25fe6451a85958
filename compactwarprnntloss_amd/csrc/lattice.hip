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
// Walk one strip of nl columns and T frames, Q = T+nl-1 steps; step k handles row q = k (alpha)
// or q = Q-1-k (beta) of the strip.  With a = value of the cell, B / L its blank / label log-prob:
//   alpha: a = lse(own, nbr);  own' = a + B(t,u);    nbr' = a + L(t,u)     -> cells (t+1,u), (t,u+1)
//   beta : a = lse(own, nbr);  own' = a + B(t-1,u);  nbr' = a + L(t,u-1)   -> cells (t-1,u), (t,u-1)
// i.e. every cell adds the log-prob of the transition INTO its successor, so that the only
// operations between receiving the neighbour's value and handing one's own on are those of the
// log-sum-exp itself (beta fetches L(t,u-1) from the lane on its left one step ahead of time).
//
// Lanes that hold no cell at a step are not masked:
//   - before its first cell a lane holds the "no path" marker (-1e30) in own and nbr'; it reads
//     zeros from the padding (cleared below), so the marker survives (1e30 absorbs any sum);
//   - the start cell is produced by seeding its lane's `own` (alpha[0][0] = lse(0, none) = 0,
//     beta[T-1][U] = lse(B, none) = B);
//   - after its last cell a lane computes junk that no lane with a cell reads any more, and
//     stores it into padding slots;
//   - lanes >= nl use an offset every buffer range check rejects (loads give 0, stores vanish).
//
// A strip hands the values of its edge column to the next strip through a boundary stream
// indexed by the producer's step; the receiving edge lane takes the value in as the `old` operand
// of the DPP shift, so it lands in the lane that has no neighbour.  The stream is either a span of
// global memory (strips walked one after the other by one wave) or a ring in LDS (strips walked
// concurrently by one wave each, `Ring`).
constexpr int kRing = 256;             // entries of an LDS boundary ring (a multiple of kPF)
constexpr int kSpinLimit = 1 << 22;    // polls after which a waiting wave gives up

struct Ring {
    double* slots;   // LDS, kRing entries (+ a dummy area behind them for the lanes that hold no edge)
    int* produced;   // LDS, steps the producer has completed (INT_MAX when it is done)
    int* consumed;   // LDS, steps the consumer has completed
};

__device__ __forceinline__ bool wait_at_least(int* counter, int need, int* status) {
    for (int spin = 0; spin < kSpinLimit; ++spin) {
        if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= need) return true;
        __builtin_amdgcn_s_sleep(2);
    }
    atomicOr(status, CWR_FLAG_INTERNAL);
    return false;
}

// LDS accesses of one wave are performed in program order, so a counter written after the ring
// slots it announces needs no hardware wait; the compiler only has to keep the order.
__device__ __forceinline__ void keep_order() { asm volatile("" ::: "memory"); }

template <bool BETA, bool HAS_IN, bool HAS_OUT, bool CONC>
__device__ __forceinline__ void sweep_strip(const int T, const int nl, const bool seed, const int in_shift,
                                            const int out_shift,
                                            const double2* lp_strip, double* out_strip,
                                            const double* bnd_in, double* bnd_out, const Ring rin,
                                            const Ring rout, int* status) {
    const int lane = threadIdx.x & 63;
    const int Q = T + nl - 1;
    const i64 rows = strip_rows(T, nl);
    const __amdgpu_buffer_rsrc_t r_lp = make_rsrc(lp_strip, rows * nl * 16);
    const __amdgpu_buffer_rsrc_t r_out = make_rsrc(out_strip, rows * nl * 8);
    const __amdgpu_buffer_rsrc_t r_in = make_rsrc(bnd_in, (HAS_IN && !CONC) ? ((i64)T + kBndPad) * 8 : 0);
    const __amdgpu_buffer_rsrc_t r_bo = make_rsrc(bnd_out, (HAS_OUT && !CONC) ? ((i64)T + kBndPad) * 8 : 0);
    const int vo_lp = lane < nl ? lane * 16 : kOob;
    const int vo_out = lane < nl ? lane * 8 : kOob;
    const int in_lane = BETA ? 63 : 0, out_lane = BETA ? 0 : 63;
    const int vo_in = lane == in_lane ? 0 : kOob;
    const int vo_bo = lane == out_lane ? 0 : kOob;
    // LDS: the edge lane writes the ring, every other lane a private dummy slot behind it
    double* ring_out = rout.slots + (lane == out_lane ? 0 : kRing + lane);
    const int p16 = nl * 16, p8 = nl * 8;
    constexpr int dq = BETA ? -1 : 1;

    // clear the triangle of padding slots this direction reads before a lane's first cell
    for (int j = 0; j < nl - 1; ++j) {
        const int row = (BETA ? T + j : j) + kRowShift;
        const bool mine = BETA ? lane <= j : (lane > j && lane < nl);
        buf_store_zero16(r_lp, mine ? lane * 16 : kOob, row * p16);
    }
    __threadfence_block();

    int qi = (BETA ? Q - 1 : 0) + kRowShift;  // current row
    double2 ring[kPF];                        // log-probs of the next kPF rows
    double ering[kPF];                        // incoming boundary values (global stream only)
#pragma unroll
    for (int j = 0; j < kPF; ++j) {
        ring[j] = buf_load_d2(r_lp, vo_lp, (qi + dq * j) * p16);
        ering[j] = (HAS_IN && !CONC) ? buf_load_d(r_in, vo_in, (j + in_shift) * 8) : kNeg;
    }
    // alpha: own = 0 in the seed lane; beta: own = B of the seed lane's first cell
    double own = seed ? (BETA ? ring[0].x : 0.0) : kNeg;
    double pass = kNeg;
    double nbr = kNeg;  // without an incoming stream the edge lane keeps this marker for good
    const int nblocks = (Q + kPF - 1) / kPF;
    int k0 = 0;  // first step of the block
    for (int blk = 0; blk < nblocks; ++blk, k0 += kPF) {
        // entries [k0+in_shift, k0+kPF+in_shift) must have been produced; the ring slots of entries
        // [k0, k0+kPF) must be free, i.e. the consumer (which reads entry i at its step
        // i-out_shift) must be past entry k0+kPF-1-kRing
        if (CONC && HAS_IN) wait_at_least(rin.produced, k0 + kPF + in_shift, status);
        if (CONC && HAS_OUT) wait_at_least(rout.consumed, k0 + kPF - kRing - out_shift, status);
        if (CONC) keep_order();
#pragma unroll
        for (int j = 0; j < kPF; ++j) {
            const double2 c = ring[j];
            // the log-probs of this lane's next cell (beta needs them now, alpha only to refill)
            const double2 cn = buf_load_d2(r_lp, vo_lp, (qi + dq * kPF) * p16);
            const double2 c1 = ring[(j + 1) % kPF];  // the step after this one
            ring[j] = cn;
            double e;
            if (HAS_IN && CONC) {
                e = rin.slots[(k0 + j + in_shift) & (kRing - 1)];
            } else {
                e = ering[j];
                if (HAS_IN) ering[j] = buf_load_d(r_in, vo_in, (k0 + j + kPF + in_shift) * 8);
            }
            // what this cell adds for its two successors
            double add_own, add_pass;
            if (BETA) {
                add_own = c1.x;                                   // B(t-1,u): this lane's next cell
                add_pass = dpp_f64<DPP_WAVE_SHR1>(0.0, c1.y);     // L(t,u-1): the left lane's next cell
                if (HAS_IN) e += c.y;                             // the stream carries plain beta(t,u+1)
            } else {
                add_own = c.x;
                add_pass = c.y;
            }
            const double old = HAS_IN ? e : nbr;
            nbr = BETA ? dpp_f64<DPP_WAVE_SHL1>(old, pass) : dpp_f64<DPP_WAVE_SHR1>(old, pass);
            const double mx = fmax(own, nbr);
            const float d = (float)(own - nbr);
            const double l = (double)fast_log2(1.0f + fast_exp2(-fabsf(d)));
            const double a = mx + l;
            own = (mx + add_own) + l;
            pass = (mx + add_pass) + l;
            buf_store_d(r_out, vo_out, qi * p8, a);
            if (HAS_OUT) {
                // alpha hands on a + L(t,u) (= pass); beta hands on plain a
                const double h = BETA ? a : pass;
                if (CONC) ring_out[(k0 + j) & (kRing - 1)] = h;
                else buf_store_d(r_bo, vo_bo, (k0 + j) * 8, h);
            }
            qi += dq;
        }
        if (CONC) keep_order();
        if (CONC && HAS_OUT)
            __hip_atomic_store(rout.produced, blk + 1 == nblocks ? 0x7fffffff : k0 + kPF, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
        if (CONC && HAS_IN)
            __hip_atomic_store(rin.consumed, blk + 1 == nblocks ? 0x7fffffff : k0 + kPF, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}

template <bool BETA, bool CONC>
__device__ __forceinline__ void sweep_dispatch(bool has_in, bool has_out, int T, int nl, bool seed, int in_shift,
                                               int out_shift, const double2* lp, double* out, const double* bi, double* bo,
                                               Ring rin, Ring rout, int* status) {
    if (has_in && has_out) sweep_strip<BETA, true, true, CONC>(T, nl, seed, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else if (has_in) sweep_strip<BETA, true, false, CONC>(T, nl, seed, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else if (has_out) sweep_strip<BETA, false, true, CONC>(T, nl, seed, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else sweep_strip<BETA, false, false, CONC>(T, nl, seed, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
}

// One workgroup per (sequence, direction), W waves.  A sequence of S <= W strips is walked by S
// waves at once, each strip trailing the one that feeds it by the 64 steps the diagonal order
// demands plus one block of kPF steps of slack; the boundary values travel through LDS rings
// guarded by two progress counters per ring.  A wave only ever waits for the wave of the strip
// before it (values) or after it (ring space), and strip 0 waits for nobody, so the chain always
// drains; every wait is bounded all the same.  Longer sequences (S > W) fall back to one wave
// walking the strips in turn with the streams in global memory.
constexpr int kMaxWaves = 8;

__global__ __launch_bounds__(kMaxWaves * 64) void k_lattice(
    const int* __restrict__ lx, const int* __restrict__ ly, const i64* __restrict__ pad_off,
    const i64* __restrict__ bnd_off, const double2* lp, double* alpha, double* beta, double* bnd_a,
    double* bnd_b, int beta_only, int* status) {
    __shared__ double s_ring[kMaxWaves - 1][2 * kRing + 64];
    __shared__ int s_produced[kMaxWaves];
    __shared__ int s_consumed[kMaxWaves];
    const int n = blockIdx.x;
    const int dir = beta_only ? 1 : (int)blockIdx.y;
    const int W = blockDim.x >> 6;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    if (threadIdx.x < kMaxWaves) {
        s_produced[threadIdx.x] = 0;
        s_consumed[threadIdx.x] = 0;
    }
    __syncthreads();
    const i64 pad = pad_off[n];
    if (pad < 0) return;
    const int T = lx[n], U = ly[n];
    const int Up = U + 1;
    const int S = (Up + 63) >> 6;
    const i64 full_strip = strip_rows(T, 64) * 64;
    double* out = dir ? beta : alpha;
    const int nl_last = Up - ((S - 1) << 6);
    Ring none;
    none.slots = nullptr; none.produced = nullptr; none.consumed = nullptr;

    if (S <= W) {
        // position p in the order of the walk: alpha strip p, beta strip S-1-p
        const int p = w;
        if (p >= S) return;
        const int s = dir ? S - 1 - p : p;
        const int nl = s == S - 1 ? nl_last : 64;
        const i64 base = pad + (i64)s * full_strip;
        const bool has_in = p > 0, has_out = p < S - 1;
        Ring rin = none, rout = none;
        if (has_in) { rin.slots = s_ring[p - 1]; rin.produced = &s_produced[p - 1]; rin.consumed = &s_consumed[p - 1]; }
        if (has_out) { rout.slots = s_ring[p]; rout.produced = &s_produced[p]; rout.consumed = &s_consumed[p]; }
        if (dir == 0) {
            sweep_dispatch<false, true>(has_in, has_out, T, nl, s == 0 && lane == 0, 63, 63, lp + base, out + base,
                                        nullptr, nullptr, rin, rout, status);
        } else {
            // the strip that feeds strip s is s+1; its edge lane 0 trails its first lane by nl-1 steps
            const int shift = (s + 1 == S - 1 ? nl_last : 64) - 1;
            // ... and this strip's own edge lane 0 trails by nl-1, which is what its consumer sees
            sweep_dispatch<true, true>(has_in, has_out, T, nl, s == S - 1 && lane == nl - 1, shift, nl - 1,
                                       lp + base, out + base, nullptr, nullptr, rin, rout, status);
        }
        return;
    }

    if (w != 0) return;
    double* bnd = (dir ? bnd_b : bnd_a) + bnd_off[n];
    const i64 bstride = (i64)T + kBndPad;
    for (int p = 0; p < S; ++p) {
        const int s = dir ? S - 1 - p : p;
        const int nl = s == S - 1 ? nl_last : 64;
        const i64 base = pad + (i64)s * full_strip;
        const bool has_in = p > 0, has_out = p < S - 1;
        // stream j runs between the strips at positions j and j+1 of the walk
        const double* bi = bnd + (i64)(p > 0 ? p - 1 : 0) * bstride;
        double* bo = bnd + (i64)p * bstride;
        if (dir == 0) {
            sweep_dispatch<false, false>(has_in, has_out, T, nl, s == 0 && lane == 0, 63, 63, lp + base, out + base,
                                         bi, bo, none, none, status);
        } else {
            const int shift = (s + 1 == S - 1 ? nl_last : 64) - 1;
            sweep_dispatch<true, false>(has_in, has_out, T, nl, s == S - 1 && lane == nl - 1, shift, nl - 1,
                                        lp + base, out + base, bi, bo, none, none, status);
        }
        __threadfence_block();
    }
}

int launch_lattice(const Batch& b, const Workspace& ws, bool beta_only) {
    if (b.N == 0) return CWR_OK;
    i64 strips = (b.max_u + 64) / 64;
    int waves = (int)(strips < 1 ? 1 : (strips > kMaxWaves ? kMaxWaves : strips));
    dim3 grid((unsigned)b.N, beta_only ? 1 : 2);
    hipLaunchKernelGGL(k_lattice, grid, dim3(waves * 64), 0, b.stream, b.lx, b.ly, ws.pad_off, ws.bnd_off, ws.lp,
                       ws.alpha, ws.beta, ws.bnd_a, ws.bnd_b, beta_only ? 1 : 0, b.status);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// per-row gradient w.r.t. the gathered log-probs, and the costs
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_fill(const int* __restrict__ lx, const int* __restrict__ ly,
                                               const i64* __restrict__ row_off,
                                               const i64* __restrict__ pad_off, int N, i64 R,
                                               const int2* __restrict__ rowinfo,
                                               const double2* __restrict__ lp, const double* __restrict__ alpha,
                                               const double* __restrict__ beta, float2* __restrict__ grads,
                                               float* __restrict__ costs, int* __restrict__ status) {
    const i64 r = (i64)blockIdx.x * 256 + threadIdx.x;
    if (r >= R) return;
    // the gather pass has already found the row's sequence
    const int n = rowinfo[r].y;
    RowInfo ri;
    ri.n = -1;
    if (n >= 0 && n < N) ri = place_row(r, n, R, row_off, lx, ly);
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

int launch_fill(const Batch& b, const Workspace& ws, const int* rowinfo, float* grads, float* costs) {
    if (b.R == 0) return CWR_OK;
    unsigned blocks = (unsigned)((b.R + 255) / 256);
    hipLaunchKernelGGL(k_fill, dim3(blocks), dim3(256), 0, b.stream, b.lx, b.ly, b.row_off, ws.pad_off, b.N,
                       b.R, reinterpret_cast<const int2*>(rowinfo), ws.lp, ws.alpha, ws.beta,
                       reinterpret_cast<float2*>(grads), costs, b.status);
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
