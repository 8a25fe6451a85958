// Offsets prefix scan, alpha/beta anti-diagonal recursions, and the per-row gradient / cost fill.
//
// Replaces, for gfx950 (wave64):
//   cwarp_cuda.cpp:72-77                      -> k_offsets
//   cwarp_cuda_rnnt_kernel.cu:31-273          -> k_lattice  (cal_alphas_kernel, cal_betas_kernel)
//   cwarp_cuda_rnnt_kernel.cu:275-367         -> k_fill     (fill_grad_blank/label, fill_cost)
//   cwarp_cuda_rnnt_kernel.cu:575             -> k_cost_from_beta
//
// Lattice walk: one wave owns a strip of 128 label positions of one sequence, two per lane, and
// walks it along skewed diagonals; at step q lane l holds the cells (t = q - l, u = 128 s + 2l) and
// (t, u + 1).  The neighbour in u of the lane's first column is the adjacent lane (one DPP wave
// shift), that of its second column the lane itself, the neighbour in t is the lane's own previous
// value, so a step needs no barrier.  A lone wave pays five to nine clocks for every instruction
// it issues, whatever its kind, so the step is written for the smallest instruction count:
//   - the strip layout (see lattice_slot) makes every step's access one row at a constant pitch:
//     buffer instructions with a per-lane constant offset and a scalar row offset that never
//     changes (the block's position sits in the descriptor), no address arithmetic at all;
//   - no lane is ever predicated: lanes that hold no cell read and write padding slots, and the
//     recursion keeps them at the "no path" marker by itself (see below);
//   - the normal number system is the scaled linear domain (one fp64 add and two multiplies per
//     cell); base-2 logarithms on the v_exp_f32 / v_log_f32 units are the fallback.
#include <atomic>

#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kOob = (int)0x80000000;  // per-lane offset that every buffer range check rejects
constexpr int kMaxFrames = 1 << 19;    // keeps a strip below the 2 GiB a buffer descriptor spans

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, i64 bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float2 buf_load_f2(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    v2i v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    return make_float2(__int_as_float(v.x), __int_as_float(v.y));
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
__device__ __forceinline__ void buf_store_d2(__amdgpu_buffer_rsrc_t r, int voff, int soff, double x, double y) {
    v4i v = {__double2loint(x), __double2hiint(x), __double2loint(y), __double2hiint(y)};
    __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, 0);
}
__device__ __forceinline__ void buf_store_zero8(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    v2i z = {0, 0};
    __builtin_amdgcn_raw_buffer_store_b64(z, r, voff, soff, 0);
}
__device__ __forceinline__ float buf_load_f(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ void buf_store_i32(__amdgpu_buffer_rsrc_t r, int voff, int soff, int x) {
    __builtin_amdgcn_raw_buffer_store_b32(x, r, voff, soff, 0);
}

// k_fill works in chunks of kFillSlots consecutive slots of the cell rows of one strip (its rows
// that hold cells: T + lanes - 1 of them, nl slots each); a sequence's chunks are numbered strip by
// strip.  Small chunks: many short waves, whose dependent loads (chunk -> sequence -> lattice
// values -> their scales) overlap across waves.
constexpr int kFillSlots = 256;
__host__ __device__ __forceinline__ i64 strip_chunks(i64 T, i64 nl) {
    return ((T + strip_lanes(nl) - 1) * strip_pitch(nl) + kFillSlots - 1) / kFillSlots;
}
__host__ __device__ __forceinline__ i64 fill_chunks(i64 T, i64 Up) {
    const i64 full = (Up - 1) >> kStripShift;
    return full * strip_chunks(T, kStripCols) + strip_chunks(T, Up - (full << kStripShift));
}

// ---------------------------------------------------------------------------------------------
// offsets
// ---------------------------------------------------------------------------------------------
// One wave.  Five exclusive scans over the sequences: compact rows, labels, lattice slots,
// boundary-stream entries and the chunks k_fill works in (fill_chunks).  A sequence the kernels cannot take (bad lengths, rows beyond R, more
// labels than max_u) gets pad_off = -1 and cost = NaN, and is skipped everywhere.
__global__ __launch_bounds__(64) void k_offsets(const int* __restrict__ lx, const int* __restrict__ ly,
                                                i64 N, i64 R, i64 max_u, i64 slot_cap, i64 bnd_cap,
                                                i64* __restrict__ row_off, i64* __restrict__ lab_off,
                                                i64* __restrict__ pad_off, i64* __restrict__ fill_off,
                                                i64* __restrict__ bnd_off, int* __restrict__ seqmode,
                                                int* __restrict__ status, float* __restrict__ costs,
                                                float* __restrict__ reduced) {
    const int lane = threadIdx.x;
    i64 carry_r = 0, carry_l = 0, carry_p = 0, carry_b = 0, carry_f = 0;
    int flags = 0, usable = 0;
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
        // whether the sequence is usable is known only after the scans it takes part in: a sequence
        // dropped below keeps its chunks, and k_fill skips them by its pad_off
        const i64 chunks = (ok && pad_off) ? fill_chunks(T, (i64)U + 1) : 0;
        const i64 inc_f = wave_inclusive_scan(chunks);
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
                usable += ok ? 1 : 0;
                fill_off[i] = carry_f + inc_f - chunks;
                bnd_off[i] = bs;
                seqmode[i] = 0;
            }
            if (costs && !ok) costs[i] = __int_as_float(0x7fc00000);
        }
        carry_r += __shfl(inc_r, 63);
        carry_l += __shfl(inc_l, 63);
        carry_p += __shfl(inc_p, 63);
        carry_b += __shfl(inc_b, 63);
        carry_f += __shfl(inc_f, 63);
    }
    flags |= __shfl_xor(flags, 1);
    flags |= __shfl_xor(flags, 2);
    flags |= __shfl_xor(flags, 4);
    flags |= __shfl_xor(flags, 8);
    flags |= __shfl_xor(flags, 16);
    flags |= __shfl_xor(flags, 32);
    for (int m = 1; m < 64; m <<= 1) usable += __shfl_xor(usable, m);
    if (lane == 0) {
        row_off[N] = carry_r;
        lab_off[N] = carry_l;
        if (pad_off) {
            pad_off[N] = carry_p;
            fill_off[N] = carry_f;
            bnd_off[N] = carry_b;
        }
        if (R >= 0 && carry_r != R) flags |= CWR_FLAG_ROWS_MISMATCH;
        status[0] = flags;
        status[1] = usable;  // sequences whose cost a later kernel writes (the others hold NaN already)
        status[2] = 0;       // how many of them have been written
        status[3] = 0;
        if (reduced && usable == 0) {  // no later kernel will write a cost: all of them are NaN
            reduced[0] = __int_as_float(0x7fc00000);
            reduced[1] = __int_as_float(0x7fc00000);
        }
    }
}

int launch_offsets(const int* lx, const int* ly, i64 N, i64 R, i64 max_u, i64 slot_cap, i64 bnd_cap,
                   i64* row_off, i64* lab_off, i64* pad_off, i64* fill_off, i64* bnd_off, int* seqmode,
                   int* status, float* costs, float* reduced, hipStream_t stream) {
    CWR_LAUNCH(k_offsets, dim3(1), dim3(64), 0, stream, lx, ly, N, R, max_u, slot_cap, bnd_cap,
                       row_off, lab_off, pad_off, fill_off, bnd_off, seqmode, status, costs, reduced);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// lattice
// ---------------------------------------------------------------------------------------------
// Walk one strip of nl columns (two per lane: lane j holds columns 2j and 2j+1 of the strip) and T
// frames.  At step k of Q = T + lanes - 1 the wave handles strip row q = k (alpha) or q = Q-1-k
// (beta): lane j the two cells of frame t = q - j.  With a = value of a cell, B / L its blank /
// label probability, and (c0, c1) the lane's columns:
//   alpha: a0 = own0 (+) nbr;          own0' = a0 (x) B(t,c0);    p = a0 (x) L(t,c0)
//          a1 = own1 (+) p;            own1' = a1 (x) B(t,c1);    nbr' = a1 (x) L(t,c1)    -> lane j+1
//   beta : a1 = own1 (+) nbr;          own1' = a1 (x) B(t-1,c1);  p = a1 (x) L(t,c0)
//          a0 = own0 (+) p;            own0' = a0 (x) B(t-1,c0);  nbr' = a0 (x) L(t,c0-1)  -> lane j-1
// i.e. every cell applies the transition INTO its successor, so that the only operations between
// receiving the neighbour's value and handing one's own on are the two (+) and two (x) of the
// lane's pair (beta fetches L(t,c0-1) from the lane on its left one step ahead of time).  Two
// columns per lane: a diagonal step serves twice the label positions for one cross-lane move, one
// store and one set of loop bookkeeping, and a sequence of up to 512 labels keeps every wave of its
// workgroup on a SIMD of its own.
//
// Two number systems implement ((+), (x)):
//   linear  values are probabilities times 2^C, C an integer kept per lane and block of kPF steps;
//           (+) is an fp64 add and (x) an fp64 multiply.  At the start of every block every lane
//           renews its scale so that the largest magnitude it can meet during the block sits at
//           2^kLinTarget, and records C for k_fill.  The gather pass has checked that no log-prob
//           of the sequence can push a value out of the fp64 range within one block (kLinMin,
//           kLinMax).
//   log     values are base-2 logarithms in fp64, (+) is max + log2(1 + 2^-|d|) on the fp32
//           exp2/log2 units, (x) an add.  Used for the sequences the gather pass marked (extreme
//           log-probs) and for those with more strips than waves.
//
// Lanes that hold no cell at a step are not masked:
//   - before its first cell a lane holds "no path" (0, or -1e30 as a logarithm) in own and nbr';
//     it reads zeros from the padding (cleared below), and "no path" survives any (x);
//   - the start cell is produced by seeding its lane's `own`;
//   - after its last cell a lane computes junk that no lane with a cell reads any more, and
//     stores it into padding slots;
//   - columns >= nl use an offset every buffer range check rejects (loads give 0, stores vanish).
//
// A strip hands the values of its edge column to the next strip through a boundary stream
// indexed by the producer's step; the receiving edge lane adds the value to the `own` of its edge
// column.  The stream is either a ring in LDS (strips walked concurrently by one wave each) or, for
// the log walk of very long label sequences, a span of global memory (strips walked one after the
// other by one wave).
constexpr int kRing = 256;             // entries of an LDS boundary ring (a multiple of kPF)
constexpr int kSpinLimit = 1 << 22;    // polls after which a waiting wave gives up
constexpr int kNoExp = -(1 << 20);     // "exponent" of zero
constexpr int kDppMin = (int)0x80000000;  // what a lane without a DPP source contributes to a maximum: with the
                                          // identity of max there, the move folds into the v_max_i32 that uses it

struct Ring {
    double* slots;   // LDS, kRing values + a dummy area behind them for the lanes that hold no edge
    int* scales;     // LDS, kRing/kPF entries: the producer's scale exponent C during the block that
                     // produced entries [16b, 16b+16)  (linear walk only)
    int* produced;   // LDS, steps the producer has completed (INT_MAX when it is done)
    int* consumed;   // LDS, steps the consumer has completed
};

// What a wait needs besides its counter: where to report, the workgroup's abort word, and how many
// polls to spend.  A wait that runs out sets the abort word; every later wait of the workgroup sees
// it first and returns at once, so a broken hand-over costs ONE spin budget, not one per block.  The
// walks do not leave their loops on a failed wait (an extra way out of the block loop makes the
// register allocator rotate the prefetch ring through copies, +15 % per block): they run on at
// their normal pace over values nobody will use, every access still inside its buffer, and the
// workgroup marks the sequence as poisoned at the end.
struct WaitCtl {
    int* status;  // the call's status word (global)
    int* abort;   // LDS, one per workgroup
    int limit;    // polls
};

__device__ __forceinline__ bool wait_at_least(int* counter, int need, const WaitCtl& wc) {
    if (__hip_atomic_load(wc.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0) return false;
    for (int spin = 0; spin < wc.limit; ++spin) {
        if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= need) return true;
        if (__hip_atomic_load(wc.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0) return false;
        __builtin_amdgcn_s_sleep(2);
    }
    __hip_atomic_store(wc.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    raise_flag(wc.status, CWR_FLAG_INTERNAL);
    return false;
}

// LDS accesses of one wave are performed in program order, so a counter written after the ring
// slots it announces needs no hardware wait; the compiler only has to keep the order.  (A signal
// fence emits nothing; an empty asm with a memory clobber would make the compiler drain every
// load in flight.)
__device__ __forceinline__ void keep_order() { __atomic_signal_fence(__ATOMIC_SEQ_CST); }

// Waits for every load issued so far.  Placed in front of a loop whose body consumes loads issued
// one trip earlier: the compiler derives ONE wait count per consuming instruction, the strictest
// over all ways of reaching it, and on the way in from the initial fill the registers consumed
// first may have been loaded last.  Without this that wait (all loads but one) would be paid on
// every trip; with it only the loop's own distance (kPF steps of loads) counts.
__device__ __forceinline__ void settle_loads() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
    __builtin_amdgcn_sched_barrier(0);
}

// Both walks share one shape.  Two rings of kPF registers hold the gathered records of the lane's
// two columns for the next kPF steps; step j issues the loads that refill entry j and prepares the
// NEXT step's transition terms from entry j+1, so a ring register is dead when its refill is issued
// (the register allocator then keeps every ring entry in place: no copies of registers with a load
// in flight, which would make the wave wait for memory at every block) and the conversions stay off
// the dependent chain.  The values that enter from the previous strip are prepared once per block
// by lanes 0..kPF-1 (lane j: the value entering at step k0+j) and picked per step with a readlane.

// Per-lane byte offsets of a lane's two columns into a row of records of `bytes` each; a column the
// strip does not have gets the offset every range check rejects.
struct LaneCols {
    int c0, c1;
};
__device__ __forceinline__ LaneCols lane_cols(int lane, int nl, int bytes) {
    LaneCols lc;
    lc.c0 = 2 * lane < nl ? 2 * lane * bytes : kOob;
    lc.c1 = 2 * lane + 1 < nl ? (2 * lane + 1) * bytes : kOob;
    return lc;
}

// The records of a lane's two columns in one row, as one 16-byte load.
__device__ __forceinline__ float4 load_pair(__amdgpu_buffer_rsrc_t r, const LaneCols v, int soff) {
    const v4i x = __builtin_amdgcn_raw_buffer_load_b128(r, v.c0, soff, 0);
    return make_float4(__int_as_float(x.x), __int_as_float(x.y), __int_as_float(x.z), __int_as_float(x.w));
}

// Zeroes the triangle of padding records a direction reads before a lane's first cell.  A zero
// record is "probability 0" for the linear walk and "log-prob 0" for the log walk; both keep a
// lane that holds "no path" there (junk in those records could be a NaN, which nothing survives).
template <bool BETA>
__device__ __forceinline__ void clear_leading(__amdgpu_buffer_rsrc_t r_cell, int T, int nl, int lane) {
    const int p8 = (int)strip_pitch(nl) * 8;
    const int nlane = (int)strip_lanes(nl);
    const LaneCols vc = lane_cols(lane, nl, 8);
#pragma unroll 4
    for (int j = 0; j < nlane - 1; ++j) {
        const int row = (BETA ? T + j : j) + kRowShift;
        const bool mine = BETA ? lane <= j : lane > j;
        buf_store_zero8(r_cell, mine ? vc.c0 : kOob, row * p8);
        buf_store_zero8(r_cell, mine ? vc.c1 : kOob, row * p8);
    }
    __threadfence_block();
}

// The linear walk wants every record it reads outside a lane's cells to be zero, before AND after
// them (and for the up to kPF-1 steps it runs past its last diagonal): then a lane outside its
// cells holds exactly 0, never junk, and "non-zero" means "a cell" for the range check below.
// Both directions of a sequence clear the same records; nothing else is ever written to them.
template <bool BETA>
__device__ __forceinline__ void clear_around(__amdgpu_buffer_rsrc_t r_cell, int T, int nl, int lane) {
    const int p8 = (int)strip_pitch(nl) * 8;
    const int nlane = (int)strip_lanes(nl);
    const int Q = T + nlane - 1;
    const LaneCols vc = lane_cols(lane, nl, 8);
    // a strip of odd width: the column of padding that completes its last lane's pair, in every row
    // (the lanes share the rows out; a few stores each)
    if (nl & 1) {
        const int rows = (int)strip_rows(T, nl);
        for (int row = lane; row < rows; row += 64) buf_store_zero8(r_cell, row * p8 + nl * 8, 0);
    }
    // row j of the cells' bounding box: lanes > j have not started; in row T+j lanes <= j have
    // finished; one store covers both (the per-lane offset picks the row)
#pragma unroll 4
    for (int j = 0; j < nlane - 1; ++j) {
        const int shift = lane > j ? 0 : T * p8;
        buf_store_zero8(r_cell, vc.c0 == kOob ? kOob : vc.c0 + shift, (j + kRowShift) * p8);
        buf_store_zero8(r_cell, vc.c1 == kOob ? kOob : vc.c1 + shift, (j + kRowShift) * p8);
    }
#pragma unroll 4
    for (int j = 1; j <= kPF; ++j) {
        buf_store_zero8(r_cell, vc.c0, (BETA ? kRowShift - j : Q - 1 + j + kRowShift) * p8);
        buf_store_zero8(r_cell, vc.c1, (BETA ? kRowShift - j : Q - 1 + j + kRowShift) * p8);
    }
    __threadfence_block();
}

// Range check of the linear walk.  All cell values must lie inside [2^kLowExp, 2^kHighExp) at their
// lane's scale, the lower bound looked at every kCheckLow-th step and the upper one every
// kCheckHigh-th; otherwise the walk reports the direction as unsafe and it is walked again in the
// log domain.  In between, a value descends from checked ones through at most two products per
// step (two columns per lane) with factors in [2^kLinMin, 2^(kLinMax+1)], so inside the bounds no
// product can leave the normal fp64 range (-600 - 4*100 > -1022, 1000 + 8*2 < 1023): the results
// are then exact up to rounding, whatever the spread of magnitudes across the lattice.  The lower
// bound is the one real data comes near (a lane's scale follows the largest of what it holds and
// hands on, and a cell whose blank is improbable holds 2^-90 of what it hands on), hence its
// closer watch.
constexpr int kCheckLow = 2;
constexpr int kCheckHigh = 4;
constexpr int kLowExp = -600;
constexpr int kHighExp = 1000;
constexpr unsigned kLowHigh = (unsigned)(1023 + kLowExp) << 20;    // high word of 2^kLowExp
constexpr unsigned kHighHigh = (unsigned)(1023 + kHighExp) << 20;  // high word of 2^kHighExp

// ---- scaled linear-domain walk (strips concurrent, LDS rings) -------------------------------
// The value entering the strip at step J of a block, moved into the edge lane's copy of `nbr`.  Lane
// J of every row of 16 lanes holds step J's entry; the edge lane (lane 0 for alpha, lane 63 for
// beta) reads it with a shift inside its row.  Under the row / bank masks the move writes the four
// lanes at the edge lane's end of the wave at most, and the shift of `pass` from the neighbouring
// lane, which follows, overwrites every lane but the edge lane.  Two moves per step, against two
// v_readlane and a multiply-add.
template <bool BETA, int J>
__device__ __forceinline__ double place_entry(double nbr, double e) {
    constexpr int ctrl = BETA ? (J == kPF - 1 ? 0xE4 : DPP_ROW_SHR + (kPF - 1 - J)) : (J == 0 ? 0xE4 : DPP_ROW_SHL + J);
    return dpp_f64<ctrl, BETA ? 0x8 : 0x1, BETA ? 0x8 : 0x1>(nbr, e);
}
template <bool BETA>
__device__ __forceinline__ double place_entry(double nbr, double e, int j) {
    static_assert(kPF == 16, "one case per step of a block");
    switch (j) {
        case 0: return place_entry<BETA, 0>(nbr, e);
        case 1: return place_entry<BETA, 1>(nbr, e);
        case 2: return place_entry<BETA, 2>(nbr, e);
        case 3: return place_entry<BETA, 3>(nbr, e);
        case 4: return place_entry<BETA, 4>(nbr, e);
        case 5: return place_entry<BETA, 5>(nbr, e);
        case 6: return place_entry<BETA, 6>(nbr, e);
        case 7: return place_entry<BETA, 7>(nbr, e);
        case 8: return place_entry<BETA, 8>(nbr, e);
        case 9: return place_entry<BETA, 9>(nbr, e);
        case 10: return place_entry<BETA, 10>(nbr, e);
        case 11: return place_entry<BETA, 11>(nbr, e);
        case 12: return place_entry<BETA, 12>(nbr, e);
        case 13: return place_entry<BETA, 13>(nbr, e);
        case 14: return place_entry<BETA, 14>(nbr, e);
        default: return place_entry<BETA, 15>(nbr, e);
    }
}

// Every LANE carries its own scale: the values of its two columns are probabilities times 2^C, with
// C renewed at the start of every block of kPF steps so that the largest of the lane's own values
// and of what its neighbour is about to hand over sits at 2^kLinTarget.  A value arriving from the
// neighbouring lane is brought to the lane's scale by the (block-constant) power of two that
// separates the two scales, inside the multiply-add that takes it in.  Like a logarithm, this
// loses nothing across lanes, however far apart their magnitudes are: the only thing that can
// underflow is a summand that is negligible next to the other summand of the SAME cell, or one of
// a lane's two columns next to the other.
// Within a block a lane's value can still drift out of the fp64 range (a run of extreme factors,
// or a much larger magnitude arriving from several columns away), which the range check catches.
// In a strip of odd width the last lane's second column is the layout's column of padding: zero
// probabilities in, zeros out.  seed_col: column of this strip that holds the start cell of the
// walk, or -1.  Returns false when the check failed.
template <bool BETA, bool HAS_IN, bool HAS_OUT>
__device__ __forceinline__ bool sweep_strip_lin(const int T, const int nl, const int seed_col, const int in_shift,
                                                const int out_shift, const float2* lp_strip,
                                                double* out_strip, int* scale_strip, const Ring rin,
                                                const Ring rout, const WaitCtl wc) {
    const int lane = threadIdx.x & 63;
    const int nlane = (int)strip_lanes(nl);
    const int Q = T + nlane - 1;
    const i64 rows = strip_rows(T, nl);
    const int nblocks = (Q + kPF - 1) / kPF;
    const int pitch = (int)strip_pitch(nl);
    const int p8 = pitch * 8, p4 = nlane * 4;
    const __amdgpu_buffer_rsrc_t r_cell = make_rsrc(lp_strip, rows * p8);
    const __amdgpu_buffer_rsrc_t r_sc = make_rsrc(scale_strip, (i64)nblocks * p4);
    const LaneCols vo = lane_cols(lane, pitch, 8);  // a lane's two columns in a row of 8-byte records
    const LaneCols vp = vo;
    const int vo_sc = lane < nlane ? lane * 4 : kOob;
    constexpr int in_lane = BETA ? 63 : 0;  // a strip that takes values in is 128 wide
    constexpr int out_lane = BETA ? 0 : 63;
    double* ring_out = rout.slots + (lane == out_lane ? 0 : kRing + lane);
    constexpr int dq = BETA ? -1 : 1;

    clear_around<BETA>(r_cell, T, nl, lane);

    const int row0 = (BETA ? Q - 1 : 0) + kRowShift;  // row of step 0
    const int mi = BETA ? row0 - 1 : row0;            // row that holds step 0's multipliers
    float4 ring[kPF];  // (blank, label) probabilities of the two columns, rows mi .. mi+dq*(kPF-1)
#pragma unroll
    for (int j = 0; j < kPF; ++j) ring[j] = load_pair(r_cell, vp, (mi + dq * j) * p8);
    int C = kLinTarget;  // this lane's scale exponent
    int d = 0;           // C minus the scale exponent of the lane the neighbour values come from
    // alpha[0][0] = 1; beta[T-1][U] = blank probability of that cell
    double own0 = 0.0, own1 = 0.0;
    float l_row0 = 0.f, l_row1 = 0.f;  // beta: L(t,c0), L(t,c1) of the row of step 0
    {
        const bool seed0 = seed_col == 2 * lane, seed1 = seed_col == 2 * lane + 1;
        if (BETA) {
            const float pb = buf_load_f(r_cell, (seed0 || seed1) ? seed_col * 8 : kOob, row0 * p8);
            l_row0 = buf_load_f(r_cell, vp.c0 == kOob ? kOob : vp.c0 + 4, row0 * p8);
            l_row1 = buf_load_f(r_cell, vp.c1 == kOob ? kOob : vp.c1 + 4, row0 * p8);
            const double sv = __builtin_ldexp((double)pb, kLinTarget);
            own0 = seed0 ? sv : 0.0;
            own1 = seed1 ? sv : 0.0;
        } else {
            own0 = seed0 ? __builtin_ldexp(1.0, kLinTarget) : 0.0;
        }
    }
    double pass = 0.0;
    double nbr = 0.0;  // the edge lane has no neighbour: it keeps "no path" here for good
    // alpha applies its own cells' probabilities: (B0, L0, B1, L1) of the row, and hands on
    // alpha(t,c1) * L1.  beta applies B(t-1,c0), B(t-1,c1) of the row before and L(t,c0), L(t,c1) of
    // the row itself (kept from the step before); it hands on plain beta(t,c0), and the lane that
    // takes it in applies its own L(t,c1) together with the change of scale, whether the value comes
    // from the lane on its right or, for the edge lane, from the strip on the right.
    double mB0 = (double)ring[0].x, mB1 = (double)ring[0].z;
    double mL0 = BETA ? (double)l_row0 : (double)ring[0].y;
    double mL1 = BETA ? (double)l_row1 : (double)ring[0].w;
    double mL0_next = BETA ? (double)ring[0].y : 0.0;  // beta: L(t-1,c0), for the step after this one
    double mL1_next = BETA ? (double)ring[0].w : 0.0;  // beta: L(t-1,c1)
    double pdL = 0.0;                                  // beta: 2^d * L(t,c1)
    unsigned lo_seen = 0xffffffffu, hi_seen = 0u;  // extremes of the cell values' high words (zero excluded)
    // lane j of every row of 16 prepares the value that enters at step j of a block
    const int jl = lane & (kPF - 1);
    // Row addressing of the step loop.  A lone wave pays five to eight clocks for EVERY instruction
    // it issues, scalar ones included, so the rows of a block are reached without any arithmetic per
    // step: the kPF row offsets inside a block never change and sit in scalar registers, and the
    // block's position goes into the base address of the two descriptors, once per block.
    int srow[kPF];
#pragma unroll
    for (int j = 0; j < kPF; ++j) {
        srow[j] = (BETA ? kPF - 1 - j : j) * p8;
        asm volatile("" : "+s"(srow[j]));  // a value of its own: never re-derived inside the loop
    }
    const i64 blk_bytes = (i64)dq * kPF * p8;
    // lowest row a block's loads (kPF rows ahead of its steps) and stores touch; never below row 0
    const char* cell_blk = reinterpret_cast<const char*>(lp_strip) + (i64)(BETA ? mi - 2 * kPF + 1 : mi + kPF) * p8;
    char* out_blk = reinterpret_cast<char*>(out_strip) + (i64)(BETA ? row0 - kPF + 1 : row0) * p8;
    settle_loads();
    int k0 = 0;
    for (int blk = 0; blk < nblocks; ++blk, k0 += kPF, cell_blk += blk_bytes, out_blk += blk_bytes) {
        // sixteen rows from the block's base, of the rows * p8 bytes the strip has from ITS base
        const __amdgpu_buffer_rsrc_t r_cell_b = make_rsrc(cell_blk, rows * p8);
        const __amdgpu_buffer_rsrc_t r_out_b = make_rsrc(out_blk, rows * p8);
        // The two counters and (speculatively) the incoming entries in ONE LDS round trip: LDS
        // serves a wave's requests in order, so entries read after a counter that already shows them
        // produced are the produced ones.  Only a counter that falls short sends the wave polling.
        double en_first = 0.0;
        int cp_first = 0;
        {
            int prod = 0x7fffffff, cons = 0x7fffffff;
            if (HAS_IN) prod = __hip_atomic_load(rin.produced, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (HAS_OUT) cons = __hip_atomic_load(rout.consumed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            keep_order();
            if (HAS_IN) {
                en_first = rin.slots[(k0 + jl + in_shift) & (kRing - 1)];
                cp_first = rin.scales[((k0 + jl + in_shift) / kPF) & (kRing / kPF - 1)];
            }
            if (HAS_IN && prod < k0 + kPF + in_shift) {
                wait_at_least(rin.produced, k0 + kPF + in_shift, wc);
                keep_order();
                en_first = rin.slots[(k0 + jl + in_shift) & (kRing - 1)];
                cp_first = rin.scales[((k0 + jl + in_shift) / kPF) & (kRing / kPF - 1)];
            }
            if (HAS_OUT && cons < k0 + kPF - kRing - out_shift)
                wait_at_least(rout.consumed, k0 + kPF - kRing - out_shift, wc);
        }
        keep_order();
        // Renew the scales.  True magnitude (binary exponent minus scale) of what the lane holds,
        // of what it will hand over and of what its neighbour will hand over next:
        const int t_own0 = own0 != 0.0 ? __builtin_amdgcn_frexp_exp(own0) - C : kNoExp;
        const int t_own1 = own1 != 0.0 ? __builtin_amdgcn_frexp_exp(own1) - C : kNoExp;
        const int t_pass = pass != 0.0 ? __builtin_amdgcn_frexp_exp(pass) - C : kNoExp;
        int t = max(max(t_own0, t_own1),
                    max(t_pass, BETA ? dpp_i32<DPP_WAVE_SHL1>(kDppMin, t_pass) : dpp_i32<DPP_WAVE_SHR1>(kDppMin, t_pass)));
        double e_lane = 0.0;  // lane j < kPF: the value entering at step k0+j
        int cp = 0;           // ... and the scale it was produced at
        if (HAS_IN) {
            const double ev = en_first;
            // entry k0+j feeds frame k0+j of the edge column: beyond the last frame it is junk
            const bool ok = k0 + jl < T && ev != 0.0;
            cp = cp_first;
            e_lane = ok ? ev : 0.0;
            // the largest of the kPF entries (they sit in every row of 16 lanes), for the edge lane
            int te = ok ? __builtin_amdgcn_frexp_exp(ev) - cp : kNoExp;
            te = max(te, dpp_i32<DPP_QUAD_XOR1>(kDppMin, te));
            te = max(te, dpp_i32<DPP_QUAD_XOR2>(kDppMin, te));
            te = max(te, dpp_i32<DPP_ROW_HALF_MIRROR>(kDppMin, te));
            te = max(te, dpp_i32<DPP_ROW_MIRROR>(kDppMin, te));
            if (lane == in_lane) t = max(t, te);
        }
        // Whatever reaches a lane during this block was, at its start, in one of the kPF lanes the
        // values come from (or enters through the edge lane, counted above): take the largest
        // magnitude over that window, so that nothing arriving can exceed 2^(kLinTarget + 2*kPF*
        // (kLinMax+1)).  Window used: the lanes before it in its row of 16 and the whole row before.
        if (BETA) {
            t = max(t, dpp_i32<DPP_ROW_SHL + 1>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHL + 2>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHL + 4>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHL + 8>(kDppMin, t));
            // lane 0 of a row now holds the row's maximum: three scalar reads instead of a trip
            // through the LDS crossbar
            const int r1 = __builtin_amdgcn_readlane(t, 16), r2 = __builtin_amdgcn_readlane(t, 32),
                      r3 = __builtin_amdgcn_readlane(t, 48);
            const int next_row = lane < 16 ? r1 : (lane < 32 ? r2 : (lane < 48 ? r3 : kNoExp));
            t = max(t, next_row);
        } else {
            t = max(t, dpp_i32<DPP_ROW_SHR + 1>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHR + 2>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHR + 4>(kDppMin, t));
            t = max(t, dpp_i32<DPP_ROW_SHR + 8>(kDppMin, t));
            // lane 15 of a row now holds the row's maximum: one broadcast into the next row
            t = max(t, dpp_i32<DPP_ROW_BCAST15, 0xE>(kDppMin, t));
        }
        const bool empty = t <= kNoExp / 2;
        int Cn = empty ? C : kLinTarget - t;
        // a lane that holds nothing yet takes the scale of the lane that started last: whatever
        // reaches it during this block has come from there, through at most 2*kPF products
        const int started = BETA ? nlane - k0 : k0 - 1;
        const int last = started < 0 ? 0 : (started > nlane - 1 ? nlane - 1 : started);
        const int Cref = __builtin_amdgcn_readlane(Cn, last);
        Cn = empty ? Cref : Cn;
        own0 = __builtin_ldexp(own0, Cn - C);
        own1 = __builtin_ldexp(own1, Cn - C);
        pass = __builtin_ldexp(pass, Cn - C);
        C = Cn;
        d = C - (BETA ? dpp_i32<DPP_WAVE_SHL1>(C, C) : dpp_i32<DPP_WAVE_SHR1>(C, C));
        if (lane >= nlane) d = -8192;  // lanes beyond the strip's width take nothing in: they stay at 0
        // 2^d as a factor: the neighbour's value then enters through one fused multiply-add instead of
        // a v_ldexp_f64 and an add.  The product with a power of two is exact, so the sum is the same
        // but for d below -1022, where the term (2^-1000 of what the lane holds, at most) is dropped
        // a little earlier.  d above 1023 would overflow whatever it scales, and inf * 0 is a NaN.
        const double pd = __builtin_ldexp(1.0, min(d, 1023));
        if (BETA) pdL = pd * mL1;
        if (HAS_IN) e_lane = __builtin_ldexp(e_lane, __builtin_amdgcn_readlane(C, in_lane) - cp);
        buf_store_i32(r_sc, vo_sc, __builtin_amdgcn_readfirstlane(blk * p4), C);  // wave-uniform, and said so
        if (HAS_OUT) rout.scales[(k0 / kPF) & (kRing / kPF - 1)] = __builtin_amdgcn_readlane(C, out_lane);
#pragma unroll
        for (int j = 0; j < kPF; ++j) {
            const float4 cn = load_pair(r_cell_b, vp, srow[j]);
            if (HAS_IN) nbr = place_entry<BETA>(nbr, e_lane, j);
            nbr = BETA ? dpp_f64<DPP_WAVE_SHL1>(nbr, pass) : dpp_f64<DPP_WAVE_SHR1>(nbr, pass);
            double a0, a1;
            if (BETA) {
                a1 = __builtin_fma(nbr, pdL, own1);
                own1 = a1 * mB1;
                a0 = own0 + a1 * mL0;
                own0 = a0 * mB0;
                pass = a0;
            } else {
                a0 = __builtin_fma(nbr, pd, own0);
                own0 = a0 * mB0;
                a1 = own1 + a0 * mL0;
                own1 = a1 * mB1;
                pass = a1 * mL1;
            }
            if (j % kCheckLow == 0) {
                const unsigned h0 = (unsigned)__double2hiint(a0), h1 = (unsigned)__double2hiint(a1);
                lo_seen = min(lo_seen, min(h0 - 1u, h1 - 1u));  // zero wraps to the top and drops out
                if (j % kCheckHigh == 0) hi_seen = max(hi_seen, max(h0, h1));
            }
            buf_store_d2(r_out_b, vo.c0, srow[j], a0, a1);
            if (HAS_OUT) ring_out[(k0 + j) & (kRing - 1)] = BETA ? a0 : pass;
            const float4 nx = ring[(j + 1) % kPF];
            mB0 = (double)nx.x;
            mB1 = (double)nx.z;
            if (BETA) {
                mL0 = mL0_next;
                mL0_next = (double)nx.y;
                mL1 = mL1_next;
                mL1_next = (double)nx.w;
                pdL = pd * mL1;
            } else {
                mL0 = (double)nx.y;
                mL1 = (double)nx.w;
            }
            ring[j] = cn;
            // keeps the conversions above inside this step: gathered at the top of the block they
            // would wait for every load in flight
            __builtin_amdgcn_sched_barrier(0);
        }
        keep_order();
        // no "last block" case in here: a select on the block count has been seen compiled into a
        // scalar select that reads a condition code nobody set (the count lived in a vector register)
        if (HAS_OUT) __hip_atomic_store(rout.produced, k0 + kPF, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (HAS_IN) __hip_atomic_store(rin.consumed, k0 + kPF, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // done: whatever the neighbours still wait for will not come from here (or is not needed here)
    if (HAS_OUT) __hip_atomic_store(rout.produced, 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (HAS_IN) __hip_atomic_store(rin.consumed, 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return __ballot(lo_seen < kLowHigh - 1u || hi_seen >= kHighHigh) == 0;
}

// ---- log-domain walk ------------------------------------------------------------------------
// CONC: strips concurrent, boundary values through the LDS rings; otherwise one wave walks the
// strips in turn and the boundary values travel through a stream in global memory, which the
// lanes that prepare the incoming entries read one block ahead.
//
// log2(2^x + 2^y) = max + log2(1 + 2^-|x-y|): the form of cwarp_cuda_rnnt_kernel.cu:22-29 in
// base 2; the running values are fp64, the correction term (at most 1) comes from the fp32
// exp2 / log2 units.
struct Lse2 {
    double mx, l;  // the sum is mx + l
};
__device__ __forceinline__ Lse2 lse2(double x, double y) {
    Lse2 r;
    r.mx = fmax(x, y);
    const float d = (float)(x - y);
    r.l = (double)fast_log2(1.0f + fast_exp2(-fabsf(d)));
    return r;
}

template <bool BETA, bool HAS_IN, bool HAS_OUT, bool CONC>
__device__ __forceinline__ void sweep_strip_log(const int T, const int nl, const int seed_col, const int in_shift,
                                                const int out_shift, const float2* lp_strip,
                                                double* out_strip, const double* bnd_in, double* bnd_out,
                                                const Ring rin, const Ring rout, const WaitCtl wc) {
    const int lane = threadIdx.x & 63;
    const int nlane = (int)strip_lanes(nl);
    const int Q = T + nlane - 1;
    const i64 rows = strip_rows(T, nl);
    const int nblocks = (Q + kPF - 1) / kPF;
    const int p8 = (int)strip_pitch(nl) * 8;
    const __amdgpu_buffer_rsrc_t r_cell = make_rsrc(lp_strip, rows * p8);
    const __amdgpu_buffer_rsrc_t r_out = make_rsrc(out_strip, rows * p8);
    const __amdgpu_buffer_rsrc_t r_in = make_rsrc(bnd_in, (HAS_IN && !CONC) ? ((i64)T + kBndPad) * 8 : 0);
    const __amdgpu_buffer_rsrc_t r_bo = make_rsrc(bnd_out, (HAS_OUT && !CONC) ? ((i64)T + kBndPad) * 8 : 0);
    const LaneCols vo = lane_cols(lane, nl, 8);  // a lane's two columns in a row of 8-byte records
    const LaneCols vl = vo;
    constexpr int in_lane = BETA ? 63 : 0;
    constexpr int out_lane = BETA ? 0 : 63;
    const int vo_bo = lane == out_lane ? 0 : kOob;
    double* ring_out = rout.slots + (lane == out_lane ? 0 : kRing + lane);
    constexpr int dq = BETA ? -1 : 1;

    clear_leading<BETA>(r_cell, T, nl, lane);

    const int row0 = (BETA ? Q - 1 : 0) + kRowShift;
    int qi = row0;
    int mi = BETA ? row0 - 1 : row0;
    float2 ring0[kPF], ring1[kPF];  // (blank, label) logarithms, rows mi .. mi+dq*(kPF-1)
#pragma unroll
    for (int j = 0; j < kPF; ++j) {
        ring0[j] = buf_load_f2(r_cell, vl.c0, (mi + dq * j) * p8);
        ring1[j] = buf_load_f2(r_cell, vl.c1, (mi + dq * j) * p8);
    }
    // alpha: own = log 1 in the seed column; beta: own = B of the seed cell
    double own0 = kNeg, own1 = kNeg;
    float l_row0 = 0.f;
    {
        const bool seed0 = seed_col == 2 * lane, seed1 = seed_col == 2 * lane + 1;
        if (BETA) {
            const float lb = buf_load_f(r_cell, (seed0 || seed1) ? seed_col * 8 : kOob, row0 * p8);
            l_row0 = buf_load_f(r_cell, vl.c0 == kOob ? kOob : vl.c0 + 4, row0 * p8);
            own0 = seed0 ? (double)lb : kNeg;
            own1 = seed1 ? (double)lb : kNeg;
        } else {
            own0 = seed0 ? 0.0 : kNeg;
        }
    }
    double pass = kNeg;
    double nbr = kNeg;
    double aB0 = (double)ring0[0].x, aB1 = (double)ring1[0].x;
    double aL0 = BETA ? (double)l_row0 : (double)ring0[0].y;
    double aL1 = (double)(BETA ? dpp_f32_or_zero<DPP_WAVE_SHR1>(ring1[0].y) : ring1[0].y);
    double aL0_next = BETA ? (double)ring0[0].y : 0.0;
    const int jl = lane & (kPF - 1);
    constexpr int edge_off = (kStripCols - 1) * 8 + 4;
    float edge = 0.f;      // beta: L(t,u) of the edge column's own cells, one block ahead
    double e_next = kNeg;  // global stream: the entries of the next block
    if (BETA && HAS_IN) edge = buf_load_f(r_cell, max(row0 - jl, 0) * p8 + edge_off, 0);
    if (HAS_IN && !CONC) e_next = buf_load_d(r_in, jl * 8, in_shift * 8);
    settle_loads();
    int k0 = 0;
    for (int blk = 0; blk < nblocks; ++blk, k0 += kPF) {
        // entries [k0+in_shift, k0+kPF+in_shift) must have been produced; the ring slots of entries
        // [k0, k0+kPF) must be free, i.e. the consumer (which reads entry i at its step
        // i-out_shift) must be past entry k0+kPF-1-kRing
        if (CONC && HAS_IN) wait_at_least(rin.produced, k0 + kPF + in_shift, wc);
        if (CONC && HAS_OUT) wait_at_least(rout.consumed, k0 + kPF - kRing - out_shift, wc);
        if (CONC) keep_order();
        double e_lane = kNeg;
        if (HAS_IN) {
            double ev;
            if (CONC) {
                ev = rin.slots[(k0 + jl + in_shift) & (kRing - 1)];
            } else {
                ev = e_next;
                e_next = buf_load_d(r_in, jl * 8, (k0 + kPF + in_shift) * 8);
            }
            if (BETA) {
                ev += (double)edge;
                edge = buf_load_f(r_cell, max(row0 - (k0 + kPF + jl), 0) * p8 + edge_off, 0);
            }
            e_lane = k0 + jl < T ? ev : kNeg;  // beyond the last frame the entries are junk
        }
#pragma unroll
        for (int j = 0; j < kPF; ++j) {
            const float2 cn0 = buf_load_f2(r_cell, vl.c0, (mi + dq * kPF) * p8);
            const float2 cn1 = buf_load_f2(r_cell, vl.c1, (mi + dq * kPF) * p8);
            // the edge lane has no neighbour: the entry from the previous strip takes that place
            const double old = HAS_IN ? readlane_f64(e_lane, j) : nbr;
            nbr = BETA ? dpp_f64<DPP_WAVE_SHL1>(old, pass) : dpp_f64<DPP_WAVE_SHR1>(old, pass);
            double a0, a1;
            if (BETA) {
                const Lse2 s1 = lse2(own1, nbr);
                a1 = s1.mx + s1.l;
                own1 = (s1.mx + aB1) + s1.l;
                const Lse2 s0 = lse2(own0, (s1.mx + aL0) + s1.l);
                a0 = s0.mx + s0.l;
                own0 = (s0.mx + aB0) + s0.l;
                pass = (s0.mx + aL1) + s0.l;
            } else {
                const Lse2 s0 = lse2(own0, nbr);
                a0 = s0.mx + s0.l;
                own0 = (s0.mx + aB0) + s0.l;
                const Lse2 s1 = lse2(own1, (s0.mx + aL0) + s0.l);
                a1 = s1.mx + s1.l;
                own1 = (s1.mx + aB1) + s1.l;
                pass = (s1.mx + aL1) + s1.l;
            }
            buf_store_d(r_out, vo.c0, qi * p8, a0);
            buf_store_d(r_out, vo.c1, qi * p8, a1);
            if (HAS_OUT) {
                const double h = BETA ? a0 : pass;  // alpha hands on a + L(t,u); beta plain a
                if (CONC) ring_out[(k0 + j) & (kRing - 1)] = h;
                else buf_store_d(r_bo, vo_bo, (k0 + j) * 8, h);
            }
            const float2 nx0 = ring0[(j + 1) % kPF], nx1 = ring1[(j + 1) % kPF];
            aB0 = (double)nx0.x;
            aB1 = (double)nx1.x;
            if (BETA) {
                aL0 = aL0_next;
                aL0_next = (double)nx0.y;
                aL1 = (double)dpp_f32_or_zero<DPP_WAVE_SHR1>(nx1.y);
            } else {
                aL0 = (double)nx0.y;
                aL1 = (double)nx1.y;
            }
            ring0[j] = cn0;
            ring1[j] = cn1;
            qi += dq;
            mi += dq;
            __builtin_amdgcn_sched_barrier(0);
        }
        if (CONC) keep_order();
        if (CONC && HAS_OUT) __hip_atomic_store(rout.produced, k0 + kPF, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (CONC && HAS_IN) __hip_atomic_store(rin.consumed, k0 + kPF, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (CONC && HAS_OUT) __hip_atomic_store(rout.produced, 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (CONC && HAS_IN) __hip_atomic_store(rin.consumed, 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

template <bool BETA>
__device__ __forceinline__ bool lin_dispatch(bool has_in, bool has_out, int T, int nl, int seed_col, int in_shift,
                                             int out_shift, const float2* lp, double* out, int* sc, Ring rin,
                                             Ring rout, const WaitCtl status) {
    if (has_in && has_out) return sweep_strip_lin<BETA, true, true>(T, nl, seed_col, in_shift, out_shift, lp, out, sc, rin, rout, status);
    if (has_in) return sweep_strip_lin<BETA, true, false>(T, nl, seed_col, in_shift, out_shift, lp, out, sc, rin, rout, status);
    if (has_out) return sweep_strip_lin<BETA, false, true>(T, nl, seed_col, in_shift, out_shift, lp, out, sc, rin, rout, status);
    return sweep_strip_lin<BETA, false, false>(T, nl, seed_col, in_shift, out_shift, lp, out, sc, rin, rout, status);
}

template <bool BETA, bool CONC>
__device__ __forceinline__ void log_dispatch(bool has_in, bool has_out, int T, int nl, int seed_col, int in_shift,
                                             int out_shift, const float2* lp, double* out, const double* bi,
                                             double* bo, Ring rin, Ring rout, const WaitCtl status) {
    if (has_in && has_out) sweep_strip_log<BETA, true, true, CONC>(T, nl, seed_col, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else if (has_in) sweep_strip_log<BETA, true, false, CONC>(T, nl, seed_col, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else if (has_out) sweep_strip_log<BETA, false, true, CONC>(T, nl, seed_col, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
    else sweep_strip_log<BETA, false, false, CONC>(T, nl, seed_col, in_shift, out_shift, lp, out, bi, bo, rin, rout, status);
}

// One workgroup per (sequence, direction), W waves.  A sequence of S <= W strips is walked by S
// waves at once, each strip trailing the one that feeds it by the steps the diagonal order
// demands plus one block of kPF steps of slack; the boundary values travel through LDS rings
// guarded by two progress counters per ring.  A wave only ever waits for the wave of the strip
// before it (values) or after it (ring space), and the first strip waits for nobody, so the chain
// always drains; every wait is bounded all the same.  Longer sequences (S > W, 2048 labels or more)
// fall back to one wave walking the strips in turn, in the log domain, with the streams in global
// memory.
constexpr int kMaxWaves = 16;  // strips of a sequence that are ever walked at once

// Two shapes.  Up to eight strips (label sequences below 1024, all a batch normally holds): at most
// two waves share a SIMD, which lets a wave keep the prefetch ring and the walk's state in up to
// 256 registers.  Nine to sixteen strips: sixteen waves per workgroup, four per SIMD, 128 registers
// each; the host picks the shape from the max_u of the call, so a sequence of S <= 16 strips
// always finds S waves.
template <int MAXW>
__global__ __launch_bounds__(MAXW * 64) __attribute__((amdgpu_waves_per_eu(1, MAXW / 4))) void k_lattice(
    const int* __restrict__ lx, const int* __restrict__ ly, const i64* __restrict__ pad_off,
    const i64* __restrict__ bnd_off, int* seqmode, const LpStore lp, double* alpha,
    double* beta, int* scale_a, int* scale_b, double* bnd_a, double* bnd_b, int beta_only, int spin_limit,
    int* status_word) {
    __shared__ double s_ring[MAXW - 1][2 * kRing + 64];
    __shared__ int s_scale[MAXW - 1][kRing / kPF];
    __shared__ int s_produced[MAXW];
    __shared__ int s_consumed[MAXW];
    __shared__ volatile int s_unsafe;
    __shared__ int s_abort;
    const int n = blockIdx.x;
    const int dir = beta_only ? 1 : (int)blockIdx.y;
    const int W = blockDim.x >> 6;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (threadIdx.x < MAXW) {
        s_produced[threadIdx.x] = 0;
        s_consumed[threadIdx.x] = 0;
    }
    if (threadIdx.x == 0) { s_unsafe = 0; s_abort = 0; }
    __syncthreads();
    WaitCtl status;  // handed to every walk of this workgroup
    status.status = status_word; status.abort = &s_abort; status.limit = spin_limit;
    const i64 pad = pad_off[n];
    if (pad < 0) return;
    const int T = lx[n], U = ly[n];
    const int Up = U + 1;
    const int S = (int)strip_count(Up);
    const i64 full_strip = strip_rows(T, kStripCols) * kStripCols;
    double* out = dir ? beta : alpha;
    int* scale = dir ? scale_b : scale_a;
    const int nl_last = Up - ((S - 1) << kStripShift);
    Ring none;
    none.slots = nullptr; none.scales = nullptr; none.produced = nullptr; none.consumed = nullptr;

    const bool concurrent = S <= W;
    const bool linear = concurrent && (seqmode[n] & 1) == 0;  // what the gather pass found about the log-probs
    if (concurrent) {
        // position p in the order of the walk: alpha strip p, beta strip S-1-p
        const bool active = w < S;
        const int p = active ? w : 0;
        const int s = dir ? S - 1 - p : p;
        const int nl = s == S - 1 ? nl_last : kStripCols;
        const i64 base = pad + (i64)s * full_strip;
        const bool has_in = p > 0, has_out = p < S - 1;
        Ring rin = none, rout = none;
        if (has_in) { rin.slots = s_ring[p - 1]; rin.scales = s_scale[p - 1]; rin.produced = &s_produced[p - 1]; rin.consumed = &s_consumed[p - 1]; }
        if (has_out) { rout.slots = s_ring[p]; rout.scales = s_scale[p]; rout.produced = &s_produced[p]; rout.consumed = &s_consumed[p]; }
        // alpha: the feeding strip's edge lane 63 trails its first lane by 63 steps; beta: the
        // feeding strip is s+1 and its edge lane 0 trails by its lanes - 1; likewise for the strip fed
        const int in_shift = dir ? (int)strip_lanes(s + 1 == S - 1 ? nl_last : kStripCols) - 1 : 63;
        const int out_shift = dir ? (int)strip_lanes(nl) - 1 : 63;
        // alpha starts in cell (0,0), beta in cell (T-1,U)
        const int seed_col = dir ? (s == S - 1 ? nl - 1 : -1) : (s == 0 ? 0 : -1);
        if (!linear) {
            if (active) {
                if (dir == 0) log_dispatch<false, true>(has_in, has_out, T, nl, seed_col, in_shift, out_shift, lp.l + base, out + base, nullptr, nullptr, rin, rout, status);
                else log_dispatch<true, true>(has_in, has_out, T, nl, seed_col, in_shift, out_shift, lp.l + base, out + base, nullptr, nullptr, rin, rout, status);
            }
            __syncthreads();
            // a hand-over that never came: the lattice is incomplete, the sequence's cost becomes NaN
            if (s_abort != 0 && threadIdx.x == 0) raise_flag(&seqmode[n], kSeqPoisoned);
            return;
        }
        bool safe = true;
        if (active) {
            int* sc = scale + (base >> 4);
            safe = dir == 0 ? lin_dispatch<false>(has_in, has_out, T, nl, seed_col, in_shift, out_shift, lp.p + base, out + base, sc, rin, rout, status)
                            : lin_dispatch<true>(has_in, has_out, T, nl, seed_col, in_shift, out_shift, lp.p + base, out + base, sc, rin, rout, status);
        }
        if (!safe && (threadIdx.x & 63) == 0) s_unsafe = 1;
        __syncthreads();
        if (s_abort != 0) {
            if (threadIdx.x == 0) raise_flag(&seqmode[n], kSeqPoisoned);
            return;
        }
        if (s_unsafe == 0 || w != 0) return;
        // Some strip of this direction left the range the linear walk is exact in: wave 0 walks
        // the whole direction again, strip by strip, in the log domain (below).
        if (threadIdx.x == 0) atomicOr(&seqmode[n], dir ? 4 : 2);
    }

    if (w != 0) return;
    double* bnd = (dir ? bnd_b : bnd_a) + bnd_off[n];
    const i64 bstride = (i64)T + kBndPad;
    for (int p = 0; p < S; ++p) {
        const int s = dir ? S - 1 - p : p;
        const int nl = s == S - 1 ? nl_last : kStripCols;
        const i64 base = pad + (i64)s * full_strip;
        const bool has_in = p > 0, has_out = p < S - 1;
        // stream j runs between the strips at positions j and j+1 of the walk
        const double* bi = bnd + (i64)(p > 0 ? p - 1 : 0) * bstride;
        double* bo = bnd + (i64)p * bstride;
        const int in_shift = dir ? (int)strip_lanes(s + 1 == S - 1 ? nl_last : kStripCols) - 1 : 63;
        const int seed_col = dir ? (s == S - 1 ? nl - 1 : -1) : (s == 0 ? 0 : -1);
        if (dir == 0) log_dispatch<false, false>(has_in, has_out, T, nl, seed_col, in_shift, 63, lp.l + base, out + base, bi, bo, none, none, status);
        else log_dispatch<true, false>(has_in, has_out, T, nl, seed_col, in_shift, (int)strip_lanes(nl) - 1, lp.l + base, out + base, bi, bo, none, none, status);
        __threadfence_block();
    }
}

// Polls a wait inside k_lattice may spend; settable from the host so that the give-up path can be
// exercised (with a limit of 1 a strip that has to wait for its feeder gives up at once, and every
// wave still leaves the kernel normally).
static std::atomic<int> g_wait_limit{kSpinLimit};
void set_wait_limit(int polls) { g_wait_limit.store(polls > 0 ? polls : kSpinLimit, std::memory_order_relaxed); }
static int wait_limit() { return g_wait_limit.load(std::memory_order_relaxed); }

// one wave per strip of the longest label sequence the call admits, up to the concurrent limit
static int lattice_waves(const Batch& b) {
    const i64 strips = strip_count(b.max_u + 1);
    return (int)(strips < kMaxWaves ? (strips < 1 ? 1 : strips) : kMaxWaves);
}

int launch_lattice(const Batch& b, const Workspace& ws, bool beta_only) {
    if (b.N == 0) return CWR_OK;
    dim3 grid((unsigned)b.N, beta_only ? 1 : 2);
    const int waves = lattice_waves(b);
    if (waves <= 8)
        CWR_LAUNCH(k_lattice<8>, grid, dim3(waves * 64), 0, b.stream, b.lx, b.ly, ws.pad_off, ws.bnd_off, ws.seqmode,
                   ws.lp, ws.alpha, ws.beta, ws.scale_a, ws.scale_b, ws.bnd_a, ws.bnd_b, beta_only ? 1 : 0,
                   wait_limit(), b.status);
    else
        CWR_LAUNCH(k_lattice<16>, grid, dim3(waves * 64), 0, b.stream, b.lx, b.ly, ws.pad_off, ws.bnd_off, ws.seqmode,
                   ws.lp, ws.alpha, ws.beta, ws.scale_a, ws.scale_b, ws.bnd_a, ws.bnd_b, beta_only ? 1 : 0,
                   wait_limit(), b.status);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// per-row gradient w.r.t. the gathered log-probs, and the costs
// ---------------------------------------------------------------------------------------------
// Walk-mode word of a sequence: bit 0 = the gather pass found log-probs the linear walk cannot
// carry; bit 1 / bit 2 = the alpha / beta walk left the range it is exact in and was done again in
// the log domain.  More strips than a workgroup has waves always means the log domain.
__device__ __forceinline__ bool linear_alpha(int mode, int S) { return (mode & 3) == 0 && S <= kMaxWaves; }
__device__ __forceinline__ bool linear_beta(int mode, int S) { return (mode & 5) == 0 && S <= kMaxWaves; }

// Base-2 logarithm of the lattice value stored for cell (t,u): either stored as such (log walk),
// or as value * 2^C with C recorded per lane and block of kPF steps of the strip's walk (linear walk).
struct LatticeView {
    const double* v;
    const int* scale;
    i64 pad;
    int T, Up;
    bool linear, beta;
    // where the scale of the value that lane l of the `lanes`-lane strip starting at slot `base`
    // wrote at step k of its walk is kept
    __device__ __forceinline__ i64 scale_index(i64 base, int k, int lanes, int l) const {
        return (base >> 4) + (i64)(k / kPF) * lanes + l;
    }
    // in two steps (load, convert), so that a caller can have many loads in flight before it converts
    __device__ __forceinline__ double convert(double x, int C) const {
        if (!linear) return x;
        // log2 x = exponent + log2(mantissa), mantissa in [0.5, 1)
        const int ex = __builtin_amdgcn_frexp_exp(x);
        const float mant = (float)__builtin_amdgcn_frexp_mant(x);
        return x == 0.0 ? -INFINITY : (double)(ex - C) + (double)fast_log2(mant);
    }
    __device__ __forceinline__ double log2_at(int t, int u) const {
        const i64 slot = pad + lattice_slot(t, u, T, Up);
        const double x = v[slot];
        if (!linear) return x;
        const int s = u >> kStripShift, l = (u & (kStripCols - 1)) >> 1;
        const int nl = Up - (s << kStripShift) < kStripCols ? Up - (s << kStripShift) : kStripCols;
        const int lanes = (int)strip_lanes(nl);
        const int q = t + l;
        const int k = beta ? (T + lanes - 2 - q) : q;
        const i64 base = pad + (i64)s * strip_rows(T, kStripCols) * kStripCols;
        return convert(x, scale[scale_index(base, k, lanes, l)]);
    }
};

// Sum and mean of the N costs (cwarp_rnnt/__init__.py:66-71), by the wave that writes the last
// of them: every writer counts itself in after making its cost visible, and the wave that sees
// the count complete adds all N up in a fixed order (lane i takes costs i, i+64, ...; then a
// butterfly), so the result does not depend on which wave came last.  Called by whole waves.
__device__ __forceinline__ void finish_costs(bool wrote, int N, float* costs, float* reduced, int* status) {
    if (!reduced) return;
    bool last = false;
    if (wrote) {
        __threadfence();
        last = atomicAdd(&status[2], 1) == status[1] - 1;
    }
    if (__ballot(last) == 0) return;
    __threadfence();
    const int lane = threadIdx.x & 63;
    double s = 0.0;
    for (int i = lane; i < N; i += 64)
        s += (double)__hip_atomic_load(&costs[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int m = 1; m < 64; m <<= 1) s += __shfl_xor(s, m);
    if (lane == 0) {
        reduced[0] = (float)s;
        reduced[1] = (float)(s / (double)N);
    }
}

// One wave per chunk: kFillSlots consecutive slots of the cell rows of one strip of one sequence.
// Which sequence and strip is the same for the whole wave, so the search through the chunk offsets
// and the strip's geometry run once per wave on the scalar unit; a lane takes every 64th slot of the
// chunk, reads alpha, beta and the cell records at consecutive addresses (the strip layout is
// diagonal to the row order) and scatters the 8-byte results to the row order.  The successors of
// cell (t,u) sit close by: (t+1,u) one strip row further in the same column; (t,u+1) in the next
// slot for a lane's first column, one strip row further for its second; only the last column of a
// strip looks into the next strip.  The grid is fixed; waves stride over the chunks, whose number
// only the device knows.  A poisoned sequence (bad label, lattice wait that ran out) gets zero
// gradients next to its NaN cost.
constexpr int kFillPasses = kFillSlots / 64;

__global__ __launch_bounds__(256) void k_fill(const int* __restrict__ lx, const int* __restrict__ ly,
                                               const i64* __restrict__ row_off,
                                               const i64* __restrict__ pad_off,
                                               const i64* __restrict__ fill_off,
                                               const int* __restrict__ seqmode, int N, i64 R,
                                               const float2* __restrict__ lpl,
                                               const double* __restrict__ alpha, const double* __restrict__ beta,
                                               const int* __restrict__ scale_a, const int* __restrict__ scale_b,
                                               float2* __restrict__ grads, float* costs, float* reduced,
                                               int* status) {
    const int lane = threadIdx.x & 63;
    const i64 total = fill_off[N];
    const i64 nwaves = (i64)gridDim.x * 4;
    const i64 first = (i64)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    // Up to 64 sequences: lane i fetches everything about sequence i up front; one ballot then places
    // a chunk and cross-lane reads hand out its sequence's values (a search through memory followed
    // by the per-sequence loads would be two more rounds of dependent loads in front of everything
    // else the wave does, and this kernel is made of such rounds).
    const bool tables = N <= 64;
    i64 t_fill = 0x7fffffffffffffffLL, t_pad = -1, t_row = 0;
    int t_T = 0, t_U = 0, t_mode = 0;
    if (tables && lane < N) {
        t_fill = fill_off[lane]; t_pad = pad_off[lane]; t_row = row_off[lane];
        t_T = lx[lane]; t_U = ly[lane]; t_mode = seqmode[lane];
    }
    auto lane_i64 = [](i64 v, int i) {
        return ((i64)__builtin_amdgcn_readlane((int)(v >> 32), i) << 32) | (unsigned)__builtin_amdgcn_readlane((int)v, i);
    };
    for (i64 c = first; c < total; c += nwaves) {
        // the sequence of chunk c: fill_off[n] <= c < fill_off[n+1]
        int n;
        i64 pad, roff, f0;
        int T, U, mode;
        if (tables) {
            n = __popcll(__ballot(t_fill <= c)) - 1;
            pad = lane_i64(t_pad, n); roff = lane_i64(t_row, n); f0 = lane_i64(t_fill, n);
            T = __builtin_amdgcn_readlane(t_T, n); U = __builtin_amdgcn_readlane(t_U, n);
            mode = __builtin_amdgcn_readlane(t_mode, n);
        } else {
            int lo = 0, hi = N;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (fill_off[mid] <= c) lo = mid; else hi = mid;
            }
            n = lo;
            pad = pad_off[n]; roff = row_off[n]; f0 = fill_off[n];
            T = lx[n]; U = ly[n]; mode = seqmode[n];
        }
        bool wrote = false;
        if (pad >= 0) {
            const int Up = U + 1;
            const int S = (int)strip_count(Up);
            const unsigned per_full = (unsigned)strip_chunks(T, kStripCols);
            const unsigned local = (unsigned)(c - f0);
            unsigned s = local / per_full;
            s = s < (unsigned)(S - 1) ? s : (unsigned)(S - 1);
            const int nl = (int)s == S - 1 ? Up - ((int)s << kStripShift) : kStripCols;
            const int lanes = (int)strip_lanes(nl);
            const int Q = T + lanes - 1;  // rows of the strip that hold cells
            const i64 full = strip_rows(T, kStripCols) * kStripCols;
            const i64 base = pad + (i64)s * full;
            // first slot of the chunk, counted from the strip's first cell row, as (row, column)
            const unsigned i0 = (local - s * per_full) * (unsigned)kFillSlots;
            const int pitch = (int)strip_pitch(nl);  // slots per row; one of them padding when nl is odd
            const unsigned q_first = i0 / (unsigned)pitch;
            const int c_first = (int)(i0 - q_first * (unsigned)pitch);
            const float inv_pitch = 1.0f / (float)pitch;
            // the strip after this one, for the cells of this strip's last column
            const int nl2 = (int)s + 1 < S ? ((int)s + 2 == S ? Up - (((int)s + 1) << kStripShift) : kStripCols) : 1;
            const int lanes2 = (int)strip_lanes(nl2), pitch2 = (int)strip_pitch(nl2);
            const i64 base2 = base + full;
            LatticeView A, Bv;
            A.v = alpha; A.scale = scale_a; A.pad = pad; A.T = T; A.Up = Up; A.linear = linear_alpha(mode, S); A.beta = false;
            Bv.v = beta; Bv.scale = scale_b; Bv.pad = pad; Bv.T = T; Bv.Up = Up; Bv.linear = linear_beta(mode, S); Bv.beta = true;
            const double b00 = Bv.log2_at(0, 0);  // all values are base-2 logarithms
            // every pass's loads go out before any of them is used: lanes without a cell read
            // the strip's first cell instead and drop the result
            struct Raw { double a, bd, bn; float2 cell; int ca, cbd, cbn; int t, u; bool ok; };
            Raw raw[kFillPasses];
#pragma unroll
            for (int pass = 0; pass < kFillPasses; ++pass) {
                Raw& w = raw[pass];
                // slot c_first + 64*pass + lane of the rows from q_first on; at most
                // pitch + kFillSlots < 2^9, so the quotient by the pitch is exact in fp32
                const int il = c_first + pass * 64 + lane;
                const int dqr = (int)(((float)il + 0.5f) * inv_pitch);
                const int q = (int)q_first + dqr;
                const int col = il - dqr * pitch;
                const int l = col >> 1;
                const int t = q - l;
                w.ok = q < Q && col < nl && t >= 0 && t < T;
                const int qs = w.ok ? q : 0, cs = w.ok ? col : 0, ls = w.ok ? l : 0;
                w.t = qs - ls;
                w.u = ((int)s << kStripShift) + cs;
                const i64 slot = base + (i64)(qs + kRowShift) * pitch + cs;
                // (t+1,u): same column, next strip row, written at step Q-2-q of the beta walk.
                // (t,u+1): the lane's second column in the same row (step Q-1-q), or the next lane's
                // first column one row further (step Q-2-q), or column 0 of the next strip in row t.
                const bool second = (cs & 1) != 0;
                const bool inside = cs + 1 < nl || !w.ok || (int)s + 1 >= S;
                const i64 slot_n = inside ? (second ? slot + pitch + 1 : slot + 1) : base2 + (i64)(w.t + kRowShift) * pitch2;
                const int kb_d = max(Q - 2 - qs, 0);
                w.a = alpha[slot];
                w.cell = lpl[slot];
                w.bd = beta[slot + pitch];
                w.bn = beta[slot_n];
                w.ca = w.cbd = w.cbn = 0;
                if (A.linear) w.ca = scale_a[A.scale_index(base, qs, lanes, ls)];
                if (Bv.linear) {
                    w.cbd = scale_b[Bv.scale_index(base, kb_d, lanes, ls)];
                    w.cbn = scale_b[inside ? (second ? Bv.scale_index(base, kb_d, lanes, min(ls + 1, lanes - 1))
                                                     : Bv.scale_index(base, Q - 1 - qs, lanes, ls))
                                           : Bv.scale_index(base2, max(T + lanes2 - 2 - w.t, 0), lanes2, 0)];
                }
            }
            const bool poisoned = (mode & kSeqPoisoned) != 0;
#pragma unroll
            for (int pass = 0; pass < kFillPasses; ++pass) {
                const Raw& w = raw[pass];
                const int t = w.t, u = w.u;
                const i64 r = roff + (i64)t * Up + u;
                if (!w.ok || r >= R) continue;
                const double a = A.convert(w.a, w.ca);
                float gb = 0.f, gl = 0.f;
                if (t < T - 1) gb = -fast_exp2((float)(a + Bv.convert(w.bd, w.cbd) + (double)w.cell.x - b00));
                else if (u == U) gb = -fast_exp2((float)(a + (double)w.cell.x - b00));
                if (u < U) gl = -fast_exp2((float)(a + Bv.convert(w.bn, w.cbn) + (double)w.cell.y - b00));
                grads[r] = poisoned ? make_float2(0.f, 0.f) : make_float2(gb, gl);
                if (t == T - 1 && u == U) {
                    float cost;
                    if (cost_rule(a + (double)w.cell.x, b00, &cost)) raise_flag(status, CWR_FLAG_FB_MISMATCH);
                    costs[n] = poisoned ? __int_as_float(0x7fc00000) : cost;
                    wrote = true;
                }
            }
        }
        finish_costs(wrote, N, costs, reduced, status);
    }
}

// Waves k_fill is launched with: one GPU full of them (8 per SIMD), never more than the chunks a
// batch of R rows in N sequences can have (a strip's cell rows hold its cells and, per lane, one
// row of padding; every strip ends with one partly filled chunk).
int launch_fill(const Batch& b, const Workspace& ws, const int* rowinfo, float* grads, float* costs,
                float* reduced) {
    if (b.R == 0) return CWR_OK;
    const i64 strips = strip_count(b.max_u + 1);
    i64 waves = 2 * b.R / kFillSlots + (i64)b.N * strips * (64 * kStripCols / kFillSlots + 1) + 1;
    if (waves > 8192) waves = 8192;
    CWR_LAUNCH(k_fill, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, b.stream, b.lx, b.ly, b.row_off,
                       ws.pad_off, ws.fill_off, ws.seqmode, b.N, b.R, ws.lp.l, ws.alpha, ws.beta, ws.scale_a,
                       ws.scale_b, reinterpret_cast<float2*>(grads), costs, reduced, b.status);
    (void)rowinfo;  // rows of skipped sequences were given their zero record by the gather pass
    return check_launch();
}

__global__ __launch_bounds__(64) void k_cost_from_beta(const int* __restrict__ lx, const int* __restrict__ ly,
                                                       const i64* __restrict__ pad_off,
                                                       const int* __restrict__ seqmode, int N,
                                                       const double* __restrict__ beta,
                                                       const int* __restrict__ scale_b, float* costs,
                                                       float* reduced, int* status) {
    const int n = blockIdx.x * 64 + threadIdx.x;
    bool wrote = false;
    const i64 pad = n < N ? pad_off[n] : -1;
    if (pad >= 0) {  // else: NaN already set by k_offsets
        LatticeView Bv;
        Bv.v = beta; Bv.scale = scale_b; Bv.pad = pad; Bv.T = lx[n]; Bv.Up = ly[n] + 1; Bv.beta = true;
        const int mode = seqmode[n];
        Bv.linear = linear_beta(mode, (int)strip_count(Bv.Up));
        costs[n] = (mode & kSeqPoisoned) ? __int_as_float(0x7fc00000) : (float)(-Bv.log2_at(0, 0) * (double)kLn2);
        wrote = true;
    }
    finish_costs(wrote, N, costs, reduced, status);
}

int launch_cost_from_beta(const Batch& b, const Workspace& ws, float* costs, float* reduced) {
    if (b.N == 0) return CWR_OK;
    CWR_LAUNCH(k_cost_from_beta, dim3((unsigned)((b.N + 63) / 64)), dim3(64), 0, b.stream, b.lx,
                       b.ly, ws.pad_off, ws.seqmode, b.N, ws.beta, ws.scale_b, costs, reduced, b.status);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// export of alpha / beta as padded arrays of natural logarithms
// ---------------------------------------------------------------------------------------------
// What the reference hands back from its forward call (cwarp_cuda_rnnt_kernel.cu:383-384, 399-400,
// 496): (N, T_pad, Up_pad) arrays, zero outside a sequence's own T x (U+1) lattice.
__global__ __launch_bounds__(256) void k_export(const int* __restrict__ lx, const int* __restrict__ ly,
                                                 const i64* __restrict__ pad_off,
                                                 const int* __restrict__ seqmode, int N, i64 T_pad, i64 Up_pad,
                                                 const double* __restrict__ alpha,
                                                 const double* __restrict__ beta,
                                                 const int* __restrict__ scale_a, const int* __restrict__ scale_b,
                                                 double* __restrict__ alphas_out, double* __restrict__ betas_out) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    const i64 per_seq = T_pad * Up_pad;
    if (i >= (i64)N * per_seq) return;
    const int n = (int)(i / per_seq);
    const i64 rem = i - (i64)n * per_seq;
    const int t = (int)(rem / Up_pad), u = (int)(rem - (i64)t * Up_pad);
    const i64 pad = pad_off[n];
    const int T = lx[n], Up = ly[n] + 1;
    double a = 0.0, b = 0.0;
    if (pad >= 0 && t < T && u < Up) {
        LatticeView A, Bv;
        const int mode = seqmode[n], S = (int)strip_count(Up);
        A.v = alpha; A.scale = scale_a; A.pad = pad; A.T = T; A.Up = Up; A.linear = linear_alpha(mode, S); A.beta = false;
        Bv.v = beta; Bv.scale = scale_b; Bv.pad = pad; Bv.T = T; Bv.Up = Up; Bv.linear = linear_beta(mode, S); Bv.beta = true;
        if (alphas_out) a = A.log2_at(t, u) * 0.6931471805599453;
        b = Bv.log2_at(t, u) * 0.6931471805599453;
    }
    if (alphas_out) alphas_out[i] = a;
    if (betas_out) betas_out[i] = b;
}

int launch_export(const int* lx, const int* ly, int N, i64 T_pad, i64 Up_pad, const Workspace& ws,
                  double* alphas_out, double* betas_out, hipStream_t stream) {
    const i64 total = (i64)N * T_pad * Up_pad;
    if (total == 0) return CWR_OK;
    CWR_LAUNCH(k_export, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, lx, ly, ws.pad_off,
                       ws.seqmode, N, T_pad, Up_pad, ws.alpha, ws.beta, ws.scale_a, ws.scale_b, alphas_out,
                       betas_out);
    return check_launch();
}

}  // namespace cwr
