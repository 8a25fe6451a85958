// Padded <-> compact layout conversion of (.., V) rows.
//
// Replaces the 4-D input branch of cwarp_rnnt/__init__.py:52-59, which hands a padded joiner
// output (N, T, U+1, V) to the external `gather.cat`; here the rows of each sequence's own
// T_i x (U_i+1) sub-lattice are selected, in the order of test/test.py:44-46.  Rows move in
// 16-byte units (or element-sized units when rows are not 16-byte multiples).  pack walks the
// compact rows (k_pack_rows); unpack has to write every padded element and takes one workgroup
// per 256 units of one PADDED row, whose (n, t, u) comes straight from the grid (k_unpack).
//   pack:   compact[row_off[n] + t*(U_n+1) + u] = padded[n][t][u]      for t < T_n, u <= U_n
//   unpack: padded[n][t][u] = the same compact row, or zeros outside the sub-lattice (this is the
//           backward of pack: every element of the padded gradient is written, no memset pass)
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

template <typename U> struct Unit {
    static __device__ __forceinline__ U zero() { return U(0); }
    static __device__ __forceinline__ U load(const U* p) { return __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ void store(U* p, U v) { __builtin_nontemporal_store(v, p); }
};
typedef int v4i_t __attribute__((ext_vector_type(4)));
template <> struct Unit<v4i_t> {
    static __device__ __forceinline__ v4i_t zero() { v4i_t z = {0, 0, 0, 0}; return z; }
    static __device__ __forceinline__ v4i_t load(const v4i_t* p) { return __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ void store(v4i_t* p, v4i_t v) { store_streaming_16(p, v); }
};

// grid: x = (label position u, block of 4 chunks of 64 units), y = frame t, z = sequence n (relative
// to n0), so that no wave needs a 64-bit division and consecutive workgroups walk memory in order.
template <typename U>
__global__ __launch_bounds__(256) void k_unpack(const U* __restrict__ src, U* __restrict__ dst,
                                                 const int* __restrict__ lx, const int* __restrict__ ly,
                                                 const i64* __restrict__ row_off, int n0, int T_pad, int Up_pad,
                                                 i64 units_per_row, unsigned cblocks, i64 R) {
    const int lane = threadIdx.x & 63;
    const int n = n0 + (int)blockIdx.z;
    const int t = (int)blockIdx.y;
    const unsigned u = cblocks == 1 ? blockIdx.x : blockIdx.x / cblocks;
    const unsigned cb = blockIdx.x - u * cblocks;
    const int T = lx[n], Ul = ly[n];
    bool valid = T > 0 && Ul >= 0 && t < T && (int)u <= Ul;
    i64 crow = 0;
    if (valid) {
        crow = row_off[n] + (i64)t * ((i64)Ul + 1) + u;
        if (crow >= R) valid = false;  // lengths that do not add up to R: flagged by the offsets pass
    }
    const i64 unit = ((i64)cb * 4 + (threadIdx.x >> 6)) * 64 + lane;
    if (unit >= units_per_row) return;
    const i64 prow = ((i64)n * T_pad + t) * Up_pad + u;
    U v = Unit<U>::zero();
    if (valid) v = Unit<U>::load(src + crow * units_per_row + unit);
    Unit<U>::store(dst + prow * units_per_row + unit, v);
}

// pack, walking the COMPACT rows instead: a wave takes `rpw` consecutive rows (about 4 KiB), decodes
// the first on the scalar unit and steps through the others, so that only valid cells are visited
// however ragged the batch is (a padded grid is mostly empty workgroups then).

template <typename U>
__global__ __launch_bounds__(256) void k_pack_rows(const U* __restrict__ src, U* __restrict__ dst,
                                                    const int* __restrict__ lx, const int* __restrict__ ly,
                                                    const i64* __restrict__ row_off, int N, int T_pad, int Up_pad,
                                                    i64 units_per_row, i64 R, int rpw,
                                                    int* __restrict__ status) {
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const i64 r0 = ((i64)blockIdx.x * 4 + w) * rpw;
    if (r0 >= R) return;
    RowInfo ri = decode_row(r0, R, row_off, lx, ly, N);
    for (int k = 0; k < rpw; ++k) {
        const i64 r = r0 + k;
        if (r >= R) break;
        if (k > 0) {
            if (ri.n >= 0 && ri.u < ri.U) {
                ++ri.u;
            } else if (ri.n >= 0 && ri.t + 1 < ri.T) {
                ri.u = 0;
                ++ri.t;
            } else {
                ri = decode_row(r, R, row_off, lx, ly, N);
            }
        }
        U* pd = dst + r * units_per_row;
        bool source = ri.n >= 0;
        if (source && (ri.t >= T_pad || ri.u >= Up_pad)) {  // this cell lies outside the padded array
            if (status && lane == 0) raise_flag(status, CWR_FLAG_BAD_LENGTH);
            source = false;
        }
        if (!source) {  // a row nothing maps to is zeroed: the loss never sees uninitialised memory
            for (i64 j = lane; j < units_per_row; j += 64) Unit<U>::store(pd + j, Unit<U>::zero());
            continue;
        }
        const U* ps = src + (((i64)ri.n * T_pad + ri.t) * Up_pad + ri.u) * units_per_row;
#pragma unroll 4
        for (i64 j = lane; j < units_per_row; j += 64) Unit<U>::store(pd + j, Unit<U>::load(ps + j));
    }
}

template <typename U>
static int repack_as(const void* src, void* dst, const int* lx, const int* ly, const i64* row_off, i64 N, i64 T_pad,
                     i64 Up_pad, i64 units_per_row, i64 R, bool unpack, int* status, hipStream_t stream) {
    if (N == 0 || T_pad == 0 || Up_pad == 0) return CWR_OK;
    if (!unpack) {
        if (R == 0) return CWR_OK;
        const i64 row_bytes = units_per_row * (i64)sizeof(U);
        const int rpw = row_bytes >= 4096 ? 1 : (int)(4096 / row_bytes < 8 ? 4096 / row_bytes : 8);
        const i64 blocks = (R + 4 * rpw - 1) / (4 * rpw);
        if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
        CWR_LAUNCH((k_pack_rows<U>), dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<const U*>(src),
                           static_cast<U*>(dst), lx, ly, row_off, (int)N, (int)T_pad, (int)Up_pad, units_per_row, R,
                           rpw, status);
        return check_launch();
    }
    const i64 cblocks = (units_per_row + 255) / 256;
    if (T_pad > 65535 || Up_pad * cblocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
    for (i64 n0 = 0; n0 < N; n0 += 65535) {
        const i64 nz = N - n0 < 65535 ? N - n0 : 65535;
        dim3 grid((unsigned)(Up_pad * cblocks), (unsigned)T_pad, (unsigned)nz);
        CWR_LAUNCH((k_unpack<U>), grid, dim3(256), 0, stream, static_cast<const U*>(src),
                           static_cast<U*>(dst), lx, ly, row_off, (int)n0, (int)T_pad, (int)Up_pad,
                           units_per_row, (unsigned)cblocks, R);
        int rc = check_launch();
        if (rc != CWR_OK) return rc;
    }
    return CWR_OK;
}

int launch_repack(const void* src, void* dst, size_t esize, const int* lx, const int* ly, const i64* row_off, i64 N,
                  i64 T_pad, i64 Up_pad, i64 V, i64 R, bool unpack, int* status, hipStream_t stream) {
    const size_t row_bytes = (size_t)V * esize;
    const bool wide = row_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    if (wide) return repack_as<v4i_t>(src, dst, lx, ly, row_off, N, T_pad, Up_pad, (i64)(row_bytes / 16), R, unpack, status, stream);
    switch (esize) {
        case 2: return repack_as<unsigned short>(src, dst, lx, ly, row_off, N, T_pad, Up_pad, V, R, unpack, status, stream);
        case 4: return repack_as<unsigned int>(src, dst, lx, ly, row_off, N, T_pad, Up_pad, V, R, unpack, status, stream);
        case 8: return repack_as<unsigned long long>(src, dst, lx, ly, row_off, N, T_pad, Up_pad, V, R, unpack, status, stream);
    }
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
