// Compact joiner front: h[row(n,t,u), :] = act(f[n,t,:] + g[n,u,:]) for the cells of each
// sequence's own T_n x (U_n+1) lattice only, written straight in the compact row order that the
// loss consumes (test/test.py:44-46), and its backward
//   df[n,t,:] = sum_u dz[row(n,t,u), :]     dg[n,u,:] = sum_t dz[row(n,t,u), :]
// with dz = dh * act'(z), act' taken from the stored output (tanh: 1-h^2, relu: h > 0).
//
// The reference repository holds no joiner: its callers build the (N,T,U+1,H) broadcast sum in
// padded form and hand the padded logits to cwarp_rnnt/__init__.py:52-59.  Doing the sum for valid
// cells only never materialises the padded tensor; the linear layer that follows is a plain
// library GEMM over the (R,H) rows.
//
// All kernels work in 16-byte packs when rows allow it.  The forward pass walks the compact rows,
// one wave per row, and is bound by its (R,H) store; f and g rows are re-read from L2.  The backward
// kernels take their (n, t or u, column block) from the grid, so no wave divides.  Each backward sum is taken by one lane per column in a fixed order
// (deterministic, no atomics) and every element of df and dg is written, padding included.
#include "cwr_act.hpp"
#include "cwr_device.hpp"
#include "cwr_host.hpp"

namespace cwr {

typedef int v4i __attribute__((ext_vector_type(4)));

template <typename T, int VEC>
__device__ __forceinline__ PackT<T, VEC> ld(const T* p) { return *reinterpret_cast<const PackT<T, VEC>*>(p); }
template <typename T, int VEC>
__device__ __forceinline__ PackT<T, VEC> ld_stream(const T* p) {
    if constexpr (sizeof(T) * VEC == 16) {
        const v4i r = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
        PackT<T, VEC> o;
        __builtin_memcpy(&o, &r, 16);
        return o;
    } else {
        return *reinterpret_cast<const PackT<T, VEC>*>(p);
    }
}
template <typename T, int VEC>
__device__ __forceinline__ void st_stream(T* p, const PackT<T, VEC>& v) {
    if constexpr (sizeof(T) * VEC == 16) {
        v4i r;
        __builtin_memcpy(&r, &v, 16);
        store_streaming_16(p, r);
    } else {
        *reinterpret_cast<PackT<T, VEC>*>(p) = v;
    }
}

// A wave takes JoinRows<T>::n consecutive compact rows; the first row's (n, t, u) is decoded on the
// scalar unit and the following ones are stepped from it.  Only valid cells are visited, whatever
// the padding of f and g.
template <typename T> struct JoinRows { static constexpr int n = sizeof(T) == 2 ? 8 : 4; };  // 16-bit rows are half as long

template <typename T, int VEC, int ACT, bool FLAT>
__global__ __launch_bounds__(256) void k_join(const T* __restrict__ f, const T* __restrict__ g,
                                               const int* __restrict__ lx, const int* __restrict__ ly,
                                               const i64* __restrict__ row_off, int N, int T_pad, int Up_pad,
                                               int H, i64 R, T* __restrict__ out, int* __restrict__ status) {
    typedef typename Arith<T>::type A;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    constexpr int kJoinRows = JoinRows<T>::n;
    const i64 r0 = ((i64)blockIdx.x * 4 + w) * kJoinRows;
    if (r0 >= R) return;
    const int NV = H / VEC;
    // where the rows' operands start (element offsets; -1: no valid cell), on the scalar unit
    i64 fo[kJoinRows], go[kJoinRows];
    RowInfo ri = decode_row(r0, R, row_off, lx, ly, N);
#pragma unroll
    for (int k = 0; k < kJoinRows; ++k) {
        fo[k] = -1; go[k] = -1;  // -1: a row of the output that no valid cell maps to (it is zeroed)
        const i64 r = r0 + k;
        if (r >= R) { fo[k] = -2; continue; }  // -2: beyond the output
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
        if (ri.n < 0) continue;
        if (ri.t >= T_pad || ri.u >= Up_pad) {  // this cell lies outside the padded inputs
            if (status && lane == 0) raise_flag(status, CWR_FLAG_BAD_LENGTH);
            continue;
        }
        fo[k] = ((i64)ri.n * T_pad + ri.t) * H;
        go[k] = ((i64)ri.n * Up_pad + ri.u) * H;
    }
    if (!FLAT) {  // rows of whole multiples of 64 packs: row after row, addresses on the scalar unit
#pragma unroll
        for (int k = 0; k < kJoinRows; ++k) {
            if (fo[k] == -2) continue;
            if (fo[k] < 0) {  // no uninitialised row ever reaches the output layer that follows
                PackT<T, VEC> z;
#pragma unroll
                for (int i = 0; i < VEC; ++i) z.e[i] = Arith<T>::down(A(0));
                for (int j = lane; j < NV; j += 64) st_stream<T, VEC>(out + (r0 + k) * H + j * VEC, z);
                continue;
            }
            const T* pf = f + fo[k];
            const T* pg = g + go[k];
            T* po = out + (r0 + k) * H;
#pragma unroll 2
            for (int j = lane; j < NV; j += 64) {
                const PackT<T, VEC> a = ld<T, VEC>(pf + j * VEC);
                const PackT<T, VEC> b = ld<T, VEC>(pg + j * VEC);
                PackT<T, VEC> o;
#pragma unroll
                for (int i = 0; i < VEC; ++i)
                    o.e[i] = Arith<T>::down(activate<ACT, T>(Arith<T>::up(a.e[i]) + Arith<T>::up(b.e[i])));
                st_stream<T, VEC>(po + j * VEC, o);
            }
        }
        return;
    }
    // otherwise the packs of the wave's rows form one index space, so that every lane stays busy
    const int total = kJoinRows * NV;
#pragma unroll 2
    for (int idx = lane; idx < total; idx += 64) {
        int k = 0;
        i64 a_at = fo[0], b_at = go[0];
#pragma unroll
        for (int q = 1; q < kJoinRows; ++q) {
            const bool past = idx >= q * NV;
            k += past ? 1 : 0;
            a_at = past ? fo[q] : a_at;
            b_at = past ? go[q] : b_at;
        }
        if (a_at == -2) continue;
        const int col = (idx - k * NV) * VEC;
        if (a_at < 0) {
            PackT<T, VEC> z;
#pragma unroll
            for (int i = 0; i < VEC; ++i) z.e[i] = Arith<T>::down(A(0));
            st_stream<T, VEC>(out + (r0 + k) * H + col, z);
            continue;
        }
        const PackT<T, VEC> a = ld<T, VEC>(f + a_at + col);
        const PackT<T, VEC> b = ld<T, VEC>(g + b_at + col);
        PackT<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            o.e[i] = Arith<T>::down(activate<ACT, T>(Arith<T>::up(a.e[i]) + Arith<T>::up(b.e[i])));
        st_stream<T, VEC>(out + (r0 + k) * H + col, o);
    }
}

// df: grid x = block of 256 packs, y = t, z = sequence.  One lane sums its columns over u; the rows
// (t, 0..U) are contiguous in the compact layout.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(256) void k_join_bwd_f(const T* __restrict__ dh, const T* __restrict__ h,
                                                     const int* __restrict__ lx, const int* __restrict__ ly,
                                                     const i64* __restrict__ row_off, int n0, int T_pad, int H,
                                                     i64 R, T* __restrict__ df) {
    typedef typename Arith<T>::type A;
    const int n = n0 + (int)blockIdx.z;
    const int t = (int)blockIdx.y;
    const int col = ((int)blockIdx.x * 256 + (int)threadIdx.x) * VEC;
    if (col >= H) return;
    const int Tn = lx[n], Un = ly[n];
    A acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = A(0);
    if (Tn > 0 && Un >= 0 && t < Tn) {
        const i64 r0 = row_off[n] + (i64)t * ((i64)Un + 1);
        i64 cnt = (i64)Un + 1;
        if (r0 + cnt > R) cnt = R - r0;
        const T* pd = dh + r0 * H + col;
        const T* ph = h + r0 * H + col;
        // loads in flight per lane: twice as many rows at a time where there is no h to read beside dh
        constexpr int kAhead = ACT == kActNone ? 8 : 4;
#pragma unroll kAhead
        for (i64 u = 0; u < cnt; ++u) {
            const PackT<T, VEC> d = ld_stream<T, VEC>(pd + u * H);
            PackT<T, VEC> o;
            if (ACT != kActNone) o = ld_stream<T, VEC>(ph + u * H);
#pragma unroll
            for (int i = 0; i < VEC; ++i)
                acc[i] += act_grad<ACT, A>(Arith<T>::up(d.e[i]), ACT != kActNone ? Arith<T>::up(o.e[i]) : A(0));
        }
    }
    PackT<T, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.e[i] = Arith<T>::down(acc[i]);
    *reinterpret_cast<PackT<T, VEC>*>(df + ((i64)n * T_pad + t) * H + col) = r;
}

// dg: grid x = block of 256 packs, y = u, z = sequence.  One lane sums its columns over t; the rows
// (0..T-1, u) lie (U+1) rows apart, each visit a contiguous piece of one row per wave.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(256) void k_join_bwd_g(const T* __restrict__ dh, const T* __restrict__ h,
                                                     const int* __restrict__ lx, const int* __restrict__ ly,
                                                     const i64* __restrict__ row_off, int n0, int Up_pad, int H,
                                                     i64 R, T* __restrict__ dg) {
    typedef typename Arith<T>::type A;
    const int n = n0 + (int)blockIdx.z;
    const int u = (int)blockIdx.y;
    const int col = ((int)blockIdx.x * 256 + (int)threadIdx.x) * VEC;
    if (col >= H) return;
    const int Tn = lx[n], Un = ly[n];
    A acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = A(0);
    if (Tn > 0 && Un >= 0 && u <= Un) {
        const i64 r0 = row_off[n] + u;
        const i64 step = (i64)Un + 1;
        i64 cnt = Tn;
        if (r0 + (cnt - 1) * step >= R) cnt = r0 < R ? (R - 1 - r0) / step + 1 : 0;
        const T* pd = dh + r0 * H + col;
        const T* ph = h + r0 * H + col;
        const i64 stride = step * H;
        constexpr int kAhead = ACT == kActNone ? 16 : 8;
#pragma unroll kAhead
        for (i64 t = 0; t < cnt; ++t) {
            const PackT<T, VEC> d = ld<T, VEC>(pd + t * stride);
            PackT<T, VEC> o;
            if (ACT != kActNone) o = ld<T, VEC>(ph + t * stride);
#pragma unroll
            for (int i = 0; i < VEC; ++i)
                acc[i] += act_grad<ACT, A>(Arith<T>::up(d.e[i]), ACT != kActNone ? Arith<T>::up(o.e[i]) : A(0));
        }
    }
    PackT<T, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.e[i] = Arith<T>::down(acc[i]);
    *reinterpret_cast<PackT<T, VEC>*>(dg + ((i64)n * Up_pad + u) * H + col) = r;
}

struct JoinArgs {
    const void *a, *b;  // forward: f, g; backward: dh, h
    void *o1, *o2;      // forward: out; backward: df, dg
    const int *lx, *ly;
    const i64* row_off;
    i64 N, T_pad, Up_pad, H, R;
    int* status;
    hipStream_t stream;
};

template <typename T, int VEC, int ACT>
static int join_launch(const JoinArgs& j, bool backward) {
    if (!backward) {
        if (j.R == 0 || j.T_pad == 0 || j.Up_pad == 0) return CWR_OK;
        constexpr int kJoinRows = JoinRows<T>::n;
        const i64 blocks = (j.R + 4 * kJoinRows - 1) / (4 * kJoinRows);
        if (blocks > 0x7fffffffLL) return CWR_ERR_TOO_LARGE;
        if ((j.H / VEC) % 64 == 0)
            CWR_LAUNCH((k_join<T, VEC, ACT, false>), dim3((unsigned)blocks), dim3(256), 0, j.stream,
                               static_cast<const T*>(j.a), static_cast<const T*>(j.b), j.lx, j.ly, j.row_off,
                               (int)j.N, (int)j.T_pad, (int)j.Up_pad, (int)j.H, j.R, static_cast<T*>(j.o1), j.status);
        else
            CWR_LAUNCH((k_join<T, VEC, ACT, true>), dim3((unsigned)blocks), dim3(256), 0, j.stream,
                               static_cast<const T*>(j.a), static_cast<const T*>(j.b), j.lx, j.ly, j.row_off,
                               (int)j.N, (int)j.T_pad, (int)j.Up_pad, (int)j.H, j.R, static_cast<T*>(j.o1), j.status);
        return check_launch();
    }
    const i64 cblocks = (j.H / VEC + 255) / 256;
    if (j.T_pad > 65535 || j.Up_pad > 65535) return CWR_ERR_TOO_LARGE;
    for (i64 n0 = 0; n0 < j.N; n0 += 65535) {
        const unsigned nz = (unsigned)(j.N - n0 < 65535 ? j.N - n0 : 65535);
        if (j.T_pad > 0) {
            CWR_LAUNCH((k_join_bwd_f<T, VEC, ACT>), dim3((unsigned)cblocks, (unsigned)j.T_pad, nz), dim3(256),
                               0, j.stream, static_cast<const T*>(j.a), static_cast<const T*>(j.b), j.lx, j.ly,
                               j.row_off, (int)n0, (int)j.T_pad, (int)j.H, j.R, static_cast<T*>(j.o1));
            int rc = check_launch();
            if (rc != CWR_OK) return rc;
        }
        if (j.Up_pad > 0) {
            CWR_LAUNCH((k_join_bwd_g<T, VEC, ACT>), dim3((unsigned)cblocks, (unsigned)j.Up_pad, nz), dim3(256),
                               0, j.stream, static_cast<const T*>(j.a), static_cast<const T*>(j.b), j.lx, j.ly,
                               j.row_off, (int)n0, (int)j.Up_pad, (int)j.H, j.R, static_cast<T*>(j.o2));
            int rc = check_launch();
            if (rc != CWR_OK) return rc;
        }
    }
    return CWR_OK;
}

template <typename T, int VEC>
static int join_act(const JoinArgs& j, int act, bool backward) {
    switch (act) {
        case kActNone: return join_launch<T, VEC, kActNone>(j, backward);
        case kActTanh: return join_launch<T, VEC, kActTanh>(j, backward);
        case kActRelu: return join_launch<T, VEC, kActRelu>(j, backward);
    }
    return CWR_ERR_MODE;
}

template <typename T>
static int join_typed(const JoinArgs& j, int act, bool backward) {
    const uintptr_t all = reinterpret_cast<uintptr_t>(j.a) | reinterpret_cast<uintptr_t>(j.b) |
                          reinterpret_cast<uintptr_t>(j.o1) | reinterpret_cast<uintptr_t>(j.o2);
    constexpr int VEC = Elem<T>::VEC;
    if (j.H % VEC == 0 && (all & 15u) == 0) return join_act<T, VEC>(j, act, backward);
    return join_act<T, 1>(j, act, backward);
}

int launch_join(int dtype, int act, bool backward, const void* a, const void* b, void* o1, void* o2, const int* lx,
                const int* ly, const i64* row_off, i64 N, i64 T_pad, i64 Up_pad, i64 H, i64 R, int* status,
                hipStream_t stream) {
    if (N == 0) return CWR_OK;
    const JoinArgs j = {a, b, o1, o2, lx, ly, row_off, N, T_pad, Up_pad, H, R, status, stream};
    switch (dtype) {
        case CWR_F32: return join_typed<float>(j, act, backward);
        case CWR_F16: return join_typed<__half>(j, act, backward);
        case CWR_BF16: return join_typed<bf16_t>(j, act, backward);
        case CWR_F64: return join_typed<double>(j, act, backward);
    }
    return CWR_ERR_DTYPE;
}

}  // namespace cwr
