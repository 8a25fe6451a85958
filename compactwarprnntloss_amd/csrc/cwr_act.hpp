// Activation of the joiner (shared by the join kernels and by the output-layer kernels that form the
// joint rows themselves): the same arithmetic in both, so that the two routes give the same bits.
#pragma once

#include "cwr_device.hpp"

namespace cwr {

enum { kActNone = 0, kActTanh = 1, kActRelu = 2 };

// arithmetic type of a storage type
template <typename T> struct Arith {
    typedef float type;
    static __device__ __forceinline__ float up(T v) { return Elem<T>::to_f32(v); }
    static __device__ __forceinline__ T down(float v) { return Elem<T>::from_f32(v); }
};
template <> struct Arith<double> {
    typedef double type;
    static __device__ __forceinline__ double up(double v) { return v; }
    static __device__ __forceinline__ double down(double v) { return v; }
};

// tanh to about 1e-7 absolute: an odd polynomial near zero, where 1 - 2/(1+e^2x) cancels.  For
// 16-bit storage that cancellation (6e-8) is far below one rounding of the result and the
// polynomial is left out.
template <bool NEAR_ZERO>
__device__ __forceinline__ float act_tanh(float x) {
    const float ax = fabsf(x);
    const float e = fast_exp2(ax * (2.f * 1.4426950408889634f));
    float r = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e);
    if (NEAR_ZERO) {
        const float x2 = x * x;
        const float small =
            ax * fmaf(x2, fmaf(x2, fmaf(x2, fmaf(x2, 62.f / 2835.f, -17.f / 315.f), 2.f / 15.f), -1.f / 3.f), 1.f);
        r = ax < 0.3f ? small : r;
    }
    return copysignf(r, x);
}

// S: the storage type, A: the arithmetic type
// The result is pinned as an fp32 value before the caller rounds it to a 16-bit type: left alone,
// the compiler may fold the activation's last operation into the conversion (one rounding, straight
// to 16 bits) in one kernel and not in another, and the two then differ in the last bit wherever the
// fp32 value sits on a rounding boundary of the narrow type.  Every kernel that forms joint rows
// goes through here, so they all give the same bits.
template <int ACT, typename S, typename A>
__device__ __forceinline__ A activate(A z) {
    A r = z;
    if constexpr (ACT == kActTanh) {
        if constexpr (sizeof(A) == 8) r = tanh(z);
        else r = act_tanh<sizeof(S) == 4>(z);
    }
    if (ACT == kActRelu) r = z > A(0) ? z : A(0);
    if constexpr (sizeof(A) == 4 && sizeof(S) == 2) asm volatile("" : "+v"(r));
    return r;
}
// dz from dh and the stored output h
template <int ACT, typename A>
__device__ __forceinline__ A act_grad(A dh, A h) {
    if (ACT == kActTanh) return dh * (A(1) - h * h);
    if (ACT == kActRelu) return h > A(0) ? dh : A(0);
    return dh;
}

}  // namespace cwr
