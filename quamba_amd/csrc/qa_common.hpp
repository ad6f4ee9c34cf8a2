// Shared host/device helpers for the quamba_amd HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/quamba_amd.h"

namespace qa {

// Records the HIP error of a failed launch for qa_last_hip_error().
void set_last_hip_error(int code);

// Zeroes `bytes` bytes with a kernel (states after a scan over no steps; a memset node would not survive graph capture
// on every runtime).  Null or empty: nothing to do.
int fill_zero(void* dst, int64_t bytes, hipStream_t stream);

inline int check_launch() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_hip_error(static_cast<int>(e));
        return QA_ERR_LAUNCH;
    }
    return QA_OK;
}

// f(integral_constant<int, I>) for I = FIRST .. LAST-1: a loop whose index is a compile-time constant
template <int FIRST, int LAST, typename F>
__host__ __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>{});
        static_for<FIRST + 1, LAST>(f);
    }
}

__host__ __device__ inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__host__ __device__ inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// ---------------------------------------------------------------------------------------------
// Deterministic exp.  The int8 requantisation of the conv output rounds silu(v)/s_out to an
// integer, so the low bits of exp decide ties.  To make results reproducible bit for bit on any
// IEEE-754 machine, exp is defined here as a fixed sequence of fp32 operations (one multiply, one
// round-to-nearest-even, two FMAs of Cody-Waite reduction, a degree-7 Horner polynomial in FMAs
// and an exact power-of-two scaling).  Error is below 1.5 ulp over the whole range.
//   x >  88.0f            -> +inf
//   x < -87.0f            -> 0      (results that would be subnormal are flushed)
//   NaN                   -> NaN
// ---------------------------------------------------------------------------------------------
__host__ __device__ __forceinline__ float exp_det(float x) {
    if (x > 88.0f) return __builtin_inff();
    if (x < -87.0f) return 0.0f;
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693145751953125f, x);        // ln2 high part (exact product)
    r = __builtin_fmaf(n, -1.42860682030941723e-6f, r);         // ln2 low part
    float p = 1.0f / 5040.0f;
    p = __builtin_fmaf(p, r, 1.0f / 720.0f);
    p = __builtin_fmaf(p, r, 1.0f / 120.0f);
    p = __builtin_fmaf(p, r, 1.0f / 24.0f);
    p = __builtin_fmaf(p, r, 1.0f / 6.0f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    const int e = static_cast<int>(n);                          // in [-126, 127]
    const uint32_t bits = static_cast<uint32_t>(e + 127) << 23;
    return p * __builtin_bit_cast(float, bits);
}

// round half away from zero, then saturate to int8 (NaN -> -128)
__host__ __device__ __forceinline__ int8_t sat8_half_away(float v) {
    float r = __builtin_roundf(v);
    r = __builtin_fmaxf(r, -128.0f);
    r = __builtin_fminf(r, 127.0f);
    return static_cast<int8_t>(static_cast<int>(r));
}

// round half to even, then saturate to int8 (NaN -> -128)
__host__ __device__ __forceinline__ int8_t sat8_rne(float v) {
    float r = __builtin_rintf(v);
    r = __builtin_fmaxf(r, -128.0f);
    r = __builtin_fminf(r, 127.0f);
    return static_cast<int8_t>(static_cast<int>(r));
}

}  // namespace qa
