// Pieces of the gated RMS norm that every kernel evaluating it must share, so that a kernel fusing the
// norm into another operation produces the bits of the stand-alone one: the gate, the reductions over
// a wave and the reciprocal standard deviation, each as one fixed sequence of fp32 operations.
// Reference: quamba/triton/quant_normgated.py:48-69.
#pragma once

#include "qa_common.hpp"

namespace qa {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}
__device__ __forceinline__ float silu_of(float z) { return z * (1.0f / (1.0f + expf(-z))); }

// gate value of int8 code (i - 128)
__device__ __forceinline__ float gate_of_code(int i, float z_scale) { return silu_of(z_scale * static_cast<float>(i - 128)); }

// one more term of a lane's running sum of squares
__device__ __forceinline__ float ssq_step(float ssq, float v) { return __builtin_fmaf(v, v, ssq); }

__device__ __forceinline__ float rstd_of(float ssq, int n, float eps) {
    const float var = ssq / static_cast<float>(n);
    return 1.0f / sqrtf(var + eps);
}

// (x * rstd) * w, then the gate when it comes after the norm
__device__ __forceinline__ float norm_value(float v, float rstd, float w) { return (v * rstd) * w; }

// fp16 of a value that is already an fp32 number.  The empty asm separates the conversion from the
// multiplication that produced y: merged into one mixed-precision instruction the two would round the
// exact product once, and the result would depend on whether the compiler found the pair.
__device__ __forceinline__ __half half_of_f32(float y) {
    asm("" : "+v"(y));
    return __float2half(y);
}

}  // namespace qa
