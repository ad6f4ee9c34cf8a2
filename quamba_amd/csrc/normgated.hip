// Gated RMS norm over groups of columns of fp16 rows, int8 gate, int8 or fp16 output.
//
// Reference: quamba/triton/quant_normgated.py:11-82 (one program per (row, group)):
//   x' = x * z * sigmoid(z) with z = z_scale * qz when the gate comes first (:48-50),
//   var = sum(x'^2) / N, rstd = 1 / sqrt(var + eps) (:55-58), y = x' * rstd * w (:65-66),
//   y *= z * sigmoid(z) when the gate comes last (:67-69), then fp16, rint(y / s) with a static s, or with
//   s = max(y) / 127 per (row, group) written out (:70-82).
// The sum of squares is a tree here as in Triton, but in this kernel's own order, so results agree with
// any other evaluation to the last bit of the row's scale only.
//
// Mapping: one wave per (row, group); a lane holds group_size / 64 values in 16-byte pieces (piece c of
// lane l covers columns (c*64 + l)*8 .. +8, so every load and store of a wave is one contiguous run).
#include "qa_common.hpp"

namespace qa {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxPieces = 16;      // 16 pieces * 64 lanes * 8 columns = 8192 columns per group

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

template <int PIECES>
__global__ __launch_bounds__(64 * kWavesPerBlock) void rmsnorm_gated_kernel(QaNormGatedParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ngroups = p.dim / p.group_size;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    if (item >= static_cast<int64_t>(p.rows) * ngroups) return;
    const int64_t row = item / ngroups;
    const int group = static_cast<int>(item % ngroups);
    const int N = p.group_size;
    const int col0 = group * N;
    const __half* x = static_cast<const __half*>(p.x) + row * p.x_row_stride + col0;
    const __half* w = static_cast<const __half*>(p.weight) + col0;
    const int8_t* qz = p.qz ? p.qz + row * p.z_row_stride + col0 : nullptr;
    const int npieces = N / 512 + (N % 512 ? 1 : 0);        // pieces per lane (last may be partial across lanes)

    float v[PIECES][8], gate[PIECES][8];
    float ssq = 0.0f;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = (c * 64 + lane) * 8;
        const bool on = c < npieces && e0 < N;
#pragma unroll
        for (int j = 0; j < 8; ++j) { v[c][j] = 0.0f; gate[c][j] = 1.0f; }
        if (on) {
            const uint4 raw = *reinterpret_cast<const uint4*>(x + e0);
            const __half* h = reinterpret_cast<const __half*>(&raw);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[c][j] = __half2float(h[j]);
            if (qz) {
                const uint2 zr = *reinterpret_cast<const uint2*>(qz + e0);
                const int8_t* zb = reinterpret_cast<const int8_t*>(&zr);
#pragma unroll
                for (int j = 0; j < 8; ++j) gate[c][j] = silu_of(p.z_scale * static_cast<float>(zb[j]));
                if (!p.norm_before_gate) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[c][j] *= gate[c][j];
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ssq += v[c][j] * v[c][j];
        }
    }
    const float var = wave_sum(ssq) / static_cast<float>(N);
    const float rstd = 1.0f / sqrtf(var + p.eps);

    float ymax = -INFINITY;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = (c * 64 + lane) * 8;
        if (c < npieces && e0 < N) {
            const uint4 wraw = *reinterpret_cast<const uint4*>(w + e0);
            const __half* wh = reinterpret_cast<const __half*>(&wraw);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float y = (v[c][j] * rstd) * __half2float(wh[j]);
                if (qz && p.norm_before_gate) y *= gate[c][j];
                v[c][j] = y;
                ymax = fmaxf(ymax, y);
            }
        }
    }
    float inv_scale = 0.0f, scale = p.out_scale;
    if (p.out_mode == QA_NORM_OUT_I8_DYNAMIC) {
        scale = wave_max(ymax) / 127.0f;
        if (lane == 0) p.dyn_scale[static_cast<int64_t>(group) * p.rows + row] = scale;
    }
    (void)inv_scale;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = (c * 64 + lane) * 8;
        if (c < npieces && e0 < N) {
            if (p.out_mode == QA_NORM_OUT_F16) {
                __half o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = __float2half(v[c][j]);
                *reinterpret_cast<uint4*>(static_cast<__half*>(p.out) + row * p.out_row_stride + col0 + e0) =
                    *reinterpret_cast<const uint4*>(o);
            } else {
                int8_t o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = sat8_rne(v[c][j] / scale);
                *reinterpret_cast<uint2*>(static_cast<int8_t*>(p.out) + row * p.out_row_stride + col0 + e0) =
                    *reinterpret_cast<const uint2*>(o);
            }
        }
    }
}

}  // namespace
}  // namespace qa

extern "C" int qa_rmsnorm_gated(const QaNormGatedParams* p, void* stream_) {
    using namespace qa;
    if (!p || !p->x || !p->weight || !p->out) return QA_ERR_NULL;
    if (p->out_mode == QA_NORM_OUT_I8_DYNAMIC && !p->dyn_scale) return QA_ERR_NULL;
    if (p->out_mode < 0 || p->out_mode > 2) return QA_ERR_UNSUPPORTED;
    if (p->rows < 0 || p->dim < 1 || p->group_size < 1 || p->dim % p->group_size != 0) return QA_ERR_SHAPE;
    if (p->group_size % 8 != 0 || p->group_size > kMaxPieces * 512) return QA_ERR_UNSUPPORTED;
    if (p->x_row_stride % 8 != 0 || p->out_row_stride % 8 != 0 || (p->qz && p->z_row_stride % 8 != 0)) return QA_ERR_STRIDE;
    if (!aligned16(p->x) || !aligned16(p->weight) || !aligned16(p->out) ||
        (p->qz && (reinterpret_cast<uintptr_t>(p->qz) & 7u))) return QA_ERR_STRIDE;
    if (p->rows == 0) return QA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t items = static_cast<int64_t>(p->rows) * (p->dim / p->group_size);
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
    const dim3 grid(static_cast<unsigned>(blocks)), block(64 * kWavesPerBlock);
    const int pieces = (p->group_size + 511) / 512;
    if (pieces <= 2) hipLaunchKernelGGL(rmsnorm_gated_kernel<2>, grid, block, 0, stream, *p);
    else if (pieces <= 4) hipLaunchKernelGGL(rmsnorm_gated_kernel<4>, grid, block, 0, stream, *p);
    else if (pieces <= 8) hipLaunchKernelGGL(rmsnorm_gated_kernel<8>, grid, block, 0, stream, *p);
    else hipLaunchKernelGGL(rmsnorm_gated_kernel<16>, grid, block, 0, stream, *p);
    return check_launch();
}
