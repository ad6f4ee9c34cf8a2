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
// Mapping: one wave per (row, group) for groups of up to 2048 columns, the four waves of a workgroup
// together for wider ones (holding a wide group in one wave's registers halves the rate).  A lane holds
// its values in 16-byte pieces; piece c of lane l of wave w covers columns ((c*W + w)*64 + l)*8 .. +8
// (W waves per group), so every load and store of a wave is one contiguous run.
// The gate has 256 possible values (one per int8 code): a workgroup evaluates them once into LDS and
// every element looks its gate up, which gives the same bits as evaluating it per element.
#include "normgated_core.hpp"

namespace qa {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxPieces = 16;      // per lane: 16 pieces * 4 waves * 64 lanes * 8 columns = 32768 columns per group

template <int PIECES, int WPI, bool GATE_LAST>
__global__ __launch_bounds__(64 * kWavesPerBlock) void rmsnorm_gated_kernel(QaNormGatedParams p) {
    __shared__ float s_gate[256];
    __shared__ float s_part[2][kWavesPerBlock];
    if (p.qz) {
        for (int i = threadIdx.x; i < 256; i += 64 * kWavesPerBlock) s_gate[i] = gate_of_code(i, p.z_scale);
        __syncthreads();
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ngroups = p.dim / p.group_size;
    constexpr int kItemsPerBlock = kWavesPerBlock / WPI;
    const int sub = wave % WPI;                               // this wave's share of the group
    // the item is the same for a whole wave: scalar arithmetic, 32 bits (the host bounds the item count)
    const unsigned item = __builtin_amdgcn_readfirstlane(blockIdx.x * kItemsPerBlock + wave / WPI);
    if (item >= static_cast<unsigned>(p.rows) * static_cast<unsigned>(ngroups)) return;   // with WPI > 1 the whole workgroup leaves
    const int64_t row = item / static_cast<unsigned>(ngroups);
    const int group = static_cast<int>(item % static_cast<unsigned>(ngroups));
    const int N = p.group_size;
    const int col0 = group * N;
    const __half* x = static_cast<const __half*>(p.x) + row * p.x_row_stride + col0;
    const __half* w = static_cast<const __half*>(p.weight) + col0;
    const int8_t* qz = p.qz ? p.qz + row * p.z_row_stride + col0 : nullptr;
    constexpr int kSpan = 512 * WPI;                          // columns covered by one piece index
    const int npieces = (N + kSpan - 1) / kSpan;              // pieces per lane (the last may be partial)

    float v[PIECES][8], gate[GATE_LAST ? PIECES : 1][8];
    float ssq = 0.0f;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = ((c * WPI + sub) * 64 + lane) * 8;
        const bool on = c < npieces && e0 < N;
#pragma unroll
        for (int j = 0; j < 8; ++j) { v[c][j] = 0.0f; if (GATE_LAST) gate[c][j] = 1.0f; }
        if (on) {
            const uint4 raw = *reinterpret_cast<const uint4*>(x + e0);
            const __half* h = reinterpret_cast<const __half*>(&raw);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[c][j] = __half2float(h[j]);
            if (qz) {
                const uint2 zr = *reinterpret_cast<const uint2*>(qz + e0);
                const int8_t* zb = reinterpret_cast<const int8_t*>(&zr);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float g = s_gate[static_cast<int>(zb[j]) + 128];
                    if (GATE_LAST) gate[c][j] = g;
                    else v[c][j] *= g;
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ssq = ssq_step(ssq, v[c][j]);
        }
    }
    ssq = wave_sum(ssq);
    if (WPI > 1) {
        if (lane == 0) s_part[0][wave] = ssq;
        __syncthreads();
        ssq = 0.0f;
#pragma unroll
        for (int i = 0; i < WPI; ++i) ssq += s_part[0][i];
    }
    const float rstd = rstd_of(ssq, N, p.eps);

    float ymax = -INFINITY;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = ((c * WPI + sub) * 64 + lane) * 8;
        if (c < npieces && e0 < N) {
            const uint4 wraw = *reinterpret_cast<const uint4*>(w + e0);
            const __half* wh = reinterpret_cast<const __half*>(&wraw);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float y = norm_value(v[c][j], rstd, __half2float(wh[j]));
                if (GATE_LAST && qz) y *= gate[c][j];
                v[c][j] = y;
                ymax = fmaxf(ymax, y);
            }
        }
    }
    float scale = p.out_scale;
    if (p.out_mode == QA_NORM_OUT_I8_DYNAMIC) {
        ymax = wave_max(ymax);
        if (WPI > 1) {
            if (lane == 0) s_part[1][wave] = ymax;
            __syncthreads();
#pragma unroll
            for (int i = 0; i < WPI; ++i) ymax = fmaxf(ymax, s_part[1][i]);
        }
        scale = ymax / 127.0f;
        if (lane == 0 && sub == 0) p.dyn_scale[static_cast<int64_t>(group) * p.rows + row] = scale;
    }
    const float inv_scale = 1.0f / scale;
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int e0 = ((c * WPI + sub) * 64 + lane) * 8;
        if (c < npieces && e0 < N) {
            if (p.out_mode == QA_NORM_OUT_F16) {
                __half o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = half_of_f32(v[c][j]);
                *reinterpret_cast<uint4*>(static_cast<__half*>(p.out) + row * p.out_row_stride + col0 + e0) =
                    *reinterpret_cast<const uint4*>(o);
            } else {
                int8_t o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = sat8_rne(v[c][j] * inv_scale);
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
    if (!p) return QA_ERR_NULL;
    if (p->rows > 0 && (!p->x || !p->weight || !p->out)) return QA_ERR_NULL;      // (no rows: the tensors may be null)
    if (p->rows > 0 && p->out_mode == QA_NORM_OUT_I8_DYNAMIC && !p->dyn_scale) return QA_ERR_NULL;
    if (p->out_mode < 0 || p->out_mode > 2) return QA_ERR_UNSUPPORTED;
    if (p->rows < 0 || p->dim < 1 || p->group_size < 1 || p->dim % p->group_size != 0) return QA_ERR_SHAPE;
    if (p->group_size % 8 != 0 || p->group_size > kMaxPieces * kWavesPerBlock * 512) return QA_ERR_UNSUPPORTED;
    if (p->x_row_stride % 8 != 0 || p->out_row_stride % 8 != 0 || (p->qz && p->z_row_stride % 8 != 0)) return QA_ERR_STRIDE;
    if (!aligned16(p->x) || !aligned16(p->weight) || !aligned16(p->out) ||
        (p->qz && (reinterpret_cast<uintptr_t>(p->qz) & 7u))) return QA_ERR_STRIDE;
    if (p->rows == 0) return QA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t items = static_cast<int64_t>(p->rows) * (p->dim / p->group_size);
    const bool together = p->group_size > 2048;               // four waves per group
    const int64_t blocks = together ? items : (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL || items > 0x7fffffffLL) return QA_ERR_SHAPE;
    const dim3 grid(static_cast<unsigned>(blocks)), block(64 * kWavesPerBlock);
    const int span = together ? 512 * kWavesPerBlock : 512;
    const int pieces = (p->group_size + span - 1) / span;
    const bool gate_last = p->qz && p->norm_before_gate;
    auto launch = [&](auto pieces_c) {
        constexpr int kPieces = decltype(pieces_c)::value;
        if (together) {
            if (gate_last) hipLaunchKernelGGL((rmsnorm_gated_kernel<kPieces, kWavesPerBlock, true>), grid, block, 0, stream, *p);
            else hipLaunchKernelGGL((rmsnorm_gated_kernel<kPieces, kWavesPerBlock, false>), grid, block, 0, stream, *p);
        } else {
            if (gate_last) hipLaunchKernelGGL((rmsnorm_gated_kernel<kPieces, 1, true>), grid, block, 0, stream, *p);
            else hipLaunchKernelGGL((rmsnorm_gated_kernel<kPieces, 1, false>), grid, block, 0, stream, *p);
        }
    };
    if (pieces <= 2) launch(std::integral_constant<int, 2>{});
    else if (pieces <= 4) launch(std::integral_constant<int, 4>{});
    else if (pieces <= 8) launch(std::integral_constant<int, 8>{});
    else launch(std::integral_constant<int, 16>{});
    return check_launch();
}
