// What the two implementations of the Mamba2 SSD chunk scan share (ssd.hip: the matrix-core kernels for the shapes
// of the released models; ssd_general.hip: every other head dimension, state count and chunk length): workspace
// layout, scale lookup, the shape test that picks between them.
#pragma once

#include "qa_common.hpp"

namespace qa {

constexpr float kSsdLog2e = 1.44269504088896341f;

__device__ __forceinline__ float ssd_exp(float x) { return __builtin_amdgcn_exp2f(x * kSsdLog2e); }

struct SsdWorkspace {            // sections of the workspace (byte offsets), see qa_ssd_workspace_bytes
    int64_t dt, dA, prev, xs, srow, total;
};

__host__ __device__ inline int64_t ssd_align256(int64_t v) { return (v + 255) & ~int64_t(255); }

// dt and the within-chunk cumsum of dt A, fp32 [batch, nheads, chunks, chunk_size]; the states entering the chunks,
// fp16 [batch, chunks, nheads, headdim, dstate]; the x scale of every channel, fp32 [nheads, headdim], and the row of
// the grouped state scales it quantises its final state with, int32 [nheads, headdim] (both looked up once from the
// group ranges by the first kernel: the others read them with one load instead of a chain of dependent ones)
__host__ __device__ inline SsdWorkspace ssd_workspace_layout(const QaSsdParams& p) {
    const int64_t nc = (p.seqlen + p.chunk_size - 1) / p.chunk_size;
    const int64_t B = p.batch, H = p.nheads, Q = p.chunk_size, N = p.dstate, P = p.headdim;
    SsdWorkspace w;
    int64_t off = 0;
    w.dt = off; off = ssd_align256(off + B * H * nc * Q * 4);
    w.dA = off; off = ssd_align256(off + B * H * nc * Q * 4);
    w.prev = off; off = ssd_align256(off + B * nc * H * P * N * 2);
    w.xs = off; off = ssd_align256(off + H * P * 4);
    w.srow = off; off = ssd_align256(off + H * P * 4);
    w.total = off;
    return w;
}

// x scale of channel p of head h (per-tensor, or looked up from the cumulative group ranges,
// quamba/triton/quant_chunk_state.py:202-214)
__device__ __forceinline__ void ssd_group_of(const QaSsdParams& p, int h, int& g, int& hg) {
    const int hpg = p.nheads / p.ngroups;
    g = h / hpg;
    hg = 0;
    if (p.nhead_groups > 0) {
        for (int j = 0; j < p.nhead_groups; ++j) hg += (h % hpg) >= p.x_head_group_range[g * p.nhead_groups + j] ? 1 : 0;
        hg = min(hg, p.nhead_groups - 1);
    }
}
__device__ __forceinline__ int ssd_dim_group_of(const QaSsdParams& p, int g, int hg, int ch) {
    const int32_t* dr = p.x_dim_group_range + (g * p.nhead_groups + hg) * p.ndim_groups;
    int dg = 0;
    for (int j = 0; j < p.ndim_groups; ++j) dg += ch >= dr[j] ? 1 : 0;
    return min(dg, p.ndim_groups - 1);
}
__device__ __forceinline__ float ssd_x_scale_of(const QaSsdParams& p, int g, int hg, int ch) {
    if (p.nhead_groups == 0) return p.x_scale[0];
    return p.x_scale[(g * p.nhead_groups + hg) * p.ndim_groups + ssd_dim_group_of(p, g, hg, ch)];
}

// The per-channel tables: called by the wave that handles (batch 0, chunk 0, head h) in the first kernel.
// srow: index of the first state's scale in state_scale for this channel (0 with one scale for everything)
__device__ __forceinline__ void ssd_write_channel_tables(const QaSsdParams& p, int h, int lane, float* xs_out, int32_t* srow_out) {
    int g, hg;
    ssd_group_of(p, h, g, hg);
    for (int ch = lane; ch < p.headdim; ch += 64) {
        xs_out[h * p.headdim + ch] = ssd_x_scale_of(p, g, hg, ch);
        srow_out[h * p.headdim + ch] = p.nhead_groups > 0 ? ((g * p.nhead_groups + hg) * p.ndim_groups + ssd_dim_group_of(p, g, hg, ch)) * p.dstate : 0;
    }
}

// int8 final state of one element (quamba/triton/quant_ssm_states.py:43,119): the reference hands fp16 states to the
// quantiser; one scale, or one per (ssd group, head group, dim group, state) with the factor 1e6 instead of 1e2
// (srow: the channel's entry of the table above)
__device__ __forceinline__ int8_t ssd_quantize_state(const QaSsdParams& p, int srow, int n, float value) {
    const bool grouped = p.nhead_groups > 0;
    const float sc = p.state_scale[grouped ? srow + n : 0];
    const float K = grouped ? 1e6f : 1e2f;
    const float s16 = __half2float(__float2half(value));
    return sat8_rne((s16 * K) / (sc * K));
}

// The shapes the matrix-core kernels are built for (everything else takes the general kernels)
inline bool ssd_fast_shape(const QaSsdParams& p) {
    if (p.headdim % 64 != 0 || (p.dstate != 64 && p.dstate != 128)) return false;
    if (p.chunk_size != 64 && p.chunk_size != 128 && p.chunk_size != 256) return false;
    // x, B, C, the gate and the output are accessed in aligned 16-byte pieces there
    if (!aligned16(p.x) || !aligned16(p.B) || !aligned16(p.C) || !aligned16(p.out)) return false;
    if (p.z && !aligned16(p.z)) return false;
    if (p.D && p.D_has_hdim && !aligned16(p.D)) return false;
    return true;
}

// ssd_general.hip
int ssd_general_grid_check(const QaSsdParams& p);
void ssd_general_launch(const QaSsdParams& p, float* dt_ws, float* dA_ws, __half* prev_ws, float* xs_ws, int32_t* srow_ws, int nc,
                        hipStream_t stream);

}  // namespace qa
