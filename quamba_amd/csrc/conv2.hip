// Mamba2 xBC conv: depthwise causal conv1d (+SiLU) over the concatenated [x | B | C] channels of
// in_proj's output, requantised into three int8 tensors with per-part input/weight/bias scales and
// grouped output scales.
//
// Arithmetic (reference csrc/causal_conv1d/quamba2_conv1d_fwd_kernel.cuh:215-246, update kernel
// quamba2_conv1d_update_kernel.cuh:134-143):
//   forward   v = fma(s_w*s_in, sum_w W[c,w]*x[t-(k-1-w)], s_b*bias[c])
//   update    v = s_b*bias[c];  v = fma((s_w*s_in)*W[c,w], x[..], v) per tap, after shifting the state
//   then v = v / (1 + exp(-v)) if silu, q = sat8(round_half_away(v / s_out[c]))
// s_out[c] for an x channel is found through the cumulative head-group / dim-group end indices of
// its ssd group (fwd kernel :151-189), for B and C channels it is the ssd group's scale (:190-212).
//
// Layout and mapping: activations are channel-contiguous (batch, seqlen, dim).  A lane owns four
// neighbouring channels and walks a run of time steps: one dword load per step (a wave reads 256
// contiguous bytes), the last four inputs of each channel are kept as a packed byte window updated
// with one byte permute, the taps are one packed int8 dot product per output (exact), the epilogue
// is the cheap-with-exact-fallback route shared with the Mamba1 conv, one dword store per step.
#include "conv_common.hpp"

namespace qa {
namespace {

constexpr int kThreads = 256;
constexpr int kRun = 64;          // time steps per wave unless the launch picks more
constexpr int kBatchLoads = 8;    // loads in flight per lane

struct Part {
    int index;        // 0 = x, 1 = B, 2 = C
    int offset;       // first channel of the part inside xBC
    float s_in;       // weight scale * input scale
    float s_bias;
};

__device__ __forceinline__ Part part_of(const QaConv2Params& p, int ch) {
    const int bc = p.d_state * p.n_groups;
    Part r;
    if (ch < p.x_dim) {
        r.index = 0; r.offset = 0; r.s_in = p.scale_wx * p.scale_x; r.s_bias = p.scale_bx;
    } else if (ch < p.x_dim + bc) {
        r.index = 1; r.offset = p.x_dim; r.s_in = p.scale_wB * p.scale_B; r.s_bias = p.scale_bB;
    } else {
        r.index = 2; r.offset = p.x_dim + bc; r.s_in = p.scale_wC * p.scale_C; r.s_bias = p.scale_bC;
    }
    return r;
}

// Output scale of channel `ch`; the range walk is the reference's (first range that contains the index).
__device__ __forceinline__ float out_scale_of(const QaConv2Params& p, const Part& part, int ch) {
    const bool grouped = p.x_head_group_range != nullptr && p.x_dim_group_range != nullptr;
    if (part.index != 0) {
        const float* s = part.index == 1 ? p.B_out_scales : p.C_out_scales;
        return grouped ? s[(ch - part.offset) / p.d_state] : s[0];
    }
    if (!grouped) return p.x_out_scales[0];
    const int group_size = p.x_dim / p.n_groups;
    const int g = ch / group_size;
    const int head = (ch % group_size) / p.x_headdim;
    const int d = ch % p.x_headdim;
    const float* scales = p.x_out_scales + g * p.nhead_groups * p.ndim_groups;
    const int32_t* hr = p.x_head_group_range + g * p.nhead_groups;
    const int32_t* dr = p.x_dim_group_range + g * p.nhead_groups * p.ndim_groups;
    float s = 0.0f;
    int h_start = 0;
    for (int hg = 0; hg < p.nhead_groups; ++hg) {
        if (h_start <= head && head < hr[hg]) {
            int d_start = 0;
            for (int dg = 0; dg < p.ndim_groups; ++dg) {
                if (d_start <= d && d < dr[hg * p.ndim_groups + dg]) {
                    s = scales[hg * p.ndim_groups + dg];
                    break;
                }
                d_start = dr[hg * p.ndim_groups + dg];
            }
            break;
        }
        h_start = hr[hg];
    }
    return s;
}

__device__ __forceinline__ int8_t* out_ptr(const QaConv2Params& p, const Part& part, int b, int ch,
                                            int64_t* l_stride, int64_t* c_stride) {
    const int local = ch - part.offset;
    if (part.index == 0) { *l_stride = p.x_l_stride; *c_stride = p.x_c_stride; return p.x + b * p.x_batch_stride + local * p.x_c_stride; }
    if (part.index == 1) { *l_stride = p.B_l_stride; *c_stride = p.B_c_stride; return p.B + b * p.B_batch_stride + local * p.B_c_stride; }
    *l_stride = p.C_l_stride; *c_stride = p.C_c_stride;
    return p.C + b * p.C_batch_stride + local * p.C_c_stride;
}

// grid: x = blocks of 256 channels, y = blocks of 4 runs of kRun steps (one run per wave), z = batch
template <bool SILU>
__global__ __launch_bounds__(kThreads) void conv2_fwd_kernel(QaConv2Params p, int run) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));   // the same in every lane: the step
                                                                                          // counters below stay in scalar registers
    const int ch0 = (blockIdx.x * 64 + lane) * 4;
    const int b = blockIdx.z;
    const int t0 = (blockIdx.y * 4 + wave) * run;
    if (ch0 >= p.dim || t0 >= p.seqlen) return;
    const int t_end = min(t0 + run, p.seqlen);

    // The inputs are requested first: the walk over the group ranges below (dependent loads, four channels) then runs
    // under their round trip instead of in front of it.
    const int8_t* src = p.xBC + b * p.xBC_batch_stride + ch0;
    uint32_t hist[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int t = t0 - 3 + i;
        hist[i] = *reinterpret_cast<const uint32_t*>(src + max(t, 0) * p.xBC_l_stride);
    }
    // the loads of the next batch of steps are in flight while the current batch is worked on
    uint32_t d[kBatchLoads], dn[kBatchLoads];
    auto fetch = [&](int tb, uint32_t (&dst)[kBatchLoads]) {
#pragma unroll
        for (int i = 0; i < kBatchLoads; ++i) {
            const int t = min(tb + i, p.seqlen - 1);              // in range for every lane; steps past the end are never used
            dst[i] = *reinterpret_cast<const uint32_t*>(src + t * p.xBC_l_stride);
        }
    };
    fetch(t0, dn);

    const Part part = part_of(p, ch0);          // the four channels of a lane never straddle two parts
    uint32_t taps[4];
    float bias_f[4], s_out[4], inv_s_out[4];
    bool exact_only[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int ch = ch0 + e;
        taps[e] = pack_taps(p.weight + ch * p.weight_c_stride, p.weight_width_stride, p.width);
        bias_f[e] = p.bias ? part.s_bias * static_cast<float>(p.bias[ch]) : 0.0f;
        s_out[e] = out_scale_of(p, part, ch);
        inv_s_out[e] = 1.0f / s_out[e];
        exact_only[e] = conv_needs_exact_route(s_out[e]);
    }
    const ConvQuantRegs kq(__builtin_fminf(__builtin_fminf(s_out[0], s_out[1]), __builtin_fminf(s_out[2], s_out[3])));
    int64_t out_ls, out_cs;
    int8_t* out = out_ptr(p, part, b, ch0, &out_ls, &out_cs);

    // byte j of win[e] holds x[t-3+j] of channel ch0+e
    uint32_t win[4] = {0u, 0u, 0u, 0u};
    auto push = [&](uint32_t d) {
        win[0] = __builtin_amdgcn_perm(d, win[0], 0x04030201u);
        win[1] = __builtin_amdgcn_perm(d, win[1], 0x05030201u);
        win[2] = __builtin_amdgcn_perm(d, win[2], 0x06030201u);
        win[3] = __builtin_amdgcn_perm(d, win[3], 0x07030201u);
    };
#pragma unroll
    for (int i = 0; i < 3; ++i) push(t0 - 3 + i >= 0 ? hist[i] : 0u);
    int8_t* out_at = out + t0 * out_ls;             // walks on by one step's stride (the stride differs from lane to lane: a
                                                    // product per step would be a 64-bit multiplication in vector registers)
    for (int tb = t0; tb < t_end; tb += kBatchLoads) {
#pragma unroll
        for (int i = 0; i < kBatchLoads; ++i) d[i] = dn[i];
        if (tb + kBatchLoads < t_end) fetch(tb + kBatchLoads, dn);
#pragma unroll
        for (int i = 0; i < kBatchLoads; ++i) {
            if (tb + i >= t_end) break;
            push(d[i]);
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(part.s_in, static_cast<float>(dot4(win[e], taps[e])), bias_f[e]);
            *reinterpret_cast<uint32_t*>(out_at) = conv_quant4(v, s_out, inv_s_out, SILU, exact_only, kq);
            out_at += out_ls;
        }
    }
}

// Any alignment: one thread per output element, same arithmetic.
__global__ __launch_bounds__(kThreads) void conv2_fwd_generic_kernel(QaConv2Params p) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t total = static_cast<int64_t>(p.batch) * p.dim * p.seqlen;
    if (idx >= total) return;
    const int ch = static_cast<int>(idx % p.dim);
    const int t = static_cast<int>((idx / p.dim) % p.seqlen);
    const int b = static_cast<int>(idx / (static_cast<int64_t>(p.seqlen) * p.dim));
    const Part part = part_of(p, ch);
    const int8_t* src = p.xBC + b * p.xBC_batch_stride + ch * p.xBC_c_stride;
    const int8_t* w = p.weight + ch * p.weight_c_stride;
    float acc = 0.0f;
    for (int k = 0; k < p.width; ++k) {
        const int ti = t - (p.width - 1 - k);
        const float xv = ti >= 0 ? static_cast<float>(src[ti * p.xBC_l_stride]) : 0.0f;
        acc += static_cast<float>(w[k * p.weight_width_stride]) * xv;      // exact integers
    }
    const float bias_f = p.bias ? part.s_bias * static_cast<float>(p.bias[ch]) : 0.0f;
    const float v = __builtin_fmaf(part.s_in, acc, bias_f);
    int64_t out_ls, out_cs;
    int8_t* out = out_ptr(p, part, b, ch, &out_ls, &out_cs);
    out[t * out_ls] = conv_epilogue(v, out_scale_of(p, part, ch), p.silu_activation);
}

__global__ __launch_bounds__(kThreads) void conv2_update_kernel(QaConv2Params p) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= static_cast<int64_t>(p.batch) * p.dim) return;
    const int ch = static_cast<int>(idx % p.dim);
    const int b = static_cast<int>(idx / p.dim);
    int8_t* st = p.conv_state + b * p.conv_state_batch_stride + ch * p.conv_state_c_stride;
    const int8_t* w = p.weight + ch * p.weight_c_stride;
    const int width = p.width;
    const int slen = p.conv_state_len;            // width (slot 0 is dropped) or width-1
    const int drop = slen - (width - 1);
    // four taps and a state of four codes, each in one aligned word (the Mamba2 layer's own buffers): one load and one
    // store per row instead of one per code
    const bool w_word = width == 4 && p.weight_width_stride == 1 && aligned4(w);
    const bool s_word = slen == 4 && p.conv_state_l_stride == 1 && aligned4(st);
    __attribute__((aligned(4))) int8_t xs[4], ws[4] = {0, 0, 0, 0};
    const int8_t x_new = p.xBC[b * p.xBC_batch_stride + ch * p.xBC_c_stride];
    if (w_word) {
        *reinterpret_cast<uint32_t*>(ws) = *reinterpret_cast<const uint32_t*>(w);
    } else {
        for (int i = 0; i < width; ++i) ws[i] = w[i * p.weight_width_stride];
    }
    if (s_word) {
        const uint32_t win = (*reinterpret_cast<const uint32_t*>(st) >> 8) | (static_cast<uint32_t>(static_cast<uint8_t>(x_new)) << 24);
        *reinterpret_cast<uint32_t*>(st) = win;                    // the whole window is the new state
        *reinterpret_cast<uint32_t*>(xs) = win;
    } else {
        for (int i = 0; i < width - 1; ++i) xs[i] = st[(i + drop) * p.conv_state_l_stride];
        xs[width - 1] = x_new;
        for (int i = 0; i < slen; ++i) st[i * p.conv_state_l_stride] = xs[i + (width - slen)];
    }
    const Part part = part_of(p, ch);
    float v = p.bias ? part.s_bias * static_cast<float>(p.bias[ch]) : 0.0f;
    for (int i = 0; i < width; ++i) v = __builtin_fmaf(part.s_in * static_cast<float>(ws[i]), static_cast<float>(xs[i]), v);
    int64_t out_ls, out_cs;
    int8_t* out = out_ptr(p, part, b, ch, &out_ls, &out_cs);
    out[0] = conv_epilogue(v, out_scale_of(p, part, ch), p.silu_activation);
}

int validate(const QaConv2Params* p, bool update) {
    if (!p) return QA_ERR_NULL;
    if (p->batch < 0 || p->dim < 0 || p->seqlen < 0 || p->batch > 65535) return QA_ERR_SHAPE;
    // (a call over no elements may pass null tensors)
    const bool empty = p->batch == 0 || p->dim == 0 || (!update && p->seqlen == 0);
    if (!empty && (!p->xBC || !p->weight || !p->x || !p->B || !p->C)) return QA_ERR_NULL;
    if (!empty && (!p->x_out_scales || !p->B_out_scales || !p->C_out_scales)) return QA_ERR_NULL;
    if ((p->x_head_group_range == nullptr) != (p->x_dim_group_range == nullptr)) return QA_ERR_NULL;
    if (!empty && update && !p->conv_state) return QA_ERR_NULL;
    if (p->width < 2 || p->width > 4) return QA_ERR_SHAPE;
    if (p->x_dim < 0 || p->x_headdim < 1 || p->d_state < 1 || p->n_groups < 1) return QA_ERR_SHAPE;
    if (p->x_dim % p->x_headdim != 0 || p->x_dim % p->n_groups != 0) return QA_ERR_SHAPE;
    if (p->x_dim + 2 * p->d_state * p->n_groups != p->dim) return QA_ERR_SHAPE;
    if (p->x_head_group_range && (p->nhead_groups < 1 || p->ndim_groups < 1)) return QA_ERR_SHAPE;
    if (update && p->conv_state_len != p->width && p->conv_state_len != p->width - 1) return QA_ERR_SHAPE;
    return QA_OK;
}

}  // namespace
}  // namespace qa

extern "C" int qa_quamba2_conv1d_fwd(const QaConv2Params* p, void* stream_) {
    using namespace qa;
    const int st = validate(p, false);
    if (st != QA_OK) return st;
    if (p->xBC_c_stride != 1 || p->x_c_stride != 1 || p->B_c_stride != 1 || p->C_c_stride != 1) return QA_ERR_STRIDE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t total = static_cast<int64_t>(p->batch) * p->dim * p->seqlen;
    if (total == 0) return QA_OK;
    const int bc = p->d_state * p->n_groups;
    auto mult4 = [](int64_t v) { return v % 4 == 0; };
    const bool vec = p->x_dim % 4 == 0 && bc % 4 == 0 && aligned4(p->xBC) && aligned4(p->x) && aligned4(p->B) &&
                     aligned4(p->C) && mult4(p->xBC_batch_stride) && mult4(p->xBC_l_stride) &&
                     mult4(p->x_batch_stride) && mult4(p->x_l_stride) && mult4(p->B_batch_stride) &&
                     mult4(p->B_l_stride) && mult4(p->C_batch_stride) && mult4(p->C_l_stride);
    if (vec) {
        // Steps per wave: 64, 128 or 256, whichever needs the fewest rounds of resident waves (seven per SIMD) times its
        // own length plus a wave's set-up (taps, scales: about 24 steps' worth).  Batch 16 x 1024 steps x 10240 channels
        // is 10240 waves of 64 steps on 7168 places - a second round at a third of the occupancy - or 5120 of 128.
        int run = kRun;
        {
            const int64_t ch_blocks = (p->dim + 255) / 256, places = 7 * 4 * 256;
            int64_t best = -1;
            for (int r = 64; r <= 256; r *= 2) {
                const int64_t waves = ch_blocks * (((p->seqlen + r - 1) / r + 3) / 4 * 4) * p->batch;
                const int64_t cost = ((waves + places - 1) / places) * (r + 24);
                if (best < 0 || cost < best) { best = cost; run = r; }
            }
        }
        const int64_t run_blocks = (p->seqlen + 4 * run - 1) / (4 * run);
        if (run_blocks > 65535) return QA_ERR_SHAPE;
        dim3 grid((p->dim + 255) / 256, static_cast<unsigned>(run_blocks), p->batch);
        if (p->silu_activation) hipLaunchKernelGGL(conv2_fwd_kernel<true>, grid, dim3(kThreads), 0, stream, *p, run);
        else hipLaunchKernelGGL(conv2_fwd_kernel<false>, grid, dim3(kThreads), 0, stream, *p, run);
        return check_launch();
    }
    const int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
    hipLaunchKernelGGL(conv2_fwd_generic_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, stream, *p);
    return check_launch();
}

extern "C" int qa_quamba2_conv1d_update(const QaConv2Params* p, void* stream_) {
    using namespace qa;
    const int st = validate(p, true);
    if (st != QA_OK) return st;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t total = static_cast<int64_t>(p->batch) * p->dim;
    if (total == 0) return QA_OK;
    const int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
    hipLaunchKernelGGL(conv2_update_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, stream, *p);
    return check_launch();
}
