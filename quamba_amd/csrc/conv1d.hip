// int8 depthwise causal conv1d (+SiLU) with int8 requantisation, forward and single-step update.
//
// Arithmetic follows the reference kernels op for op:
//   forward, seqlen-contiguous  csrc/causal_conv1d/quant_causal_conv1d_fwd_kernel.cuh:57-157
//       v = fma(s_w*s_x, sum_w W[d,w]*x[t-(k-1-w)], s_b*bias[d])
//   forward, channel-contiguous csrc/causal_conv1d/quant_causal_conv1d_fwd_kernel.cuh:267-383
//       v = s_b*bias[d];  v = fma((s_w*s_x)*W[d,w], x[..], v) per tap
//   update                      csrc/causal_conv1d/quant_causal_conv1d_update_kernel.cuh:26-76
//       same tap-wise order, after shifting the rolling state in place
//   then v = v / (1 + exp(-v)) if silu, q = sat8(round_half_away(v / s_out)).
// The kernel is memory-shaped: one 16-byte load and one 16-byte store per 16 outputs, the 3-byte
// causal halo comes from one extra aligned dword, and the four taps are one packed int8 dot
// product (exact, so equal to the reference's fp32 accumulation of integer products).
#include "conv_common.hpp"
#include <type_traits>

namespace qa {
namespace {

constexpr int kConvThreads = 256;

// One thread = 16 consecutive time steps of one (batch, channel) row.  Rows are 16-byte aligned
// (checked on the host); a ragged tail (seqlen % 16) is handled bytewise by the row's last thread.
template <bool SILU, int PIECES, bool BATCH_INNER>
__global__ __launch_bounds__(kConvThreads) void conv_fwd_rows_kernel(QaConvParams p, int segs) {
    // grid: x over runs of PIECES * 64 segments of a row (one wave each), y over groups of four channels
    // (one per wave), z = batch: no integer division on the way in, and the channel is the same for a
    // whole wave, so its taps and bias are fetched and packed once per wave by scalar instructions.
    // A lane takes segment 64*k + lane of its wave's run, k < PIECES: every load of a wave is 1 KB in one piece.
    // BATCH_INNER, for buffers in which the batch entries of one channel lie next to each other (the layout
    // in_proj writes): y over groups of four batch entries (one per wave), z = channel, so that the workgroups
    // sweep the buffer from one end to the other in the order they are dispatched.
    const int mine = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.y * 4 + (threadIdx.x >> 6)));
    const int c = BATCH_INNER ? static_cast<int>(blockIdx.z) : mine;
    const int b = BATCH_INNER ? mine : static_cast<int>(blockIdx.z);
    const int seg0 = blockIdx.x * (64 * PIECES) + (threadIdx.x & 63);
    if (c >= p.dim || b >= p.batch || seg0 >= segs) return;
    const int8_t* x = p.x + b * p.x_batch_stride + c * p.x_c_stride;
    int8_t* out = p.out + b * p.out_batch_stride + c * p.out_c_stride;

    // the row's bytes are requested first; taps, bias and scales arrive while they travel
    uint32_t w[PIECES][5];   // w[k][0] = x[t0-4 .. t0-1], w[k][1..4] = x[t0 .. t0+15]
#pragma unroll
    for (int k = 0; k < PIECES; ++k) {
        const int seg = seg0 + 64 * k;
        const int t0 = seg * 16;
        const int remaining = p.seqlen - t0;
        if (seg >= segs) break;
        w[k][0] = seg > 0 ? *reinterpret_cast<const uint32_t*>(x + t0 - 4) : 0u;
        if (remaining >= 16) {
            const uint4 v = *reinterpret_cast<const uint4*>(x + t0);
            w[k][1] = v.x; w[k][2] = v.y; w[k][3] = v.z; w[k][4] = v.w;
        } else {
            w[k][1] = w[k][2] = w[k][3] = w[k][4] = 0u;
            for (int i = 0; i < remaining; ++i) {
                w[k][1 + (i >> 2)] |= static_cast<uint32_t>(static_cast<uint8_t>(x[t0 + i])) << (8 * (i & 3));
            }
        }
    }
    // Taps and bias of the wave's channel: one scalar load each when the four taps are an aligned word and the
    // bias vector consists of whole aligned words (the usual case), else byte by byte.
    const int8_t* taps_at = p.weight + c * p.weight_c_stride;
    uint32_t taps;
    if (p.width == 4 && p.weight_width_stride == 1 && aligned4(taps_at)) taps = *reinterpret_cast<const uint32_t*>(taps_at);
    else taps = pack_taps(taps_at, p.weight_width_stride, p.width);
    float bias_f = 0.0f;
    if (p.bias) {
        int bias_q;
        if (aligned4(p.bias) && (p.dim & 3) == 0)
            bias_q = static_cast<int8_t>(reinterpret_cast<const uint32_t*>(p.bias)[c >> 2] >> (8 * (c & 3)));
        else bias_q = p.bias[c];
        bias_f = static_cast<float>(bias_q) * p.scale_b;
    }
    const float s_wx = p.scale_w * p.scale_x;
    const float inv_s_out = 1.0f / p.scale_out;
    const bool exact_only = conv_needs_exact_route(p.scale_out);
    const ConvQuantRegs kq(p.scale_out);
#pragma unroll
    for (int k = 0; k < PIECES; ++k) {
        const int seg = seg0 + 64 * k;
        const int t0 = seg * 16;
        const int remaining = p.seqlen - t0;
        if (seg >= segs) break;
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // window ending at element 4q+j: bytes (4q+j-3 .. 4q+j) of the stream starting at w[k][1]
                const uint32_t win = j == 3 ? w[k][q + 1] : __builtin_amdgcn_alignbyte(w[k][q + 1], w[k][q], j + 1);
                v[j] = __builtin_fmaf(s_wx, static_cast<float>(dot4(win, taps)), bias_f);
            }
            o[q] = conv_quant4(v, p.scale_out, inv_s_out, SILU, exact_only, kq);
        }
        if (remaining >= 16) {
            *reinterpret_cast<uint4*>(out + t0) = make_uint4(o[0], o[1], o[2], o[3]);
        } else {
            for (int i = 0; i < remaining; ++i) {
                out[t0 + i] = static_cast<int8_t>((o[i >> 2] >> (8 * (i & 3))) & 0xff);
            }
        }
    }
}

// The same arithmetic for a tile of 64 channels x 64 time steps per workgroup, writing the output twice:
// in the input's layout (16 bytes per thread, as above) and with channels contiguous, (batch, seqlen, dim).
// Thread (channel tid/4, segment tid%4) computes 16 steps of one channel; the 64 x 64 byte tile then
// passes through LDS and thread (step tid/4, piece tid%4) gathers 16 channels of one step.
template <bool SILU>
__global__ __launch_bounds__(kConvThreads) void conv_fwd_rows_dual_kernel(QaConvParams p, int tiles_l, int tiles_c) {
    constexpr int kPitch = 80;                       // bytes per staged channel row (16-byte aligned, 64 used)
    __shared__ __attribute__((aligned(16))) uint8_t s_tile[64 * kPitch];
    const int tid = threadIdx.x;
    const int tl = blockIdx.x % tiles_l;
    const int tc = (blockIdx.x / tiles_l) % tiles_c;
    const int b = blockIdx.x / (tiles_l * tiles_c);
    const int c_local = tid >> 2, seg = tid & 3;
    const int c = tc * 64 + c_local;
    const int t0 = tl * 64 + seg * 16;
    const int remaining = p.seqlen - t0;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
    if (c < p.dim && remaining > 0) {
        const int8_t* x = p.x + b * p.x_batch_stride + c * p.x_c_stride;
        int8_t* out = p.out + b * p.out_batch_stride + c * p.out_c_stride;
        // the row's bytes are requested first; taps, bias and scales arrive while they travel
        uint32_t w[5];   // w[0] = x[t0-4 .. t0-1], w[1..4] = x[t0 .. t0+15]
        w[0] = t0 > 0 ? *reinterpret_cast<const uint32_t*>(x + t0 - 4) : 0u;
        if (remaining >= 16) {
            const uint4 v = *reinterpret_cast<const uint4*>(x + t0);
            w[1] = v.x; w[2] = v.y; w[3] = v.z; w[4] = v.w;
        } else {
            w[1] = w[2] = w[3] = w[4] = 0u;
            for (int i = 0; i < remaining; ++i) {
                w[1 + (i >> 2)] |= static_cast<uint32_t>(static_cast<uint8_t>(x[t0 + i])) << (8 * (i & 3));
            }
        }
        const int8_t* taps_at = p.weight + c * p.weight_c_stride;
        uint32_t taps;
        if (p.width == 4 && p.weight_width_stride == 1 && aligned4(taps_at)) taps = *reinterpret_cast<const uint32_t*>(taps_at);
        else taps = pack_taps(taps_at, p.weight_width_stride, p.width);
        const float s_wx = p.scale_w * p.scale_x;
        const float bias_f = p.bias ? static_cast<float>(p.bias[c]) * p.scale_b : 0.0f;
        const float inv_s_out = 1.0f / p.scale_out;
        const bool exact_only = conv_needs_exact_route(p.scale_out);
        const ConvQuantRegs kq(p.scale_out);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t win = j == 3 ? w[q + 1] : __builtin_amdgcn_alignbyte(w[q + 1], w[q], j + 1);
                v[j] = __builtin_fmaf(s_wx, static_cast<float>(dot4(win, taps)), bias_f);
            }
            o[q] = conv_quant4(v, p.scale_out, inv_s_out, SILU, exact_only, kq);
        }
        if (remaining >= 16) {
            *reinterpret_cast<uint4*>(out + t0) = make_uint4(o[0], o[1], o[2], o[3]);
        } else {
            for (int i = 0; i < remaining; ++i) out[t0 + i] = static_cast<int8_t>((o[i >> 2] >> (8 * (i & 3))) & 0xff);
        }
    }
    *reinterpret_cast<uint4*>(s_tile + c_local * kPitch + seg * 16) = make_uint4(o[0], o[1], o[2], o[3]);
    __syncthreads();
    const int t_local = tid >> 2, piece = tid & 3;
    const int t = tl * 64 + t_local;
    const int cc0 = tc * 64 + piece * 16;
    if (t >= p.seqlen || cc0 >= p.dim) return;
    uint32_t g[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) g[i >> 2] |= static_cast<uint32_t>(s_tile[(piece * 16 + i) * kPitch + t_local]) << (8 * (i & 3));
    int8_t* dst = p.out_t + b * p.out_t_batch_stride + t * p.out_t_l_stride + cc0;
    if (cc0 + 16 <= p.dim && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
        *reinterpret_cast<uint4*>(dst) = make_uint4(g[0], g[1], g[2], g[3]);
    } else {
        for (int i = 0; i < 16 && cc0 + i < p.dim; ++i) dst[i] = static_cast<int8_t>((g[i >> 2] >> (8 * (i & 3))) & 0xff);
    }
}

// Any strides, one thread per output element.  kTapWise selects the channel-contiguous op order.
// Lanes run along the contiguous dimension chosen by the host (lanes_along_l).
template <bool kTapWise>
__global__ __launch_bounds__(kConvThreads) void conv_fwd_generic_kernel(QaConvParams p, int lanes_along_l) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kConvThreads + threadIdx.x;
    const int64_t total = static_cast<int64_t>(p.batch) * p.dim * p.seqlen;
    if (idx >= total) return;
    int b, c, t;
    if (lanes_along_l) {
        t = static_cast<int>(idx % p.seqlen);
        c = static_cast<int>((idx / p.seqlen) % p.dim);
        b = static_cast<int>(idx / (static_cast<int64_t>(p.seqlen) * p.dim));
    } else {
        c = static_cast<int>(idx % p.dim);
        t = static_cast<int>((idx / p.dim) % p.seqlen);
        b = static_cast<int>(idx / (static_cast<int64_t>(p.seqlen) * p.dim));
    }
    const int8_t* x = p.x + b * p.x_batch_stride + c * p.x_c_stride;
    const int8_t* w = p.weight + c * p.weight_c_stride;
    const float s_wx = p.scale_w * p.scale_x;
    const float bias_f = p.bias ? static_cast<float>(p.bias[c]) * p.scale_b : 0.0f;
    float v;
    if (kTapWise) {
        v = bias_f;
        for (int k = 0; k < p.width; ++k) {
            const int ti = t - (p.width - 1 - k);
            const float xv = ti >= 0 ? static_cast<float>(x[ti * p.x_l_stride]) : 0.0f;
            const float wv = static_cast<float>(w[k * p.weight_width_stride]);
            v = __builtin_fmaf(s_wx * wv, xv, v);
        }
    } else {
        int acc = 0;
        for (int k = 0; k < p.width; ++k) {
            const int ti = t - (p.width - 1 - k);
            const int xv = ti >= 0 ? x[ti * p.x_l_stride] : 0;
            acc += xv * static_cast<int>(w[k * p.weight_width_stride]);
        }
        v = __builtin_fmaf(s_wx, static_cast<float>(acc), bias_f);
    }
    p.out[b * p.out_batch_stride + c * p.out_c_stride + t * p.out_l_stride] =
        conv_epilogue(v, p.scale_out, p.silu_activation);
}

// Decode step: one thread per (batch, channel); lanes along channels so x/out are coalesced.
__global__ __launch_bounds__(kConvThreads) void conv_update_kernel(QaConvParams p) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kConvThreads + threadIdx.x;
    if (idx >= static_cast<int64_t>(p.batch) * p.dim) return;
    const int c = static_cast<int>(idx % p.dim);
    const int b = static_cast<int>(idx / p.dim);
    conv_step_row<0>(p, b, c, true);
}

// (a call over no elements - no batch entries, no channels, forward: no steps - may pass null tensors)
int validate_common(const QaConvParams* p, bool update) {
    if (!p) return QA_ERR_NULL;
    if (p->batch < 0 || p->dim < 0 || p->seqlen < 0) return QA_ERR_SHAPE;
    const bool empty = p->batch == 0 || p->dim == 0 || (!update && p->seqlen == 0);
    if (!empty && (!p->x || !p->weight || !p->out)) return QA_ERR_NULL;
    if (!empty && update && !p->conv_state) return QA_ERR_NULL;
    if (p->width < 2 || p->width > 4) return QA_ERR_SHAPE;
    return QA_OK;
}

}  // namespace
}  // namespace qa

extern "C" int qa_causal_conv1d_fwd(const QaConvParams* p, void* stream_) {
    using namespace qa;
    int st = validate_common(p, false);
    if (st != QA_OK) return st;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t total = static_cast<int64_t>(p->batch) * p->dim * p->seqlen;
    if (total == 0) return QA_OK;
    const bool l_contig = p->x_l_stride == 1 || p->seqlen == 1;
    const bool c_contig = p->x_c_stride == 1 || p->dim == 1;
    if (!l_contig && !c_contig) return QA_ERR_STRIDE;
    const bool channel_last = !l_contig || (p->x_c_stride == 1 && p->x_l_stride > 1);
    if (!channel_last) {
        const bool rows_ok = p->out_l_stride == 1 && aligned16(p->x) && aligned16(p->out) &&
                             p->x_batch_stride % 16 == 0 && p->x_c_stride % 16 == 0 &&
                             p->out_batch_stride % 16 == 0 && p->out_c_stride % 16 == 0;
        if (p->out_t && !rows_ok) return QA_ERR_STRIDE;
        if (rows_ok && p->out_t) {
            const int tiles_l = (p->seqlen + 63) / 64, tiles_c = (p->dim + 63) / 64;
            const int64_t blocks = static_cast<int64_t>(p->batch) * tiles_l * tiles_c;
            if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
            if (p->silu_activation) hipLaunchKernelGGL(conv_fwd_rows_dual_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(kConvThreads), 0, stream, *p, tiles_l, tiles_c);
            else hipLaunchKernelGGL(conv_fwd_rows_dual_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(kConvThreads), 0, stream, *p, tiles_l, tiles_c);
            return check_launch();
        }
        if (rows_ok) {
            const int segs = (p->seqlen + 15) / 16;
            const int64_t groups = (static_cast<int64_t>(p->dim) + 3) / 4;
            if (groups > 65535 || p->batch > 65535) return QA_ERR_SHAPE;
            // two segments per lane once a row has at least 128 of them (2048 steps)
            const int pieces = segs >= 128 ? 2 : 1;
            const unsigned runs = static_cast<unsigned>((segs + 64 * pieces - 1) / (64 * pieces));
            // the batch entries of a channel next to each other, in input and output, and enough of them for a workgroup
            const bool batch_inner = p->batch >= 4 && p->dim <= 65535 && p->x_batch_stride < p->x_c_stride &&
                                     p->out_batch_stride < p->out_c_stride;
            const dim3 grid = batch_inner ? dim3(runs, static_cast<unsigned>((p->batch + 3) / 4), static_cast<unsigned>(p->dim))
                                          : dim3(runs, static_cast<unsigned>(groups), static_cast<unsigned>(p->batch));
            auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(kConvThreads), 0, stream, *p, segs); };
            auto pick = [&](auto silu, auto pcs) {
                constexpr bool S = decltype(silu)::value;
                constexpr int P = decltype(pcs)::value;
                batch_inner ? go(conv_fwd_rows_kernel<S, P, true>) : go(conv_fwd_rows_kernel<S, P, false>);
            };
            using T = std::true_type; using F = std::false_type;
            using P1 = std::integral_constant<int, 1>; using P2 = std::integral_constant<int, 2>;
            if (pieces == 2) p->silu_activation ? pick(T{}, P2{}) : pick(F{}, P2{});
            else p->silu_activation ? pick(T{}, P1{}) : pick(F{}, P1{});
            return check_launch();
        }
    }
    if (p->out_t) return QA_ERR_STRIDE;               // the second output exists for the seqlen-contiguous layout only
    const int64_t blocks = (total + kConvThreads - 1) / kConvThreads;
    if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
    if (channel_last) {
        hipLaunchKernelGGL(conv_fwd_generic_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(kConvThreads),
                           0, stream, *p, 0);
    } else {
        hipLaunchKernelGGL(conv_fwd_generic_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(kConvThreads),
                           0, stream, *p, 1);
    }
    return check_launch();
}

extern "C" int qa_causal_conv1d_update(const QaConvParams* p, void* stream_) {
    using namespace qa;
    int st = validate_common(p, true);
    if (st != QA_OK) return st;
    if (p->conv_state_len != p->width && p->conv_state_len != p->width - 1) return QA_ERR_SHAPE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t total = static_cast<int64_t>(p->batch) * p->dim;
    if (total == 0) return QA_OK;
    const int64_t blocks = (total + kConvThreads - 1) / kConvThreads;
    hipLaunchKernelGGL(conv_update_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kConvThreads), 0, stream, *p);
    return check_launch();
}
