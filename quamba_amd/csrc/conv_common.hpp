// Pieces shared by the int8 causal conv kernels (Mamba1 conv and Mamba2 xBC conv): the SiLU +
// requantisation epilogue in its exact and its cheap-with-fallback form, and tap packing for the
// four-way int8 dot product.
#pragma once
#include "qa_common.hpp"

namespace qa {

__device__ __forceinline__ int8_t conv_epilogue(float v, float s_out, int silu) {
    if (silu) v = v / (1.0f + exp_det(-v));
    return sat8_half_away(v / s_out);
}

// Requantised output by the cheap route (hardware exp2 / rcp, multiply by 1/s_out, round to nearest)
// whenever that provably equals the exact route, else by the exact route.  The cheap value y differs
// from the exactly-evaluated one by less than 3.3e-4 for |y| < 129 and v >= -16: the exponent argument
// v * log2(e) is rounded twice (a relative error of 1e-7 |v| in the exponential), exp2, rcp and the exact
// route's own steps are each within 1-1.5 ulp, together below 2.5e-6 relative.  So if y is further than
// 5e-4 from every half-integer both round to the same integer (a margin proportional to |y| was tried
// and measured no faster).  y is clamped to +-128.75 first: beyond that both routes saturate, and the
// clamped value (a quarter away from 129) passes the test on its own.  For v < -16 the bound no longer
// holds, but there |y| < 1.8e-6 / s_out: with s_out >= 1e-5 both routes give zero, and for smaller
// output scales the caller sets `exact_only` and every lane takes the exact route.
// A wave takes the exact route whenever one of its 64 lanes does, which is why the margin is kept as
// narrow as the error bound allows (at 2e-3, 0.4 % of the lanes, a quarter of all wave-elements went
// through the exact route's ~100 instructions).
__device__ __forceinline__ bool conv_needs_exact_route(float s_out) { return !(s_out >= 1e-5f); }

// The constants of the cheap route, held in registers for the life of the thread.  They are not values an
// instruction can carry inline, and the compiler would otherwise load each of them into a register again for
// every output (three extra instructions on a path of under thirty).
struct ConvQuantRegs {
    float clamp_hi, magic;
    __device__ __forceinline__ ConvQuantRegs() {
        asm volatile("v_mov_b32 %0, 0x42fe8000" : "=v"(clamp_hi));     // 127.25
        asm volatile("v_mov_b32 %0, 0x4b400000" : "=v"(magic));        // 1.5 * 2^23
    }
};

// Returns a word whose low byte is the int8 code (the bytes above it are not meaningful).
// y is clamped to [-128.25, 127.25] first: beyond +-127.5 / -128.5 both routes saturate to the same code whatever
// side of the half-integer they fall on, and the clamped value (a quarter away from a half-integer) passes the
// distance test on its own.  Adding 1.5 * 2^23 rounds to the nearest integer in the addition itself (ties to
// even; ties are not decided here) and leaves that integer's two's-complement byte in the low 8 bits of the sum.
// the low bytes of four words, in order
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3) {
    const uint32_t lo = __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u);      // bytes: b0.0, b1.0, 0, 0
    const uint32_t hi = __builtin_amdgcn_perm(b3, b2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);                   // lo.0, lo.1, hi.0, hi.1
}

// The cheap route alone: the word with the code in its low byte, and whether the exact route must decide instead.
__device__ __forceinline__ uint32_t conv_quant_cheap(float v, float inv_s_out, int silu, const ConvQuantRegs& k, bool& undecided) {
    float y = v;
    if (silu) {
        const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896341f);
        y = v * __builtin_amdgcn_rcpf(1.0f + e);
    }
    y = __builtin_amdgcn_fmed3f(y * inv_s_out, -128.25f, k.clamp_hi);
    const float t = y + k.magic;
    const float d = __builtin_fabsf(y - (t - k.magic));
    undecided = !(d <= 0.4995f);
    return __float_as_uint(t);
}

__device__ __forceinline__ uint32_t conv_quant_bits(float v, float s_out, float inv_s_out, int silu, bool exact_only,
                                                   const ConvQuantRegs& k) {
    bool undecided;
    uint32_t q = conv_quant_cheap(v, inv_s_out, silu, k, undecided);
    if (exact_only || undecided) q = static_cast<uint32_t>(static_cast<uint8_t>(conv_epilogue(v, s_out, silu)));
    return q;
}

// Four outputs at once: the four cheap evaluations are independent and interleave (each is a chain of dependent
// instructions with two transcendentals), then every output that the cheap route could not decide - rare, so the
// branch around each is almost never taken - goes through the exact route on its own.
__device__ __forceinline__ uint32_t conv_quant4(const float (&v)[4], float s_out, float inv_s_out, int silu, bool exact_only,
                                               const ConvQuantRegs& k) {
    uint32_t q[4];
    bool undecided[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = conv_quant_cheap(v[j], inv_s_out, silu, k, undecided[j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (exact_only || undecided[j]) q[j] = static_cast<uint32_t>(static_cast<uint8_t>(conv_epilogue(v[j], s_out, silu)));
    }
    return pack_low_bytes(q[0], q[1], q[2], q[3]);
}

__device__ __forceinline__ int conv_quant(float v, float s_out, float inv_s_out, int silu, bool exact_only,
                                          const ConvQuantRegs& k) {
    return static_cast<int8_t>(conv_quant_bits(v, s_out, inv_s_out, silu, exact_only, k) & 0xffu);
}

// packed taps for sdot4: byte j of the window holds x[t-3+j]; tap for x[t-(k-1-w)] is W[w],
// so byte j pairs with W[j-(4-k)] (zero for j < 4-k).
__device__ __forceinline__ uint32_t pack_taps(const int8_t* w, int64_t wstride, int width) {
    uint32_t packed = 0;
    for (int j = 0; j < 4; ++j) {
        const int wi = j - (4 - width);
        const uint32_t b = wi >= 0 ? static_cast<uint8_t>(w[wi * wstride]) : 0u;
        packed |= b << (8 * j);
    }
    return packed;
}

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), 0, false);
}

// One decode step of channel c of batch entry b (quant_causal_conv1d_update_kernel.cuh:34-75): the conv state moves
// on by one step (in place), the window meets the taps, bias, SiLU, requantisation.  Returns the int8 output and,
// with `store`, writes state and output.  Taps and a four-wide state row are fetched as one word when their layout
// allows; the requantisation takes the cheap route whenever it provably equals the exact one (conv_quant).
// W4: four taps with unit stride and a state of four codes (conv_state_len 4, unit stride), each row one aligned
// word, known at compile time.
template <bool W4 = false>
__device__ __forceinline__ int8_t conv_step_row(const QaConvParams& p, int b, int c, bool store) {
    int8_t* st = p.conv_state + b * p.conv_state_batch_stride + c * p.conv_state_c_stride;
    const int8_t* w = p.weight + c * p.weight_c_stride;
    const int width = p.width;
    const int slen = p.conv_state_len;            // width (slot 0 is dropped) or width-1
    const int drop = slen - (width - 1);          // 1 or 0
    __attribute__((aligned(4))) int8_t xs[4], ws[4] = {0, 0, 0, 0};
    if constexpr (W4) {
        // the caller has checked: four taps in one aligned word, a state of four codes in one aligned word.  Every
        // load is issued at once (the bias through a stand-in address when there is none), no branch in between.
        const int8_t* x_a = p.x + b * p.x_batch_stride + c * p.x_c_stride;
        const uint32_t w_word4 = *reinterpret_cast<const uint32_t*>(w);
        const uint32_t row4 = *reinterpret_cast<const uint32_t*>(st);
        const int8_t x_new = *x_a;
        const int8_t bias_q = *(p.bias ? p.bias + c : x_a);
        const uint32_t win4 = (row4 >> 8) | (static_cast<uint32_t>(static_cast<uint8_t>(x_new)) << 24);
        if (store) *reinterpret_cast<uint32_t*>(st) = win4;
        *reinterpret_cast<uint32_t*>(ws) = w_word4;
        *reinterpret_cast<uint32_t*>(xs) = win4;
        const float s_wx = p.scale_w * p.scale_x;
        float v = p.bias ? static_cast<float>(bias_q) * p.scale_b : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) v = __builtin_fmaf(s_wx * static_cast<float>(ws[i]), static_cast<float>(xs[i]), v);
        const ConvQuantRegs kq;
        const int8_t q = static_cast<int8_t>(conv_quant(v, p.scale_out, 1.0f / p.scale_out, p.silu_activation,
                                                        conv_needs_exact_route(p.scale_out), kq));
        if (store && p.out) p.out[b * p.out_batch_stride + c * p.out_c_stride] = q;
        return q;
    }
    const bool w_word = width == 4 && p.weight_width_stride == 1 && (reinterpret_cast<uintptr_t>(w) & 3u) == 0;
    const bool s_word = slen == 4 && p.conv_state_l_stride == 1 && (reinterpret_cast<uintptr_t>(st) & 3u) == 0;
    if (w_word) {
        *reinterpret_cast<uint32_t*>(ws) = *reinterpret_cast<const uint32_t*>(w);
    } else {
        for (int i = 0; i < width; ++i) ws[i] = w[i * p.weight_width_stride];
    }
    if (s_word) {
        __attribute__((aligned(4))) int8_t row[4];
        *reinterpret_cast<uint32_t*>(row) = *reinterpret_cast<const uint32_t*>(st);
        for (int i = 0; i < width - 1; ++i) xs[i] = row[i + drop];
    } else {
        for (int i = 0; i < width - 1; ++i) xs[i] = st[(i + drop) * p.conv_state_l_stride];
    }
    xs[width - 1] = p.x[b * p.x_batch_stride + c * p.x_c_stride];
    const float bias_f = p.bias ? static_cast<float>(p.bias[c]) * p.scale_b : 0.0f;
    if (store) {
        if (s_word) {
            // state as long as the window: the whole window is the new state
            *reinterpret_cast<uint32_t*>(st) = *reinterpret_cast<const uint32_t*>(xs);
        } else {
            for (int i = 0; i < slen; ++i) st[i * p.conv_state_l_stride] = xs[i + (width - slen)];
        }
    }
    const float s_wx = p.scale_w * p.scale_x;
    float v = bias_f;
    for (int i = 0; i < width; ++i) v = __builtin_fmaf(s_wx * static_cast<float>(ws[i]), static_cast<float>(xs[i]), v);
    const ConvQuantRegs kq;
    const int8_t q = static_cast<int8_t>(conv_quant(v, p.scale_out, 1.0f / p.scale_out, p.silu_activation,
                                                    conv_needs_exact_route(p.scale_out), kq));
    if (store && p.out) p.out[b * p.out_batch_stride + c * p.out_c_stride] = q;
    return q;
}

}  // namespace qa
