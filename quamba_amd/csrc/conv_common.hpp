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

// Requantised output by the cheap route (hardware exp2 / rcp, round to nearest) whenever that provably equals the
// exact route, else by the exact route.  The cheap route forms y = v / (s_out (1 + E)), E = 2^(-v log2 e), with one
// reciprocal: SiLU and the division by the output scale share it.  Relative to the true value, for v >= -16:
//   cheap route: E carries 7.3e-8 |v| (its argument is rounded twice) + 1.2e-7 (exp2, 1 ulp), which enters 1 + E with
//                the weight E / (1 + E); then 6e-8 (fused multiply-add), 1.2e-7 (rcp, 1 ulp), 6e-8 (product);
//   exact route: 1.8e-7 (exp_det, 1.5 ulp) with the same weight; then 6e-8 each for the sum and the two divisions.
// v >= 0: the weight is at most one half and |v| E / (1 + E) <= 0.28, so the two routes differ by less than 5.9e-7 |y|,
//         7.6e-5 for |y| <= 128.25.
// v <  0: they differ by less than (7.3e-8 |v| + 7.2e-7) |y| and |y| = |v| / (s_out (1 + e^|v|)); the product of the
//         two is at most 2.3e-7 / s_out: 9.2e-5 for s_out >= 2.5e-3.  For smaller output scales |y| can reach 128 at
//         v = -16, where the difference is below 2.6e-6 |y| = 3.3e-4.
// So if y is further than the margin - 1.25e-4 for s_out >= 2.5e-3, 5e-4 below - from every half-integer, both
// routes round to the same integer.  y is clamped to [-128.25, 127.25] first: beyond +-127.5 / -128.5 both routes
// saturate to the same code whatever side of the half-integer they fall on, and the clamped value (a quarter away
// from a half-integer) passes the test on its own.  For v < -16 the bounds no longer hold, but there
// |y| < 1.8e-6 / s_out: with s_out >= 1e-5 both routes give zero, and for smaller output scales the caller sets
// `exact_only` and every lane takes the exact route.
// A wave takes the exact route's ~100 instructions for an output whenever one of its 64 lanes needs it, which is
// why the margin is kept as narrow as the bounds allow: at 5e-4 a wave does so for 6 % of its outputs, a third of
// the kernel's vector instructions; at 1.25e-4 for 1.6 %.
__device__ __forceinline__ bool conv_needs_exact_route(float s_out) { return !(s_out >= 1e-5f); }
__device__ __forceinline__ float conv_cheap_margin(float s_out) { return s_out >= 2.5e-3f ? 1.25e-4f : 5e-4f; }

// The constants of the cheap route, held in registers for the life of the thread.  They are not values an
// instruction can carry inline, and the compiler would otherwise load each of them into a register again for
// every output (three extra instructions on a path of under thirty).  `smallest_s_out`: the smallest output scale
// the thread will requantise with.
struct ConvQuantRegs {
    float clamp_hi, magic, margin;
    __device__ __forceinline__ explicit ConvQuantRegs(float smallest_s_out) : margin(conv_cheap_margin(smallest_s_out)) {
        asm volatile("v_mov_b32 %0, 0x42fe8000" : "=v"(clamp_hi));     // 127.25
        asm volatile("v_mov_b32 %0, 0x4b400000" : "=v"(magic));        // 1.5 * 2^23
    }
};

// The cheap route's value in units of the output code, clamped.
__device__ __forceinline__ float conv_cheap_units(float v, float s_out, float inv_s_out, int silu, const ConvQuantRegs& k) {
    float y;
    if (silu) {
        const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896341f);
        y = v * __builtin_amdgcn_rcpf(__builtin_fmaf(e, s_out, s_out));
    } else {
        y = v * inv_s_out;
    }
    return __builtin_amdgcn_fmed3f(y, -128.25f, k.clamp_hi);
}
// Signed distance of y's fractional part from one half (exact for the values that matter: the fraction of |y| < 129
// is exact, and so is the subtraction for fractions of a quarter and more); the cheap route decides when its
// magnitude is at least the margin.
__device__ __forceinline__ float conv_cheap_off_half(float y) { return __builtin_amdgcn_fractf(y) - 0.5f; }

// One output: a word whose low byte is the int8 code (the bytes above it are not meaningful).  Adding 1.5 * 2^23
// rounds to the nearest integer in the addition itself (ties to even; ties are not decided here) and leaves that
// integer's two's-complement byte in the low 8 bits of the sum.
__device__ __forceinline__ uint32_t conv_quant_bits(float v, float s_out, float inv_s_out, int silu, bool exact_only,
                                                   const ConvQuantRegs& k) {
    const float y = conv_cheap_units(v, s_out, inv_s_out, silu, k);
    uint32_t q = __float_as_uint(y + k.magic);
    if (exact_only || !(__builtin_fabsf(conv_cheap_off_half(y)) >= k.margin))
        q = static_cast<uint32_t>(static_cast<uint8_t>(conv_epilogue(v, s_out, silu)));
    return q;
}

// Four outputs at once, as the four bytes of a word: the four cheap evaluations are independent and interleave (each
// is a chain of dependent instructions with two transcendentals); the rounding additions of the second to fourth
// output write their low byte straight into its place (sub-dword destination select, the other bytes preserved), so
// nothing is spent on packing; one comparison on the smallest of the four distances decides whether any output goes
// through the exact route - rare, so the branch is almost never taken.
__device__ __forceinline__ uint32_t conv_quant4(const float (&v)[4], const float (&s_out)[4], const float (&inv_s_out)[4], int silu,
                                               const bool (&exact_only)[4], const ConvQuantRegs& k) {
    float y[4], off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) y[j] = conv_cheap_units(v[j], s_out[j], inv_s_out[j], silu, k);
    uint32_t word = __float_as_uint(y[0] + k.magic);                     // byte 0; bytes 1..3 replaced below
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(y[1]), "v"(k.magic));
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(y[2]), "v"(k.magic));
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(y[3]), "v"(k.magic));
#pragma unroll
    for (int j = 0; j < 4; ++j) off[j] = conv_cheap_off_half(y[j]);
    float nearest;                                                       // min |off[j]|: two instructions
    asm("v_min3_f32 %0, |%1|, |%2|, |%3|" : "=v"(nearest) : "v"(off[0]), "v"(off[1]), "v"(off[2]));
    asm("v_min_f32_e64 %0, %1, |%2|" : "=v"(nearest) : "v"(nearest), "v"(off[3]));
    const bool any_exact = exact_only[0] || exact_only[1] || exact_only[2] || exact_only[3];
    if (any_exact || !(nearest >= k.margin)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (exact_only[j] || !(__builtin_fabsf(off[j]) >= k.margin)) {
                const uint32_t code = static_cast<uint8_t>(conv_epilogue(v[j], s_out[j], silu));
                word = (word & ~(0xffu << (8 * j))) | (code << (8 * j));
            }
        }
    }
    return word;
}
// the same with one output scale for the four
__device__ __forceinline__ uint32_t conv_quant4(const float (&v)[4], float s_out, float inv_s_out, int silu, bool exact_only,
                                               const ConvQuantRegs& k) {
    const float s[4] = {s_out, s_out, s_out, s_out}, inv[4] = {inv_s_out, inv_s_out, inv_s_out, inv_s_out};
    const bool ex[4] = {exact_only, exact_only, exact_only, exact_only};
    return conv_quant4(v, s, inv, silu, ex, k);
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

// Asked for with the clamp flag (saturation of the 32-bit sum, which four products of bytes never reach): that
// selects the three-operand form with a literal zero as the addend; without it the compiler picks the accumulating
// two-operand form, which costs a register clear per product.
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), 0, true);
}

// One decode step of channel c of batch entry b (quant_causal_conv1d_update_kernel.cuh:34-75): the conv state moves
// on by one step (in place), the window meets the taps, bias, SiLU, requantisation.  Returns the int8 output and,
// with `store`, writes state and output.  Taps and a four-wide state row are fetched as one word when their layout
// allows; the requantisation takes the cheap route whenever it provably equals the exact one (conv_quant).
// FIXED 4: four taps with unit stride and a state of four codes (conv_state_len 4, unit stride), each row one aligned
// word, known at compile time.  FIXED 3: four taps in one aligned word and a state of three codes per row, the rows
// back to back in memory ([batch, dim, 3] contiguous): a row is read with one unaligned word, whose fourth byte
// belongs to the next row and is not used (the last row of the tensor reads the word that ends with it instead),
// and written back as three bytes.
template <int FIXED = 0>
__device__ __forceinline__ int8_t conv_step_row(const QaConvParams& p, int b, int c, bool store) {
    int8_t* st = p.conv_state + b * p.conv_state_batch_stride + c * p.conv_state_c_stride;
    const int8_t* w = p.weight + c * p.weight_c_stride;
    const int width = p.width;
    const int slen = p.conv_state_len;            // width (slot 0 is dropped) or width-1
    const int drop = slen - (width - 1);          // 1 or 0
    __attribute__((aligned(4))) int8_t xs[4], ws[4] = {0, 0, 0, 0};
    if constexpr (FIXED != 0) {
        // the caller has checked: four taps in one aligned word, a state of four codes in one aligned word or of
        // three codes in back-to-back rows.  Every load is issued at once (the bias through a stand-in address when
        // there is none), no branch in between.
        const int8_t* x_a = p.x + b * p.x_batch_stride + c * p.x_c_stride;
        const uint32_t w_word4 = *reinterpret_cast<const uint32_t*>(w);
        uint32_t held;                     // the codes the window keeps, in its low three bytes
        if constexpr (FIXED == 4) {
            held = *reinterpret_cast<const uint32_t*>(st) >> 8;
        } else {
            const int last = (b == p.batch - 1 && c == p.dim - 1) ? 1 : 0;
            uint32_t word;
            __builtin_memcpy(&word, st - last, 4);               // (an unaligned load)
            held = (last ? word >> 8 : word) & 0x00ffffffu;
        }
        const int8_t x_new = *x_a;
        const int8_t bias_q = *(p.bias ? p.bias + c : x_a);
        const uint32_t win4 = held | (static_cast<uint32_t>(static_cast<uint8_t>(x_new)) << 24);
        if (store) {
            if constexpr (FIXED == 4) {
                *reinterpret_cast<uint32_t*>(st) = win4;
            } else {
                st[0] = static_cast<int8_t>(win4 >> 8);
                st[1] = static_cast<int8_t>(win4 >> 16);
                st[2] = x_new;
            }
        }
        *reinterpret_cast<uint32_t*>(ws) = w_word4;
        *reinterpret_cast<uint32_t*>(xs) = win4;
        const float s_wx = p.scale_w * p.scale_x;
        float v = p.bias ? static_cast<float>(bias_q) * p.scale_b : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) v = __builtin_fmaf(s_wx * static_cast<float>(ws[i]), static_cast<float>(xs[i]), v);
        const ConvQuantRegs kq(p.scale_out);
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
    const ConvQuantRegs kq(p.scale_out);
    const int8_t q = static_cast<int8_t>(conv_quant(v, p.scale_out, 1.0f / p.scale_out, p.silu_activation,
                                                    conv_needs_exact_route(p.scale_out), kq));
    if (store && p.out) p.out[b * p.out_batch_stride + c * p.out_c_stride] = q;
    return q;
}

}  // namespace qa
