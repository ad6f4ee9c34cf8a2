// Mamba1 int8 selective scan: forward over a sequence, and the single-token state update.
//
// Arithmetic (reference csrc/selective_scan/quant_sscan_fwd_kernel.cuh:110-293):
//   u = s_u q_u;  dt = softplus20(s_dt q_dt + s_db q_db[d]);  A[n] = -exp(s_A q_Alog[d,n])
//   h[n] = exp(dt A[n]) h[n] + (s_B q_B[n,t]) (dt u);  y = D u + sum_n h[n] (s_C q_C[n,t]);  y *= silu(s_z q_z)
// Output fp16 (tolerance, not bits): exp runs on the hardware exp2 with A pre-multiplied by log2(e).
//
// Mapping for gfx950.  The recurrence is sequential in time and costs one transcendental plus four
// multiply-adds per (channel, step, state), which is more VALU time than the bytes cost HBM time,
// so the kernel walks time once, keeps the state in registers and never recomputes:
//   * a lane owns one channel and NPL of its states; NSPLIT neighbouring lanes share a channel
//     (their partial dot products meet in a cross-lane add), so the number of waves can be raised
//     without a second pass over time;
//   * u / dt / z rows are staged through LDS in tiles of T steps with 16-byte global loads, rows
//     padded so the per-lane dword reads are bank-conflict free;
//   * B and C (shared by every channel of a batch entry) are converted to fp32 and scaled once per
//     workgroup and read from LDS as 16-byte broadcasts;
//   * the fp16 output is staged through LDS so each time step is written as one contiguous run of
//     channels in the (batch, seqlen, dim) tensor - no transposition pass afterwards;
//   * global loads of tile i+1 are issued before the arithmetic of tile i and held in registers
//     until the tile has been consumed, then written to LDS.
#include "qa_common.hpp"
#include "conv_common.hpp"

namespace qa {
namespace {

constexpr float kLog2e = 1.44269504088896341f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// float(int8 code in byte n of w) in one instruction (the sub-dword operand select converts the byte in place; the
// compiler, left to itself, shifts and sign-extends the byte out first)
__device__ __forceinline__ float code_byte_to_float(uint32_t w, int n) {
    float r;
    switch (n) {
        case 0: asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(r) : "v"(w)); break;
        case 1: asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(r) : "v"(w)); break;
        case 2: asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(r) : "v"(w)); break;
        default: asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(r) : "v"(w)); break;
    }
    return r;
}

// softplus with the reference's threshold; log1p evaluated so that small exp(x) keeps full
// relative accuracy (series below 2^-6, log2 above).
__device__ __forceinline__ float softplus20(float x) {
    if (x > 20.0f) return x;
    const float e = fast_exp2(x * kLog2e);
    const float series = e * __builtin_fmaf(e, __builtin_fmaf(e, __builtin_fmaf(e, -0.25f, 1.0f / 3.0f), -0.5f), 1.0f);
    const float big = fast_log2(1.0f + e) * 0.693147180559945309f;
    return e < 0.015625f ? series : big;
}

// The same function without a branch and with one rounding compensated instead of a series:
//   softplus(x) = max(x, 0) + log1p(e),  e = exp(-|x|) in (0, 1]
//   u = fl(1 + e) = 1 + e + r with r = (u - 1) - e exact, so log1p(e) = ln(u - r) = ln u - r / u + ..., and with
//   u in [1, 2] taking r for r / u is wrong by less than 2^-24 of the result.
// Above the threshold the second term is below half an ulp of x, so x comes back exactly, as the reference returns it.
__device__ __forceinline__ float softplus20_flat(float x) {
    const float e = fast_exp2(__builtin_fabsf(x) * -kLog2e);
    const float u = 1.0f + e;
    const float r = (u - 1.0f) - e;
    const float sp = __builtin_fmaf(fast_log2(u), 0.693147180559945309f, -r);
    float pos;                                        // max(x, 0): written out, because the builtins put a second
    asm("v_max_f32 %0, 0, %1" : "=v"(pos) : "v"(x));  // maximum of x with itself in front of it (quieting of NaNs)
    return pos + sp;
}

__device__ __forceinline__ float silu_gate(float z) {
    return z * fast_rcp(1.0f + fast_exp2(-z * kLog2e));
}

// Value of `v` in the lane of this quad that holds slice SRC of the same channel (NSPLIT lanes per
// channel, NSPLIT in {1,2,4}), as a DPP quad permutation that the compiler folds into the consumer.
template <int NSPLIT, int SRC>
__device__ __forceinline__ float quad_bcast(float v) {
    if (NSPLIT == 1) return v;
    constexpr int ctrl = NSPLIT == 4 ? (SRC | (SRC << 2) | (SRC << 4) | (SRC << 6))
                                     : (SRC | (SRC << 2) | ((2 + SRC) << 4) | ((2 + SRC) << 6));
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false);
    return __builtin_bit_cast(float, r);
}
// Same with a source slice that is a constant only after loop unrolling.
template <int NSPLIT>
__device__ __forceinline__ float quad_bcast_sel(float v, int src) {
    switch (src) {
        case 0: return quad_bcast<NSPLIT, 0>(v);
        case 1: return quad_bcast<NSPLIT, 1>(v);
        case 2: return quad_bcast<NSPLIT, (NSPLIT > 2 ? 2 : 0)>(v);
        default: return quad_bcast<NSPLIT, (NSPLIT > 2 ? 3 : 1)>(v);
    }
}
// Value of `v` in lane (lane ^ M) of the quad, M in {1,2}.
template <int M>
__device__ __forceinline__ float quad_xor(float v) {
    constexpr int ctrl = M == 1 ? (1 | (0 << 2) | (3 << 4) | (2 << 6)) : (2 | (3 << 2) | (0 << 4) | (1 << 6));
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false);
    return __builtin_bit_cast(float, r);
}

__device__ __forceinline__ float i8_of(uint32_t word, int j) {
    return static_cast<float>(static_cast<int8_t>((word >> (8 * j)) & 0xffu));
}

// 16 bytes starting at row[t]; bytes at or beyond t_end read as zero.
__device__ __forceinline__ uint4 load16(const int8_t* row, int t, int t_end, bool vec) {
    if (vec && t + 16 <= t_end) return *reinterpret_cast<const uint4*>(row + t);
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    for (int i = 0; i < 16; ++i) {
        if (t + i < t_end) w[i >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(row[t + i])) << (8 * (i & 3));
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <int NPL, int NSPLIT, int T, int WAVES>
struct ScanCfg {
    static constexpr int kThreads = 64 * WAVES;
    static constexpr int kCh = kThreads / NSPLIT;          // channels per workgroup
    static constexpr int kNP = NPL * NSPLIT;               // padded state count
    static constexpr int kRow = T + 4;                     // staged row pitch in bytes
    static constexpr int kInPieces = (kCh * T / 16 + kThreads - 1) / kThreads;       // per tensor
    static constexpr int kBcPieces = (2 * kNP * T / 16 + kThreads - 1) / kThreads;
    static constexpr int kOutPitch = kCh + 8;              // halves; keeps rows 16-byte aligned
};

// LDS of one workgroup
template <class Cfg, int T>
struct ScanSmem {
    __attribute__((aligned(16))) uint32_t in[3][Cfg::kCh * Cfg::kRow / 4];
    __attribute__((aligned(16))) float bc[T][2][Cfg::kNP];
    __attribute__((aligned(16))) __half out[T][Cfg::kOutPitch];
    float gate[256];                   // SiLU gate per z code (indexed by the raw byte)
};

// One workgroup: channels c0 .. c0 + kCh - 1 of batch entry b.
template <int NPL, int NSPLIT, int T, int WAVES>
__device__ __forceinline__ void sscan_fwd_body(const QaSScanParams& p, int vec_in, int vec_bc, int vec_out, int c0, int b,
                                               ScanSmem<ScanCfg<NPL, NSPLIT, T, WAVES>, T>& sm) {
    using Cfg = ScanCfg<NPL, NSPLIT, T, WAVES>;
    constexpr int kThreads = Cfg::kThreads, kCh = Cfg::kCh, kNP = Cfg::kNP, kRow = Cfg::kRow;
    constexpr int kInPieces = Cfg::kInPieces, kBcPieces = Cfg::kBcPieces;
    constexpr int kPiecesPerRow = T / 16;
    // Lanes that share the per-step work and reduce together: the NSPLIT lanes of a channel, at most a quad.
    // With eight lanes per channel the two quads each do the per-step work for themselves (it costs a lane
    // what it costs with four) and their partial sums meet in one cross-lane add per four steps.
    constexpr int QS = NSPLIT < 4 ? NSPLIT : 4;
    auto& s_in = sm.in;
    auto& s_bc = sm.bc;
    auto& s_out = sm.out;
    auto& s_gate = sm.gate;

    const int tid = threadIdx.x;
    const int c_local = tid / NSPLIT;
    const int slice = tid % NSPLIT;
    const int qslice = slice % QS;
    const int c = c0 + c_local;
    const bool c_ok = c < p.dim;
    const int cc = c_ok ? c : p.dim - 1;                   // clamped channel for parameter loads
    const int g = c0 / (p.dim / p.n_groups);
    const bool has_z = p.z != nullptr;
    const int L = p.seqlen;

    const float s_u = *p.scale_u, s_dt = *p.scale_delta, s_A = *p.scale_A, s_B = *p.scale_B, s_C = *p.scale_C;
    const float s_z = has_z ? *p.scale_z : 0.0f;
    const float D_f = p.D ? *p.scale_D * static_cast<float>(p.D[cc]) : 0.0f;
    const float db = p.delta_bias ? *p.scale_delta_bias * static_cast<float>(p.delta_bias[cc]) : 0.0f;

    float A2[NPL], h[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int n = slice * NPL + j;
        h[j] = 0.0f;
        A2[j] = n < p.dstate
                    ? -expf(s_A * static_cast<float>(p.A_log[cc * p.A_d_stride + n * p.A_dstate_stride])) * kLog2e
                    : 0.0f;
    }
    // Segments of one sequence scanned in parallel: this batch entry is segment carry_first + b and starts from
    // the state that the earlier segments (scanned from a zero state) chain up to:
    // h <- exp(A * (sum of the segment's step sizes)) h + (the segment's own end state)
    if (p.carry_state) {
        const int seg = p.carry_first + b;
        for (int sp = 0; sp < seg; ++sp) {
            const float sd = p.carry_dt_sum[static_cast<int64_t>(sp) * p.dim + cc];
#pragma unroll
            for (int j = 0; j < NPL; ++j) {
                const int n = min(slice * NPL + j, p.dstate - 1);
                h[j] = __builtin_fmaf(fast_exp2(sd * A2[j]), h[j],
                                      p.carry_state[(static_cast<int64_t>(sp) * p.dim + cc) * p.dstate + n]);
            }
        }
    }
    float dt_sum = 0.0f;                 // of the steps this lane evaluates the step size for

    const int8_t* in_base[3] = {p.u + b * p.u_batch_stride, p.delta + b * p.delta_batch_stride,
                                has_z ? p.z + b * p.z_batch_stride : nullptr};
    const int64_t in_dstride[3] = {p.u_d_stride, p.delta_d_stride, p.z_d_stride};
    const int8_t* bc_base[2] = {p.B + b * p.B_batch_stride + g * p.B_group_stride,
                                p.C + b * p.C_batch_stride + g * p.C_group_stride};
    const int64_t bc_nstride[2] = {p.B_dstate_stride, p.C_dstate_stride};
    const float bc_scale[2] = {s_B, s_C};

    uint4 r_in[3][kInPieces];
    uint4 r_bc[kBcPieces];

    auto issue_loads = [&](int t0) {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (k == 2 && !has_z) break;
#pragma unroll
            for (int i = 0; i < kInPieces; ++i) {
                const int piece = tid + i * kThreads;
                const int row = piece / kPiecesPerRow, col = piece % kPiecesPerRow;
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (piece < kCh * kPiecesPerRow && c0 + row < p.dim) {
                    v = load16(in_base[k] + (c0 + row) * in_dstride[k], t0 + col * 16, L, vec_in);
                }
                r_in[k][i] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < kBcPieces; ++i) {
            const int piece = tid + i * kThreads;
            const int which = piece / (kNP * kPiecesPerRow);
            const int rem = piece % (kNP * kPiecesPerRow);
            const int n = rem / kPiecesPerRow, col = rem % kPiecesPerRow;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (which < 2 && n < p.dstate) {
                v = load16(bc_base[which] + n * bc_nstride[which], t0 + col * 16, L, vec_bc);
            }
            r_bc[i] = v;
        }
    };

    auto stage = [&]() {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (k == 2 && !has_z) break;
#pragma unroll
            for (int i = 0; i < kInPieces; ++i) {
                const int piece = tid + i * kThreads;
                if (piece < kCh * kPiecesPerRow) {
                    const int row = piece / kPiecesPerRow, col = piece % kPiecesPerRow;
                    uint32_t* dst = &s_in[k][(row * kRow + col * 16) / 4];
                    dst[0] = r_in[k][i].x; dst[1] = r_in[k][i].y; dst[2] = r_in[k][i].z; dst[3] = r_in[k][i].w;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kBcPieces; ++i) {
            const int piece = tid + i * kThreads;
            const int which = piece / (kNP * kPiecesPerRow);
            if (which < 2) {
                const int rem = piece % (kNP * kPiecesPerRow);
                const int n = rem / kPiecesPerRow, col = rem % kPiecesPerRow;
                const uint32_t w[4] = {r_bc[i].x, r_bc[i].y, r_bc[i].z, r_bc[i].w};
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    s_bc[col * 16 + e][which][n] = bc_scale[which] * i8_of(w[e >> 2], e & 3);
                }
            }
        }
    };

    const int n_tiles = (L + T - 1) / T;
    issue_loads(0);
    if (has_z) {
        for (int i = tid; i < 256; i += kThreads) s_gate[i] = silu_gate(s_z * static_cast<float>(static_cast<int8_t>(i)));
    }
    stage();
    __syncthreads();

    for (int tile = 0; tile < n_tiles; ++tile) {
        const int t0 = tile * T;
        const int nt = min(T, L - t0);
        if (tile + 1 < n_tiles) issue_loads(t0 + T);

        const uint32_t* su = &s_in[0][c_local * kRow / 4];
        const uint32_t* sd = &s_in[1][c_local * kRow / 4];
        const uint32_t* sz = &s_in[2][c_local * kRow / 4];
        const int n_quads = (nt + 3) / 4;
        for (int tq = 0; tq < n_quads; ++tq) {
            const uint32_t u4 = su[tq], d4 = sd[tq];
            const uint32_t z4 = has_z ? sz[tq] : 0u;
            if constexpr (NSPLIT <= 4 || NSPLIT == 8) {
                // The per-step work that does not depend on the state index (dequantise, softplus,
                // gate) is shared out: of the 4 steps in this dword, the lane with slice s does
                // steps o*NSPLIT + s and the others read its results through quad DPP.
                constexpr int OWN = 4 / QS;
                float own_u[OWN], own_dt[OWN], own_du[OWN];
#pragma unroll
                for (int o = 0; o < OWN; ++o) {
                    const int j = o * QS + qslice;
                    own_u[o] = s_u * i8_of(u4, j);
                    float dt = __builtin_fmaf(s_dt, i8_of(d4, j), db);
                    if (p.delta_softplus) dt = softplus20(dt);
                    // steps past the end of the sequence must leave the state alone: a = 1, b = 0
                    dt = tq * 4 + j < nt ? dt : 0.0f;
                    own_dt[o] = dt;
                    dt_sum += dt;
                    own_du[o] = dt * own_u[o];
                }
                float acc[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int t = tq * 4 + j;
                    acc[j] = 0.0f;
                    const float dt = quad_bcast_sel<QS>(own_dt[j / QS], j % QS);
                    const float du = quad_bcast_sel<QS>(own_du[j / QS], j % QS);
                    if constexpr (NPL == 2) {
                        const float2 Bv = *reinterpret_cast<const float2*>(&s_bc[t][0][slice * NPL]);
                        const float2 Cv = *reinterpret_cast<const float2*>(&s_bc[t][1][slice * NPL]);
                        const float Bs[2] = {Bv.x, Bv.y};
                        const float Cs[2] = {Cv.x, Cv.y};
#pragma unroll
                        for (int n = 0; n < 2; ++n) {
                            const float a = fast_exp2(dt * A2[n]);
                            h[n] = __builtin_fmaf(a, h[n], Bs[n] * du);
                            acc[j] = __builtin_fmaf(h[n], Cs[n], acc[j]);
                        }
                    } else {
                        const float4* bf = reinterpret_cast<const float4*>(&s_bc[t][0][slice * NPL]);
                        const float4* cf = reinterpret_cast<const float4*>(&s_bc[t][1][slice * NPL]);
#pragma unroll
                        for (int q = 0; q < NPL / 4; ++q) {
                            const float4 Bv = bf[q];
                            const float4 Cv = cf[q];
                            const float Bs[4] = {Bv.x, Bv.y, Bv.z, Bv.w};
                            const float Cs[4] = {Cv.x, Cv.y, Cv.z, Cv.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int n = q * 4 + e;
                                const float a = fast_exp2(dt * A2[n]);
                                h[n] = __builtin_fmaf(a, h[n], Bs[e] * du);
                                acc[j] = __builtin_fmaf(h[n], Cs[e], acc[j]);
                            }
                        }
                    }
                }
                // each lane needs the full sum of the steps it owns only: a transposing reduction
                // (keep one half, hand the other half to the neighbour) instead of four full ones
                float own_sum[OWN];
                if constexpr (QS == 4) {
                    const bool odd = qslice & 1, hi = qslice & 2;
                    const float w01 = (odd ? acc[1] : acc[0]) + quad_xor<1>(odd ? acc[0] : acc[1]);
                    const float w23 = (odd ? acc[3] : acc[2]) + quad_xor<1>(odd ? acc[2] : acc[3]);
                    own_sum[0] = (hi ? w23 : w01) + quad_xor<2>(hi ? w01 : w23);
                    // eight lanes per channel: the other quad holds the other half of the states
                    if constexpr (NSPLIT == 8) own_sum[0] += __shfl_xor(own_sum[0], 4);
                } else if constexpr (QS == 2) {
#pragma unroll
                    for (int o = 0; o < OWN; ++o) {
                        own_sum[o] = (slice ? acc[o * 2 + 1] : acc[o * 2]) + quad_xor<1>(slice ? acc[o * 2] : acc[o * 2 + 1]);
                    }
                } else {
#pragma unroll
                    for (int o = 0; o < OWN; ++o) own_sum[o] = acc[o];
                }
#pragma unroll
                for (int o = 0; o < OWN; ++o) {
                    const int j = o * QS + qslice;
                    const int t = tq * 4 + j;
                    float y = __builtin_fmaf(D_f, own_u[o], own_sum[o]);
                    if (has_z) y *= s_gate[(z4 >> (8 * j)) & 0xffu];
                    if (t < nt && slice < QS) s_out[t][c_local] = __float2half(y);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int t = tq * 4 + j;
                    if (t >= nt) break;
                    const float u_val = s_u * i8_of(u4, j);
                    float dt = __builtin_fmaf(s_dt, i8_of(d4, j), db);
                    if (p.delta_softplus) dt = softplus20(dt);
                    dt_sum += dt;
                    const float du = dt * u_val;
                    const float4* bf = reinterpret_cast<const float4*>(&s_bc[t][0][slice * NPL]);
                    const float4* cf = reinterpret_cast<const float4*>(&s_bc[t][1][slice * NPL]);
                    float acc = 0.0f;
#pragma unroll
                    for (int q = 0; q < NPL / 4; ++q) {
                        const float4 Bv = bf[q];
                        const float4 Cv = cf[q];
                        const float Bs[4] = {Bv.x, Bv.y, Bv.z, Bv.w};
                        const float Cs[4] = {Cv.x, Cv.y, Cv.z, Cv.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int n = q * 4 + e;
                            const float a = fast_exp2(dt * A2[n]);
                            h[n] = __builtin_fmaf(a, h[n], Bs[e] * du);
                            acc = __builtin_fmaf(h[n], Cs[e], acc);
                        }
                    }
#pragma unroll
                    for (int m = 1; m < NSPLIT; m <<= 1) acc += __shfl_xor(acc, m);
                    float y = __builtin_fmaf(D_f, u_val, acc);
                    if (has_z) y *= s_gate[(z4 >> (8 * j)) & 0xffu];
                    if (slice == 0) s_out[t][c_local] = __float2half(y);
                }
            }
        }
        __syncthreads();   // s_out complete; everyone is done reading the staged tile

        // write the tile's output rows: (t, kCh channels) contiguous along channels
        {
            constexpr int kChunk = kCh >= 8 ? 8 : kCh;
            constexpr int kChunksPerRow = kCh / kChunk;
            __half* out_b = static_cast<__half*>(p.out) + b * p.out_batch_stride;
            for (int piece = tid; piece < nt * kChunksPerRow; piece += kThreads) {
                const int t = piece / kChunksPerRow, ch8 = (piece % kChunksPerRow) * kChunk;
                __half* dst = out_b + (t0 + t) * p.out_l_stride + (c0 + ch8) * p.out_d_stride;
                if (kChunk == 8 && vec_out && c0 + ch8 + 8 <= p.dim) {
                    *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(&s_out[t][ch8]);
                } else {
                    for (int e = 0; e < kChunk; ++e) {
                        if (c0 + ch8 + e < p.dim) dst[e * p.out_d_stride] = s_out[t][ch8 + e];
                    }
                }
            }
        }
        if (tile + 1 < n_tiles) stage();
        __syncthreads();
    }

    if (p.dt_sum_out) {
        // shared-out steps: the lanes of a quad hold the sums of different steps
        if constexpr (NSPLIT <= 4 || NSPLIT == 8) {
            if constexpr (QS >= 2) dt_sum += quad_xor<1>(dt_sum);
            if constexpr (QS == 4) dt_sum += quad_xor<2>(dt_sum);
        }
        if (c_ok && slice == 0) p.dt_sum_out[static_cast<int64_t>(b) * p.dim + c] = dt_sum;
    }
    if (c_ok) {
        const int64_t base = (static_cast<int64_t>(b) * p.dim + c) * p.dstate;
        const float s_state = p.last_state_i8 ? *p.scale_ssm_state : 1.0f;
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const int n = slice * NPL + j;
            if (n < p.dstate) {
                if (p.last_state_f32) p.last_state_f32[base + n] = h[j];
                if (p.last_state_i8) p.last_state_i8[base + n] = sat8_half_away(h[j] / s_state);
            }
        }
    }
}

template <int NPL, int NSPLIT, int T, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void sscan_fwd_kernel(QaSScanParams p, int vec_in, int vec_bc, int vec_out) {
    using Cfg = ScanCfg<NPL, NSPLIT, T, WAVES>;
    __shared__ ScanSmem<Cfg, T> sm;
    sscan_fwd_body<NPL, NSPLIT, T, WAVES>(p, vec_in, vec_bc, vec_out, blockIdx.x * Cfg::kCh, blockIdx.y, sm);
}

// ---------------------------------------------------------------------------------------------
// d_state <= 16, many channels: the same walk with everything that does not depend on the state index taken out
// of the time loop.  While a tile of T = 32 steps is staged, the thread that loaded a channel's bytes also
// evaluates the step size (bias, softplus) and step size x input for those steps and leaves them in LDS as
// fp32; all of these evaluations are independent, so their long dependent chains (two transcendentals each)
// overlap instead of standing at the head of every group of four steps, and the time loop reads them with two
// 16-byte loads that every lane of a channel shares - no cross-lane operands in the multiplications.
//   lanes of a channel: NSPLIT in {4, 8}; states per lane: NPL = 16 / NSPLIT; a lane stages T / NSPLIT steps
//   of its own channel per tile.
// ---------------------------------------------------------------------------------------------
template <int NPL, int NSPLIT, int WAVES>
struct PreCfg {
    static constexpr int T = 32;
    static constexpr int kThreads = 64 * WAVES;
    static constexpr int kCh = kThreads / NSPLIT;
    static constexpr int kNP = NPL * NSPLIT;               // 16
    static constexpr int kStage = T / NSPLIT;              // steps (= bytes per tensor) a lane stages per tile
    static constexpr int kPitch = T + 4;                   // floats per row of per-step values: rows 16-byte
                                                           // aligned, eight rows cover the 32 banks
    static constexpr int kUzPitch = T + 8;                 // 16-bit (u | z << 8) codes per row: rows 16-byte aligned
    static constexpr int kBcPitch = 2 * kNP + 4;           // floats per step of B | C
    static constexpr int kOutPitch = kCh + 8;              // halves; keeps rows 16-byte aligned
    static constexpr int kBcPieces = (2 * kNP * T / 4 + kThreads - 1) / kThreads;   // dwords of B/C per thread
};

template <class Cfg>
struct PreSmem {
    __attribute__((aligned(16))) float d[Cfg::kCh][Cfg::kPitch];     // step size
    __attribute__((aligned(16))) float du[Cfg::kCh][Cfg::kPitch];    // step size x input
    // input and gate codes of a step as they came from memory, u in the low byte and z in the high byte: the lane
    // that owns the step forms the skip term and looks the gate up itself (two fp32 rows per channel less in LDS)
    __attribute__((aligned(16))) uint16_t uz[Cfg::kCh][Cfg::kUzPitch];
    // the two tiles that all waves of the workgroup share, twice each: while tile t is scanned out of one copy the
    // next tile is staged into the other, so that one barrier per tile is enough (the per-step rows above belong to
    // the wave that staged them and need none)
    __attribute__((aligned(16))) float bc[2][Cfg::T][Cfg::kBcPitch];    // B (kNP) | C (kNP) of a step, scaled
    __attribute__((aligned(16))) __half out[2][Cfg::T][Cfg::kOutPitch];
    float gate_table[256];             // SiLU gate per z code (indexed by the raw byte)
};

// BYTES bytes starting at row[t]; bytes at or beyond t_end read as zero.
template <int BYTES>
__device__ __forceinline__ void load_bytes(uint32_t (&w)[BYTES / 4], const int8_t* row, int t, int t_end, bool vec) {
    if (vec && t + BYTES <= t_end) {
        if constexpr (BYTES == 8) {
            const uint2 v = *reinterpret_cast<const uint2*>(row + t);
            w[0] = v.x; w[1] = v.y;
        } else {
            w[0] = *reinterpret_cast<const uint32_t*>(row + t);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < BYTES / 4; ++i) w[i] = 0u;
    for (int i = 0; i < BYTES; ++i) {
        if (t + i < t_end) w[i >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(row[t + i])) << (8 * (i & 3));
    }
}

template <int NPL, int NSPLIT, int WAVES, bool HAS_Z>
__device__ __forceinline__ void sscan_fwd_pre_body(const QaSScanParams& p, int vec_in, int vec_bc, int vec_out, int c0, int b,
                                                   PreSmem<PreCfg<NPL, NSPLIT, WAVES>>& sm) {
    using Cfg = PreCfg<NPL, NSPLIT, WAVES>;
    constexpr int T = Cfg::T, kThreads = Cfg::kThreads, kCh = Cfg::kCh, kNP = Cfg::kNP, kStage = Cfg::kStage;
    constexpr int kBcPieces = Cfg::kBcPieces;
    static_assert(NSPLIT == 4 || NSPLIT == 8, "four or eight lanes per channel");
    static_assert(kNP == 16 && (NPL == 4 || NPL == 2), "sixteen states");

    const int tid = threadIdx.x;
    const int c_local = tid / NSPLIT;
    const int slice = tid % NSPLIT;
    const int qslice = slice & 3;
    const int c = c0 + c_local;
    const bool c_ok = c < p.dim;
    const int cc = c_ok ? c : p.dim - 1;                   // clamped channel for parameter loads
    const int g = c0 / (p.dim / p.n_groups);
    const int L = p.seqlen;
    const bool softplus = p.delta_softplus != 0;

    const float s_u = *p.scale_u, s_dt = *p.scale_delta, s_A = *p.scale_A, s_B = *p.scale_B, s_C = *p.scale_C;
    const float s_z = HAS_Z ? *p.scale_z : 0.0f;
    const float D_u = p.D ? (*p.scale_D * static_cast<float>(p.D[cc])) * s_u : 0.0f;       // skip weight per input code
    const float db = p.delta_bias ? *p.scale_delta_bias * static_cast<float>(p.delta_bias[cc]) : 0.0f;
    const bool want_dt_sum = p.dt_sum_out != nullptr;

    float A2[NPL], h[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int n = slice * NPL + j;
        h[j] = 0.0f;
        A2[j] = n < p.dstate
                    ? -expf(s_A * static_cast<float>(p.A_log[cc * p.A_d_stride + n * p.A_dstate_stride])) * kLog2e
                    : 0.0f;
    }
    if (p.carry_state) {                 // segments of one sequence side by side, see sscan_fwd_body
        const int seg = p.carry_first + b;
        for (int sp = 0; sp < seg; ++sp) {
            const float sd = p.carry_dt_sum[static_cast<int64_t>(sp) * p.dim + cc];
#pragma unroll
            for (int j = 0; j < NPL; ++j) {
                const int n = min(slice * NPL + j, p.dstate - 1);
                h[j] = __builtin_fmaf(fast_exp2(sd * A2[j]), h[j],
                                      p.carry_state[(static_cast<int64_t>(sp) * p.dim + cc) * p.dstate + n]);
            }
        }
    }
    float dt_sum = 0.0f;                 // of the steps this lane stages

    const int8_t* u_row = p.u + b * p.u_batch_stride + static_cast<int64_t>(cc) * p.u_d_stride;
    const int8_t* d_row = p.delta + b * p.delta_batch_stride + static_cast<int64_t>(cc) * p.delta_d_stride;
    const int8_t* z_row = HAS_Z ? p.z + b * p.z_batch_stride + static_cast<int64_t>(cc) * p.z_d_stride : nullptr;
    uint32_t r_u[kStage / 4], r_d[kStage / 4], r_z[kStage / 4];
    uint32_t r_bc[kBcPieces];

    // B / C dword `piece` of a tile: the state index varies fastest over the lanes, so that the four scattered
    // LDS writes of stage() spread over the banks
    auto bc_piece = [&](int piece, int& which, int& n, int& col) {
        which = piece / (kNP * T / 4);
        n = piece % kNP;
        col = (piece / kNP) % (T / 4);
    };
    // this thread's dwords of a tile's B / C codes: the row they come from (states beyond d_state read the last state's
    // row and are scaled by zero) and the scale they are staged with
    const int8_t* bc_row[kBcPieces];
    float bc_factor[kBcPieces];
#pragma unroll
    for (int i = 0; i < kBcPieces; ++i) {
        int which, n, col;
        bc_piece(tid + i * kThreads, which, n, col);
        const int nn = min(n, p.dstate - 1);
        const int8_t* rowB = p.B + b * p.B_batch_stride + g * p.B_group_stride + nn * p.B_dstate_stride;
        const int8_t* rowC = p.C + b * p.C_batch_stride + g * p.C_group_stride + nn * p.C_dstate_stride;
        bc_row[i] = which ? rowC : rowB;
        bc_factor[i] = n < p.dstate ? (which ? s_C : s_B * s_u) : 0.0f;
    }

    // A tile that lies inside the sequence, of rows that allow vector loads, is requested without a branch per lane: the
    // requests then stay in flight until stage() needs them.  (With the byte-wise alternative in the same control
    // flow the compiler waits for every request where the two paths join.)
    auto issue_loads = [&](int t0) {
        const int t = t0 + slice * kStage;
        const bool whole = t0 + T <= L;
        // rows past the last channel read the last channel's bytes; nothing of theirs is stored
        if (vec_in && whole) {
            if constexpr (kStage == 8) {
                const uint2 vu = *reinterpret_cast<const uint2*>(u_row + t), vd = *reinterpret_cast<const uint2*>(d_row + t);
                r_u[0] = vu.x; r_u[1] = vu.y; r_d[0] = vd.x; r_d[1] = vd.y;
                if constexpr (HAS_Z) {
                    const uint2 vz = *reinterpret_cast<const uint2*>(z_row + t);
                    r_z[0] = vz.x; r_z[1] = vz.y;
                }
            } else {
                r_u[0] = *reinterpret_cast<const uint32_t*>(u_row + t);
                r_d[0] = *reinterpret_cast<const uint32_t*>(d_row + t);
                if constexpr (HAS_Z) r_z[0] = *reinterpret_cast<const uint32_t*>(z_row + t);
            }
        } else {
            load_bytes<kStage>(r_u, u_row, t, L, false);
            load_bytes<kStage>(r_d, d_row, t, L, false);
            if constexpr (HAS_Z) load_bytes<kStage>(r_z, z_row, t, L, false);
        }
        if (vec_bc && whole) {
#pragma unroll
            for (int i = 0; i < kBcPieces; ++i) {
                int which, n, col;
                bc_piece(tid + i * kThreads, which, n, col);
                r_bc[i] = *reinterpret_cast<const uint32_t*>(bc_row[i] + t0 + col * 4);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kBcPieces; ++i) {
                int which, n, col;
                bc_piece(tid + i * kThreads, which, n, col);
                uint32_t v[1];
                load_bytes<4>(v, bc_row[i], t0 + col * 4, L, false);
                r_bc[i] = v[0];
            }
        }
    };

    // Writes the staged tile.  Per step of this lane's share of its channel: step size (bias, softplus), step
    // size x input, skip term and gate - everything the time loop needs that does not depend on the state.
    auto stage = [&](int t0, int into) {
        float dv[kStage], duv[kStage];
#pragma unroll
        for (int e = 0; e < kStage; ++e) dv[e] = __builtin_fmaf(s_dt, i8_of(r_d[e >> 2], e & 3), db);
        if (softplus) {                  // one uniform branch per tile: the evaluations below overlap
#pragma unroll
            for (int e = 0; e < kStage; ++e) dv[e] = softplus20_flat(dv[e]);
        }
        if (t0 + T > L) {
            // ragged last tile: steps past the end of the sequence must leave the state alone (a = 1, b = 0)
#pragma unroll
            for (int e = 0; e < kStage; ++e) dv[e] = t0 + slice * kStage + e < L ? dv[e] : 0.0f;
        }
        if (want_dt_sum) {
#pragma unroll
            for (int e = 0; e < kStage; ++e) dt_sum += dv[e];
        }
#pragma unroll
        for (int e = 0; e < kStage; ++e) {
            // the input scale rides with B and D: (s_B q_B) (dt (s_u q_u)) = ((s_B s_u) q_B) (dt q_u)
            duv[e] = dv[e] * i8_of(r_u[e >> 2], e & 3);
        }
#pragma unroll
        for (int q = 0; q < kStage / 4; ++q) {
            const int t = slice * kStage + q * 4;
            *reinterpret_cast<float4*>(&sm.d[c_local][t]) = make_float4(dv[q * 4], dv[q * 4 + 1], dv[q * 4 + 2], dv[q * 4 + 3]);
            *reinterpret_cast<float4*>(&sm.du[c_local][t]) = make_float4(duv[q * 4], duv[q * 4 + 1], duv[q * 4 + 2], duv[q * 4 + 3]);
            // four steps' codes, interleaved bytewise: (u0 z0 u1 z1) (u2 z2 u3 z3)
            const uint32_t zw = HAS_Z ? r_z[q] : 0u;
            uint2 codes;
            codes.x = __builtin_amdgcn_perm(zw, r_u[q], 0x05010400u);
            codes.y = __builtin_amdgcn_perm(zw, r_u[q], 0x07030602u);
            *reinterpret_cast<uint2*>(&sm.uz[c_local][t]) = codes;
        }
#pragma unroll
        for (int i = 0; i < kBcPieces; ++i) {
            int which, n, col;
            bc_piece(tid + i * kThreads, which, n, col);
#pragma unroll
            for (int e = 0; e < 4; ++e) sm.bc[into][col * 4 + e][which * kNP + n] = bc_factor[i] * i8_of(r_bc[i], e);
        }
    };

    // operands of one group of four steps
    struct Group {
        float d[4], du[4], B[4][NPL], C[4][NPL];
        uint32_t code;                  // of the step this lane owns: u in byte 0, z in byte 1
    };
    auto fetch = [&](Group& o, int tq, int from) {
        const float4 d4 = *reinterpret_cast<const float4*>(&sm.d[c_local][tq * 4]);
        const float4 du4 = *reinterpret_cast<const float4*>(&sm.du[c_local][tq * 4]);
        o.d[0] = d4.x; o.d[1] = d4.y; o.d[2] = d4.z; o.d[3] = d4.w;
        o.du[0] = du4.x; o.du[1] = du4.y; o.du[2] = du4.z; o.du[3] = du4.w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float* row = sm.bc[from][tq * 4 + j];
            if constexpr (NPL == 2) {
                const float2 Bv = *reinterpret_cast<const float2*>(row + slice * NPL);
                const float2 Cv = *reinterpret_cast<const float2*>(row + kNP + slice * NPL);
                o.B[j][0] = Bv.x; o.B[j][1] = Bv.y; o.C[j][0] = Cv.x; o.C[j][1] = Cv.y;
            } else {
                const float4 Bv = *reinterpret_cast<const float4*>(row + slice * NPL);
                const float4 Cv = *reinterpret_cast<const float4*>(row + kNP + slice * NPL);
                o.B[j][0] = Bv.x; o.B[j][1] = Bv.y; o.B[j][2] = Bv.z; o.B[j][3] = Bv.w;
                o.C[j][0] = Cv.x; o.C[j][1] = Cv.y; o.C[j][2] = Cv.z; o.C[j][3] = Cv.w;
            }
        }
        o.code = sm.uz[c_local][tq * 4 + qslice];
    };

    const int n_tiles = (L + T - 1) / T;
    issue_loads(0);
    if constexpr (HAS_Z) {
        for (int i = tid; i < 256; i += kThreads) sm.gate_table[i] = silu_gate(s_z * static_cast<float>(static_cast<int8_t>(i)));
        __syncthreads();
    }
    stage(0, 0);
    __syncthreads();
    int buf = 0;                          // copy of the shared tiles that holds the tile being scanned

    for (int tile = 0; tile < n_tiles; ++tile) {
        const int t0 = tile * T;
        const int nt = min(T, L - t0);
        if (tile + 1 < n_tiles) issue_loads(t0 + T);

        // All T / 4 groups of four steps, also in a ragged last tile: steps past the end have step size 0 and leave
        // the state alone, and their output rows are never stored.  No branch in the body and constant LDS
        // offsets; the operands of a group are fetched while the group before is being computed.
        Group grp[2];
        fetch(grp[0], 0, buf);
#pragma unroll
        for (int tq = 0; tq < T / 4; ++tq) {
            Group& o = grp[tq & 1];
            if (tq + 1 < T / 4) fetch(grp[(tq + 1) & 1], tq + 1, buf);
            // keep the reads of the next group ahead of this group's arithmetic (the scheduler would sink them
            // to their first use, and a wave would then wait for LDS once per group)
            __builtin_amdgcn_sched_barrier(0);
            // the gate of the step this lane owns: looked up now, used when the group's sums are complete
            float gate = 1.0f;
            if constexpr (HAS_Z) gate = sm.gate_table[(o.code >> 8) & 0xffu];
            float acc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] = 0.0f;
#pragma unroll
                for (int n = 0; n < NPL; ++n) {
                    const float a = fast_exp2(o.d[j] * A2[n]);
                    h[n] = __builtin_fmaf(a, h[n], o.B[j][n] * o.du[j]);
                    acc[j] = __builtin_fmaf(h[n], o.C[j][n], acc[j]);
                }
            }
            // each lane of a quad completes the step it owns: a transposing reduction (keep one half, hand the
            // other half to the neighbour) instead of four full ones
            const bool odd = qslice & 1, hi = qslice & 2;
            const float w01 = (odd ? acc[1] : acc[0]) + quad_xor<1>(odd ? acc[0] : acc[1]);
            const float w23 = (odd ? acc[3] : acc[2]) + quad_xor<1>(odd ? acc[2] : acc[3]);
            float own_sum = (hi ? w23 : w01) + quad_xor<2>(hi ? w01 : w23);
            // eight lanes per channel: the other quad holds the other half of the states (both quads then hold
            // the same sums and store the same values)
            if constexpr (NSPLIT == 8) own_sum += __shfl_xor(own_sum, 4);
            float y = own_sum + D_u * code_byte_to_float(o.code, 0);
            if constexpr (HAS_Z) y *= gate;
            sm.out[buf][tq * 4 + qslice][c_local] = __float2half(y);
        }
        // the next tile goes into the other copy (every wave left it at the barrier of the tile before)
        if (tile + 1 < n_tiles) stage(t0 + T, buf ^ 1);
        __syncthreads();   // this tile's outputs and the next tile's B / C are complete

        // write the tile's output rows: (t, kCh channels) contiguous along channels
        {
            constexpr int kChunksPerRow = kCh / 8;
            __half* out_b = static_cast<__half*>(p.out) + b * p.out_batch_stride;
            for (int piece = tid; piece < nt * kChunksPerRow; piece += kThreads) {
                const int t = piece / kChunksPerRow, ch8 = (piece % kChunksPerRow) * 8;
                __half* dst = out_b + (t0 + t) * p.out_l_stride + (c0 + ch8) * p.out_d_stride;
                if (vec_out && c0 + ch8 + 8 <= p.dim) {
                    *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(&sm.out[buf][t][ch8]);
                } else {
                    for (int e = 0; e < 8; ++e) {
                        if (c0 + ch8 + e < p.dim) dst[e * p.out_d_stride] = sm.out[buf][t][ch8 + e];
                    }
                }
            }
        }
        buf ^= 1;
    }

    if (p.dt_sum_out) {
        // the lanes of a channel staged different steps
        dt_sum += quad_xor<1>(dt_sum);
        dt_sum += quad_xor<2>(dt_sum);
        if constexpr (NSPLIT == 8) dt_sum += __shfl_xor(dt_sum, 4);
        if (c_ok && slice == 0) p.dt_sum_out[static_cast<int64_t>(b) * p.dim + c] = dt_sum;
    }
    if (c_ok) {
        const int64_t base = (static_cast<int64_t>(b) * p.dim + c) * p.dstate;
        const float s_state = p.last_state_i8 ? *p.scale_ssm_state : 1.0f;
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const int n = slice * NPL + j;
            if (n < p.dstate) {
                if (p.last_state_f32) p.last_state_f32[base + n] = h[j];
                if (p.last_state_i8) p.last_state_i8[base + n] = sat8_half_away(h[j] / s_state);
            }
        }
    }
}

template <int NPL, int NSPLIT, int WAVES, bool HAS_Z>
__global__ __launch_bounds__(64 * WAVES) void sscan_fwd_pre_kernel(QaSScanParams p, int vec_in, int vec_bc, int vec_out) {
    using Cfg = PreCfg<NPL, NSPLIT, WAVES>;
    __shared__ PreSmem<Cfg> sm;
    sscan_fwd_pre_body<NPL, NSPLIT, WAVES, HAS_Z>(p, vec_in, vec_bc, vec_out, blockIdx.x * Cfg::kCh, blockIdx.y, sm);
}

// Two kinds of workgroup in one launch, for d_state 16: the first `blocks_a` workgroups of a batch entry take
// 64 channels each with four lanes per channel, the others 32 channels each with eight lanes per channel (half
// the states per lane, a little more than half the time).  The kernel is bound by vector-ALU issue and a wave's
// time does not depend on how many of its lanes are busy, so what counts is the number of waves per SIMD: when
// the four-lane mapping alone would leave half of the SIMDs with one wave more than the others, the tail of the
// channels goes to the short kind and every SIMD gets the same mix.
template <bool HAS_Z>
__global__ __launch_bounds__(256) void sscan_fwd_mixed_kernel(QaSScanParams p, int vec_in, int vec_bc, int vec_out, int blocks_a) {
    using CfgA = PreCfg<4, 4, 4>;
    using CfgB = PreCfg<2, 8, 4>;
    __shared__ union Smem {
        PreSmem<CfgA> a;
        PreSmem<CfgB> b;
        __device__ Smem() {}
    } sm;
    const int bx = blockIdx.x;
    if (bx < blocks_a) {
        sscan_fwd_pre_body<4, 4, 4, HAS_Z>(p, vec_in, vec_bc, vec_out, bx * CfgA::kCh, blockIdx.y, sm.a);
    } else {
        sscan_fwd_pre_body<2, 8, 4, HAS_Z>(p, vec_in, vec_bc, vec_out, blocks_a * CfgA::kCh + (bx - blocks_a) * CfgB::kCh, blockIdx.y, sm.b);
    }
}

template <int NPL, int NSPLIT, int T, int WAVES>
int launch_fwd(const QaSScanParams& p, hipStream_t stream, int vec_in, int vec_bc, int vec_out) {
    using Cfg = ScanCfg<NPL, NSPLIT, T, WAVES>;
    if (p.n_groups > 1 && (p.dim / p.n_groups) % Cfg::kCh != 0) return QA_ERR_UNSUPPORTED;
    dim3 grid((p.dim + Cfg::kCh - 1) / Cfg::kCh, p.batch);
    hipLaunchKernelGGL((sscan_fwd_kernel<NPL, NSPLIT, T, WAVES>), grid, dim3(Cfg::kThreads), 0, stream, p, vec_in,
                       vec_bc, vec_out);
    return check_launch();
}

template <int NPL, int NSPLIT, int WAVES>
int launch_fwd_pre(const QaSScanParams& p, hipStream_t stream, int vec_in, int vec_bc, int vec_out) {
    using Cfg = PreCfg<NPL, NSPLIT, WAVES>;
    if (p.n_groups > 1 && (p.dim / p.n_groups) % Cfg::kCh != 0) return QA_ERR_UNSUPPORTED;
    dim3 grid((p.dim + Cfg::kCh - 1) / Cfg::kCh, p.batch);
    if (p.z) {
        hipLaunchKernelGGL((sscan_fwd_pre_kernel<NPL, NSPLIT, WAVES, true>), grid, dim3(Cfg::kThreads), 0, stream, p, vec_in,
                           vec_bc, vec_out);
    } else {
        hipLaunchKernelGGL((sscan_fwd_pre_kernel<NPL, NSPLIT, WAVES, false>), grid, dim3(Cfg::kThreads), 0, stream, p, vec_in,
                           vec_bc, vec_out);
    }
    return check_launch();
}

// Channels [0, 64 * blocks_a) with four lanes per channel, the rest with eight.
int launch_fwd_mixed(const QaSScanParams& p, hipStream_t stream, int vec_in, int vec_bc, int vec_out, int blocks_a) {
    const int rest = p.dim - 64 * blocks_a;
    dim3 grid(blocks_a + (rest + 31) / 32, p.batch);
    if (p.z) hipLaunchKernelGGL(sscan_fwd_mixed_kernel<true>, grid, dim3(256), 0, stream, p, vec_in, vec_bc, vec_out, blocks_a);
    else hipLaunchKernelGGL(sscan_fwd_mixed_kernel<false>, grid, dim3(256), 0, stream, p, vec_in, vec_bc, vec_out, blocks_a);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// Single-token update.  LPR lanes share one (batch, head, channel) row, up to sixteen states per lane
// in pieces of four, so consecutive lanes touch consecutive 16-byte (fp32 state) or 4-byte (int8
// state) pieces.
// Reference: quamba/triton/selective_state_update.py:83-126 and :303-362.
// ---------------------------------------------------------------------------------------------
// VEC: the state axis has unit stride in state, A_log, B and C and every row piece of four states is
// naturally aligned, so a lane moves its four states with one load and one store per operand.
// A wave's life here is a chain of memory round trips, not arithmetic, so optional operands are read
// through a stand-in address instead of behind a branch: every load of the row is in flight at once.
// CONV: the row's input code is not read from p.x but produced here by the causal conv's single-step update on
// channel d of batch entry b (quant_causal_conv1d_update_kernel.cuh:34-75: shift the conv state, dot product with
// the taps, bias, SiLU, requantise - the arithmetic of conv_update_kernel, same bits), for one lane per row.
// FAST: the shape of the Mamba1 decode step is known at compile time (one head, one B/C group, sixteen states whose
// A_log codes are one aligned 16-byte row, per-tensor scales, no fp16 bias, four taps), so the lane's work is one
// run of loads, arithmetic and stores without loops or branches on the parameter block.
// CONV_STATE: with CONV and FAST, the codes per row of the conv state (4: a word per row; 3: rows back to back).
template <int LPR, bool VEC, bool FP32, bool CONV, bool FAST = false, int CONV_STATE = 4>
__device__ __forceinline__ void ssm_update_body(const QaSsmUpdateParams& p, const QaConvParams* cp) {
    static_assert(!CONV || LPR == 1, "the conv step needs one lane per row");
    static_assert(!FAST || (LPR == 1 && VEC), "the fixed shape has one lane per row and whole pieces");
    const int dstate = FAST ? 16 : p.dstate;
    // grid: x over the channels of one head, y = head, z = batch (no integer division on the way in)
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int sub = gid % LPR;
    const bool row_ok = gid / LPR < p.dim;
    const int d = row_ok ? gid / LPR : p.dim - 1;
    const int hd = FAST ? 0 : blockIdx.y;
    const int64_t b = blockIdx.z;
    const int heads_per_group = FAST ? 1 : p.nheads / p.ngroups;
    const int g = FAST ? 0 : hd / heads_per_group;

    const bool grouped = !FAST && p.nhead_groups > 0;
    int sidx = 0;                       // grouped: index of this row's (g, head group, dim group)
    if (grouped) {
        int hg = 0, dg = 0;
        const int hrel = hd % heads_per_group;
        for (int j = 0; j < p.nhead_groups; ++j) hg += hrel >= p.x_head_group_range[g * p.nhead_groups + j] ? 1 : 0;
        hg = min(hg, p.nhead_groups - 1);
        const int32_t* dr = p.x_dim_group_range + (g * p.nhead_groups + hg) * p.ndim_groups;
        for (int j = 0; j < p.ndim_groups; ++j) dg += d >= dr[j] ? 1 : 0;
        dg = min(dg, p.ndim_groups - 1);
        sidx = (g * p.nhead_groups + hg) * p.ndim_groups + dg;
    }
    const float* standin = p.x_scale;   // always readable, four bytes
    const float* state_scale_row = (grouped && !FP32) ? p.state_scale + static_cast<int64_t>(sidx) * dstate : nullptr;
    const bool bias_i8 = p.dt_bias && !p.dt_bias_is_fp16;
    const bool bias_f16 = !FAST && p.dt_bias && p.dt_bias_is_fp16;
    const int64_t bias_i = hd * p.dt_bias_head_stride + d * p.dt_bias_dim_stride;
    const int8_t* x_a = p.x + b * p.x_batch_stride + hd * p.x_head_stride + d * p.x_dim_stride;
    const int8_t* dt_a = p.dt + b * p.dt_batch_stride + hd * p.dt_head_stride + d * p.dt_dim_stride;
    const int8_t* standin8 = CONV ? dt_a : x_a;             // always readable, one byte (p.x is not used with CONV)
    const int8_t* z_a = p.z ? p.z + b * p.z_batch_stride + hd * p.z_head_stride + d * p.z_dim_stride : standin8;
    const int8_t* D_a = p.D ? p.D + hd * p.D_head_stride + d * p.D_dim_stride : standin8;
    const int8_t* b8_a = bias_i8 ? static_cast<const int8_t*>(p.dt_bias) + bias_i : standin8;
    const __half* b16_a = bias_f16 ? static_cast<const __half*>(p.dt_bias) + bias_i : reinterpret_cast<const __half*>(standin);

    const float x_scale = p.x_scale[sidx];
    const float B_scale = p.B_scale[grouped ? g : 0];
    const float C_scale = p.C_scale[grouped ? g : 0];
    const float dt_scale = *p.dt_scale;
    const float A_scale = *p.A_log_scale;
    const float s_state = *((!grouped && !FP32) ? p.state_scale : standin);
    const float D_scale = *(p.D ? p.D_scale : standin);
    const float z_scale = *(p.z ? p.z_scale : standin);
    const float bias_scale = *(bias_i8 ? p.dt_bias_scale : standin);
    const float requant_k = grouped ? 1e6f : 1e2f;

    const int64_t st_base = b * p.state_batch_stride + hd * p.state_head_stride + d * p.state_dim_stride;
    const int8_t* Bp = p.B + b * p.B_batch_stride + g * p.B_group_stride;
    const int8_t* Cp = p.C + b * p.C_batch_stride + g * p.C_group_stride;
    const int8_t* Ap = p.A_log + hd * p.A_head_stride + d * p.A_dim_stride;
    // A lane owns up to kPieces pieces of four states: piece k of lane `sub` starts at state
    // (sub + k * LPR) * 4.  All loads first, then the arithmetic, then the stores.
    constexpr int kPieces = 4;
    float hv[kPieces][4], sc[kPieces][4];
    __attribute__((aligned(16))) int8_t a8[kPieces][4];
    uint32_t a_word[kPieces];               // FAST: the row of A_log as four words
    // STAGED (FAST with an fp32 state whose rows lie back to back, whole waves of rows): a lane that reads its own
    // 64-byte row touches one sixteen-byte piece of 64 different rows per load, and the memory system moves such
    // a wave at about half the rate of one that reads 1 KB in a run.  So the wave moves its 64 rows (4 KB, one run
    // in memory) with four loads of 1 KB and turns them by way of LDS: piece q of row r sits in slot
    // 4 r + (q ^ (r / 4 % 4)), which keeps both the run-order and the row-order accesses off each other's banks.
    constexpr bool STAGED = FAST && FP32;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float staged[kPieces][4];
    float4* wave_state = nullptr;
    const float4* wave_state_in = nullptr;  // a wave past the last row reads the batch entry's first rows, and stores nothing
    if constexpr (STAGED) {
        float4* entry = reinterpret_cast<float4*>(static_cast<float*>(p.state) + b * p.state_batch_stride);
        wave_state = entry + static_cast<int64_t>(gid - lane) * 4;
        wave_state_in = row_ok ? wave_state : entry;
    }
    __attribute__((aligned(4))) int8_t b8v[kPieces][4], c8[kPieces][4], s8[kPieces][4];
    // one lane per row with sixteen states in a row of A_log: the lane's sixteen codes come as one 16-byte piece
    const bool a_row16 = FAST || (VEC && LPR == 1 && dstate == 16 && p.A_dstate_stride == 1 && (reinterpret_cast<uintptr_t>(Ap) & 15u) == 0);
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
        const int n0 = (sub + k * LPR) * 4;
        if (n0 >= dstate) continue;
        if constexpr (VEC) {
            // dstate is a multiple of four here, so the piece is whole.  A_log alone may be a broadcast view
            // (one value per head, stride 0 along the states, as Mamba2 passes it): it is read through its
            // stride, the state and B, C with one load per piece
            if (a_row16) {
                if (k == 0) {
                    const uint4 row = *reinterpret_cast<const uint4*>(Ap);
                    if constexpr (FAST) { a_word[0] = row.x; a_word[1] = row.y; a_word[2] = row.z; a_word[3] = row.w; }
                    else *reinterpret_cast<uint4*>(&a8[0][0]) = row;
                }
            } else if (p.A_dstate_stride == 1 && (reinterpret_cast<uintptr_t>(Ap + n0) & 3u) == 0) {
                *reinterpret_cast<int32_t*>(a8[k]) = *reinterpret_cast<const int32_t*>(Ap + n0);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) a8[k][e] = Ap[(n0 + e) * p.A_dstate_stride];
            }
            if constexpr (FAST) {
                // B and C come as floats through LDS (below)
            } else if constexpr (LPR == 1) {
                // every lane of the wave reads the same B and C words (one batch entry per workgroup): scalar loads
                typedef const __attribute__((address_space(4))) int32_t* const_words;
                *reinterpret_cast<int32_t*>(b8v[k]) = reinterpret_cast<const_words>(reinterpret_cast<uintptr_t>(Bp))[n0 / 4];
                *reinterpret_cast<int32_t*>(c8[k]) = reinterpret_cast<const_words>(reinterpret_cast<uintptr_t>(Cp))[n0 / 4];
            } else {
                *reinterpret_cast<int32_t*>(b8v[k]) = *reinterpret_cast<const int32_t*>(Bp + n0);
                *reinterpret_cast<int32_t*>(c8[k]) = *reinterpret_cast<const int32_t*>(Cp + n0);
            }
            if constexpr (STAGED) {
                // piece k of the wave's 4 KB of state, in memory order: lane l brings 16 bytes at (64 k + l) * 16
                const float4 v = wave_state_in[k * 64 + lane];
                staged[k][0] = v.x; staged[k][1] = v.y; staged[k][2] = v.z; staged[k][3] = v.w;
            } else if constexpr (FP32) {
                const float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(p.state) + st_base + n0);
                hv[k][0] = v.x; hv[k][1] = v.y; hv[k][2] = v.z; hv[k][3] = v.w;
            } else {
                *reinterpret_cast<int32_t*>(s8[k]) = *reinterpret_cast<const int32_t*>(static_cast<const int8_t*>(p.state) + st_base + n0);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) sc[k][e] = state_scale_row ? state_scale_row[n0 + e] : s_state;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = min(n0 + e, dstate - 1);
                const int64_t si = st_base + n * p.state_dstate_stride;
                sc[k][e] = state_scale_row ? state_scale_row[n] : s_state;
                if constexpr (FP32) hv[k][e] = static_cast<const float*>(p.state)[si];
                else s8[k][e] = static_cast<const int8_t*>(p.state)[si];
                a8[k][e] = Ap[n * p.A_dstate_stride];
                b8v[k][e] = Bp[n * p.B_dstate_stride];
                c8[k][e] = Cp[n * p.C_dstate_stride];
            }
        }
    }
    // FAST: B_scale * B[n] and C_scale * C[n] are the same in every lane of the workgroup (one batch entry), and
    // converting and scaling them in every lane is an eighth of the lane's arithmetic.  Lanes 0-31 of each wave form
    // one value each (same expression, same bits) and the wave reads all 32 back from LDS as broadcasts.
    int8_t bc_code = 0;
    if constexpr (FAST) bc_code = ((lane & 16) ? Cp : Bp)[lane & 15];      // every lane loads: no branch, no wait here
    // The row's other operands come after the state's pieces are on their way: with CONV the conv step's own loads,
    // arithmetic and stores then run under the state's round trip instead of before it.
    const float dtq = static_cast<float>(*dt_a);
    const float zq = static_cast<float>(*z_a), Dq = static_cast<float>(*D_a);
    const float b8 = static_cast<float>(*b8_a), b16 = __half2float(*b16_a);
    float xq;
    if constexpr (CONV) {
        xq = static_cast<float>(conv_step_row<FAST ? CONV_STATE : 0>(*cp, static_cast<int>(b), d, row_ok));
    } else {
        xq = static_cast<float>(*x_a);
    }
    float bvf[kPieces][4], cvf[kPieces][4];
    if constexpr (FAST) {
        // a wave writes and reads only its own part of LDS, and a wave's LDS operations complete in order: the
        // fences keep the compiler from reordering them, no barrier is needed
        __shared__ __attribute__((aligned(16))) float bc_f32[4][32];
        if (lane < 32) bc_f32[wv][lane] = (lane < 16 ? B_scale : C_scale) * static_cast<float>(bc_code);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int k = 0; k < kPieces; ++k) {
            const float4 bq = *reinterpret_cast<const float4*>(&bc_f32[wv][4 * k]);
            const float4 cq = *reinterpret_cast<const float4*>(&bc_f32[wv][16 + 4 * k]);
            bvf[k][0] = bq.x; bvf[k][1] = bq.y; bvf[k][2] = bq.z; bvf[k][3] = bq.w;
            cvf[k][0] = cq.x; cvf[k][1] = cq.y; cvf[k][2] = cq.z; cvf[k][3] = cq.w;
        }
    }
    __shared__ __attribute__((aligned(16))) float4 turn[STAGED ? 4 : 1][STAGED ? 256 : 1];
    if constexpr (STAGED) {
#pragma unroll
        for (int k = 0; k < kPieces; ++k) {
            const int r = k * 16 + lane / 4, q = lane % 4;
            turn[wv][4 * r + (q ^ (r / 4 % 4))] = make_float4(staged[k][0], staged[k][1], staged[k][2], staged[k][3]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int k = 0; k < kPieces; ++k) {
            const float4 v = turn[wv][4 * lane + (k ^ (lane / 4 % 4))];
            hv[k][0] = v.x; hv[k][1] = v.y; hv[k][2] = v.z; hv[k][3] = v.w;
        }
    }
    const float xv = x_scale * xq;
    float dt = dt_scale * dtq;
    dt += bias_i8 ? bias_scale * b8 : (bias_f16 ? b16 : 0.0f);
    if (p.dt_softplus) dt = softplus20_flat(dt);
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
        const int n0 = (sub + k * LPR) * 4;
        if (n0 >= dstate) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (!FP32) hv[k][e] = sc[k][e] * static_cast<float>(s8[k][e]);
            const float a_code = FAST ? code_byte_to_float(a_word[k], e) : static_cast<float>(a8[k][e]);
            const float A = -__expf(A_scale * a_code);
            const float dA = __expf(A * dt);
            const float Bv = FAST ? bvf[k][e] : B_scale * static_cast<float>(b8v[k][e]);
            const float Cv = FAST ? cvf[k][e] : C_scale * static_cast<float>(c8[k][e]);
            hv[k][e] = hv[k][e] * dA + (Bv * dt) * xv;
            if (VEC || n0 + e < dstate) acc += hv[k][e] * Cv;
        }
        if (!row_ok) continue;
        if constexpr (STAGED) {
            turn[wv][4 * lane + (k ^ (lane / 4 % 4))] = make_float4(hv[k][0], hv[k][1], hv[k][2], hv[k][3]);
        } else if constexpr (VEC) {
            if constexpr (FP32) {
                *reinterpret_cast<float4*>(static_cast<float*>(p.state) + st_base + n0) =
                    make_float4(hv[k][0], hv[k][1], hv[k][2], hv[k][3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) s8[k][e] = sat8_rne((hv[k][e] * requant_k) / (sc[k][e] * requant_k));
                *reinterpret_cast<int32_t*>(static_cast<int8_t*>(p.state) + st_base + n0) = *reinterpret_cast<const int32_t*>(s8[k]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n0 + e;
                if (n >= dstate) break;
                const int64_t si = st_base + n * p.state_dstate_stride;
                if constexpr (FP32) static_cast<float*>(p.state)[si] = hv[k][e];
                else static_cast<int8_t*>(p.state)[si] = sat8_rne((hv[k][e] * requant_k) / (sc[k][e] * requant_k));
            }
        }
    }
    if constexpr (STAGED) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (row_ok) {
#pragma unroll
            for (int k = 0; k < kPieces; ++k) {
                const int r = k * 16 + lane / 4, q = lane % 4;
                wave_state[k * 64 + lane] = turn[wv][4 * r + (q ^ (r / 4 % 4))];
            }
        }
    }
#pragma unroll
    for (int m = 1; m < LPR; m <<= 1) acc += __shfl_xor(acc, m);
    if (row_ok && sub == 0) {
        if (p.D) acc += xv * (D_scale * Dq);
        if (p.z) {
            const float zv = z_scale * zq;
            acc *= zv * (1.0f / (1.0f + expf(-zv)));
        }
        static_cast<__half*>(p.out)[b * p.out_batch_stride + hd * p.out_head_stride + d * p.out_dim_stride] =
            __float2half(acc);
    }
}

template <int LPR, bool VEC, bool FP32, bool FAST = false>
__global__ __launch_bounds__(256) void ssm_update_kernel(QaSsmUpdateParams p) {
    ssm_update_body<LPR, VEC, FP32, false, FAST>(p, nullptr);
}

// conv step + state update of one token in one launch (d_state <= 16, one head)
template <bool VEC, bool FP32, bool FAST, int CONV_STATE = 4>
__global__ __launch_bounds__(256) void decode_step_kernel(QaSsmUpdateParams p, QaConvParams cp) {
    ssm_update_body<1, VEC, FP32, true, FAST, CONV_STATE>(p, &cp);
}

template <int LPR>
int launch_update(const QaSsmUpdateParams& p, hipStream_t stream, const QaConvParams* conv = nullptr) {
    const int64_t blocks = (static_cast<int64_t>(p.dim) * LPR + 255) / 256;
    if (blocks > 0x7fffffffLL / 256 || p.nheads > 65535 || p.batch > 65535) return QA_ERR_SHAPE;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(p.nheads), static_cast<unsigned>(p.batch));
    const int64_t st_align = p.state_is_fp32 ? 16 : 4;      // bytes of one lane's four states
    const int64_t st_el = p.state_is_fp32 ? 4 : 1;
    auto mult = [](int64_t v, int64_t m) { return v % m == 0; };
    const bool vec = p.dstate % 4 == 0 && p.state_dstate_stride == 1 &&
                     p.B_dstate_stride == 1 && p.C_dstate_stride == 1 &&
                     reinterpret_cast<uintptr_t>(p.state) % st_align == 0 &&
                     mult(p.state_batch_stride * st_el, st_align) && mult(p.state_head_stride * st_el, st_align) &&
                     mult(p.state_dim_stride * st_el, st_align) &&
                     aligned4(p.B) && mult(p.B_batch_stride, 4) && mult(p.B_group_stride, 4) &&
                     aligned4(p.C) && mult(p.C_batch_stride, 4) && mult(p.C_group_stride, 4);
    if constexpr (LPR == 1) {
        // the fixed shape of the Mamba1 decode step (see FAST in ssm_update_body)
        const bool fast_update = vec && p.dstate == 16 && p.nheads == 1 && p.ngroups == 1 && p.nhead_groups == 0 &&
                                 p.A_dstate_stride == 1 && p.A_dim_stride % 16 == 0 && aligned16(p.A_log) &&
                                 (!p.state_is_fp32 || (p.state_dim_stride == 16 && p.dim % 64 == 0)) &&
                                 !(p.dt_bias && p.dt_bias_is_fp16);
        if (!conv && fast_update) {
            auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, p); };
            p.state_is_fp32 ? go(ssm_update_kernel<1, true, true, true>) : go(ssm_update_kernel<1, true, false, true>);
            return check_launch();
        }
        if (conv) {
            auto fused = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, p, *conv); };
            const bool taps4 = fast_update && conv->width == 4 && conv->weight_width_stride == 1 &&
                               aligned4(conv->weight) && conv->weight_c_stride % 4 == 0 && conv->conv_state_l_stride == 1;
            const bool fast = taps4 && conv->conv_state_len == 4 && aligned4(conv->conv_state) &&
                              conv->conv_state_batch_stride % 4 == 0 && conv->conv_state_c_stride % 4 == 0;
            // a state of three codes per row, the rows back to back (the whole tensor has at least two rows)
            const bool fast3 = taps4 && conv->conv_state_len == 3 && conv->conv_state_c_stride == 3 &&
                               conv->conv_state_batch_stride == 3 * static_cast<int64_t>(conv->dim) &&
                               static_cast<int64_t>(conv->batch) * conv->dim >= 2;
            if (fast) p.state_is_fp32 ? fused(decode_step_kernel<true, true, true>) : fused(decode_step_kernel<true, false, true>);
            else if (fast3) p.state_is_fp32 ? fused(decode_step_kernel<true, true, true, 3>) : fused(decode_step_kernel<true, false, true, 3>);
            else if (p.state_is_fp32) vec ? fused(decode_step_kernel<true, true, false>) : fused(decode_step_kernel<false, true, false>);
            else vec ? fused(decode_step_kernel<true, false, false>) : fused(decode_step_kernel<false, false, false>);
            return check_launch();
        }
    }
    auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, p); };
    if (p.state_is_fp32) vec ? go(ssm_update_kernel<LPR, true, true>) : go(ssm_update_kernel<LPR, false, true>);
    else vec ? go(ssm_update_kernel<LPR, true, false>) : go(ssm_update_kernel<LPR, false, false>);
    return check_launch();
}

}  // namespace
}  // namespace qa

namespace qa {
namespace {
// How lanes are laid over channels and states for d_state <= 16, as a QA_SSCAN_MAPPING code.
// The kernel is bound by vector-ALU issue, so the mapping that wastes the fewest issue slots wins: four lanes per
// channel and, when the channel count allows, four waves per workgroup sharing one staged B/C tile.  With channel
// groups a workgroup must stay inside one group.
int choose_mapping16(const QaSScanParams& p) {
    const int per_group = p.dim / p.n_groups;
    int waves = p.dim % 64 == 0 ? 4 : (p.dim % 32 == 0 ? 2 : 1);
    while (waves > 1 && p.n_groups > 1 && per_group % (16 * waves) != 0) waves >>= 1;
    if (waves < 4) return QA_SSCAN_MAPPING(4, waves);
    // Waves per SIMD with four lanes per channel: q + f.  With 0 < f <= 1/2 the last f/(q+f) of the
    // channels of every batch entry go to the eight-lane kind (see sscan_fwd_mixed_kernel), as long as
    // both parts stay whole workgroups and, with channel groups, whole groups.
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
        cus = 256;
    }
    const int64_t simds = 4LL * cus;
    const int64_t waves_a = static_cast<int64_t>(p.batch) * p.dim / 16;
    const int64_t q = waves_a / simds, rem_waves = waves_a % simds;
    // Few waves (small batches): a launch takes about as long as the busiest SIMD's waves one after the
    // other, and with so few of them latency, not issue, sets a wave's pace - so twice as many waves
    // of two thirds the length (eight lanes per channel) finish sooner: up to 1.5 four-lane waves per SIMD.
    if (2 * waves_a <= 3 * simds && (p.n_groups <= 1 || per_group % 32 == 0)) return QA_SSCAN_MAPPING(8, 4);
    if (p.n_groups == 1 && q >= 1 && rem_waves > 0 && 2 * rem_waves <= simds) {
        const int64_t short_channels = rem_waves * 16 / p.batch;      // channels per batch entry for the short kind
        const int64_t blocks_a = (p.dim - short_channels) / 64;
        if (short_channels % 32 == 0 && (p.dim - short_channels) % 64 == 0 && blocks_a > 0 && blocks_a <= 0xfffff) {
            return QA_SSCAN_MAPPING(0, static_cast<int>(blocks_a));
        }
    }
    return QA_SSCAN_MAPPING(4, 4);
}
}  // namespace
}  // namespace qa

extern "C" int qa_sscan_chosen_mapping(const QaSScanParams* p) {
    if (!p) return QA_ERR_NULL;
    if (p->batch < 1 || p->dim < 1 || p->dstate < 1 || p->dstate > 256) return QA_ERR_SHAPE;
    if (p->n_groups < 1 || p->dim % p->n_groups != 0) return QA_ERR_SHAPE;
    if (p->dstate > 16) return 0;
    if (p->mapping != 0) return p->mapping;
    return qa::choose_mapping16(*p);
}

extern "C" int qa_sscan_fwd(const QaSScanParams* p, void* stream_) {
    using namespace qa;
    if (!p) return QA_ERR_NULL;
    if (p->batch < 0 || p->dim < 0 || p->seqlen < 0 || p->dstate < 1 || p->dstate > 256) return QA_ERR_SHAPE;
    if (p->n_groups < 1 || (p->dim > 0 && p->dim % p->n_groups != 0)) return QA_ERR_SHAPE;
    if (p->batch == 0 || p->dim == 0) return QA_OK;                 // (no channel rows: the tensors may be null)
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (p->seqlen == 0) {
        // no steps (the step tensors may be null): a scan from the zero state ends in the zero state
        if (p->carry_state || p->carry_dt_sum) return QA_ERR_SHAPE;
        const int64_t rows = static_cast<int64_t>(p->batch) * p->dim;
        int st = fill_zero(p->last_state_i8, rows * p->dstate, stream);
        if (st == QA_OK) st = fill_zero(p->last_state_f32, rows * p->dstate * 4, stream);
        if (st == QA_OK) st = fill_zero(p->dt_sum_out, rows * 4, stream);
        return st;
    }
    if (!p->u || !p->delta || !p->A_log || !p->B || !p->C || !p->out) return QA_ERR_NULL;
    if (!p->scale_u || !p->scale_delta || !p->scale_A || !p->scale_B || !p->scale_C) return QA_ERR_NULL;
    if ((p->D && !p->scale_D) || (p->delta_bias && !p->scale_delta_bias) || (p->z && !p->scale_z)) return QA_ERR_NULL;
    if (p->last_state_i8 && !p->scale_ssm_state) return QA_ERR_NULL;
    if (p->batch > 65535) return QA_ERR_SHAPE;

    auto ok16 = [](const void* ptr, std::initializer_list<int64_t> strides) {
        if (!aligned16(ptr)) return 0;
        for (int64_t s : strides) if (s % 16 != 0) return 0;
        return 1;
    };
    int vec_in = ok16(p->u, {p->u_batch_stride, p->u_d_stride}) && ok16(p->delta, {p->delta_batch_stride, p->delta_d_stride});
    if (p->z) vec_in = vec_in && ok16(p->z, {p->z_batch_stride, p->z_d_stride});
    const int vec_bc = ok16(p->B, {p->B_batch_stride, p->B_group_stride, p->B_dstate_stride}) &&
                       ok16(p->C, {p->C_batch_stride, p->C_group_stride, p->C_dstate_stride});
    const int vec_out = p->out_d_stride == 1 && aligned16(p->out) && p->out_batch_stride % 8 == 0 &&
                        p->out_l_stride % 8 == 0;

    const int N = p->dstate;
    if (p->mapping != 0) {
        // a lane mapping named by the caller (tests): only d_state <= 16 has more than one
        // a value without the marker bit of QA_SSCAN_MAPPING is not a mapping (an uninitialised field, say)
        if ((p->mapping & ~0x0fffffff) != 0x40000000 || N > 16) return QA_ERR_UNSUPPORTED;
        const int lanes = (p->mapping >> 20) & 0xff, arg = p->mapping & 0xfffff;
        if (lanes == 0) {
            // mixed launch: `arg` workgroups of 64 channels with four lanes per channel, the rest with eight
            if (arg < 1 || p->n_groups != 1 || 64LL * arg > p->dim) return QA_ERR_SHAPE;
            return launch_fwd_mixed(*p, stream, vec_in, vec_bc, vec_out, arg);
        }
        if (lanes == 1 && arg == 1) return launch_fwd<16, 1, 64, 1>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 2 && arg == 1) return launch_fwd<8, 2, 64, 1>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 2 && arg == 2) return launch_fwd<8, 2, 64, 2>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 4 && arg == 1) return launch_fwd_pre<4, 4, 1>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 4 && arg == 2) return launch_fwd_pre<4, 4, 2>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 4 && arg == 4) return launch_fwd_pre<4, 4, 4>(*p, stream, vec_in, vec_bc, vec_out);
        if (lanes == 8 && arg == 4) return launch_fwd_pre<2, 8, 4>(*p, stream, vec_in, vec_bc, vec_out);
        return QA_ERR_UNSUPPORTED;
    }
    if (N <= 16) {
        const int mapping = choose_mapping16(*p);
        const int lanes = (mapping >> 20) & 0xff, arg = mapping & 0xfffff;
        if (lanes == 0) return launch_fwd_mixed(*p, stream, vec_in, vec_bc, vec_out, arg);
        if (lanes == 8) return launch_fwd_pre<2, 8, 4>(*p, stream, vec_in, vec_bc, vec_out);
        if (arg == 4) return launch_fwd_pre<4, 4, 4>(*p, stream, vec_in, vec_bc, vec_out);
        if (arg == 2) return launch_fwd_pre<4, 4, 2>(*p, stream, vec_in, vec_bc, vec_out);
        return launch_fwd_pre<4, 4, 1>(*p, stream, vec_in, vec_bc, vec_out);
    }
    // Wider states: eight states per lane, or sixteen.  A workgroup converts its B/C tile once for all of its
    // channels, so with enough channels to fill the part four waves share one tile (64 or 32 channels per
    // workgroup); few channels keep one wave per workgroup, which gives more workgroups.
    auto many = [&](int channels_per_wg) {
        const int64_t wgs = static_cast<int64_t>(p->batch) * ((p->dim + channels_per_wg - 1) / channels_per_wg);
        return wgs >= 128 && (p->n_groups <= 1 || (p->dim / p->n_groups) % channels_per_wg == 0);
    };
    if (N <= 32) {
        if (many(64)) return launch_fwd<8, 4, 64, 4>(*p, stream, vec_in, vec_bc, vec_out);
        return launch_fwd<8, 4, 64, 1>(*p, stream, vec_in, vec_bc, vec_out);
    }
    if (N <= 64) {
        if (many(32)) return launch_fwd<8, 8, 32, 4>(*p, stream, vec_in, vec_bc, vec_out);
        return launch_fwd<8, 8, 32, 1>(*p, stream, vec_in, vec_bc, vec_out);
    }
    if (N <= 128) {
        if (many(32)) return launch_fwd<16, 8, 32, 4>(*p, stream, vec_in, vec_bc, vec_out);
        return launch_fwd<16, 8, 32, 1>(*p, stream, vec_in, vec_bc, vec_out);
    }
    return launch_fwd<16, 16, 16, 1>(*p, stream, vec_in, vec_bc, vec_out);
}

namespace qa {
namespace {
int validate_update(const QaSsmUpdateParams* p, bool needs_x) {
    if (!p) return QA_ERR_NULL;
    if (p->batch == 0 && p->nheads >= 1 && p->dim >= 0) return QA_OK;      // (no batch entries: the tensors may be null)
    if (!p->state || (needs_x && !p->x) || !p->dt || !p->A_log || !p->B || !p->C || !p->out) return QA_ERR_NULL;
    if (!p->x_scale || !p->dt_scale || !p->A_log_scale || !p->B_scale || !p->C_scale) return QA_ERR_NULL;
    if (!p->state_is_fp32 && !p->state_scale) return QA_ERR_NULL;
    if ((p->D && !p->D_scale) || (p->z && !p->z_scale)) return QA_ERR_NULL;
    if (p->dt_bias && !p->dt_bias_is_fp16 && !p->dt_bias_scale) return QA_ERR_NULL;
    if (p->nhead_groups > 0 && (!p->x_head_group_range || !p->x_dim_group_range || p->ndim_groups < 1)) return QA_ERR_NULL;
    if (p->batch < 0 || p->nheads < 1 || p->dim < 0 || p->dstate < 1 || p->dstate > 256) return QA_ERR_SHAPE;
    if (p->ngroups < 1 || p->nheads % p->ngroups != 0) return QA_ERR_SHAPE;
    return QA_OK;
}
}  // namespace
}  // namespace qa

extern "C" int qa_ssm_state_update(const QaSsmUpdateParams* p, void* stream_) {
    using namespace qa;
    const int st = validate_update(p, true);
    if (st != QA_OK) return st;
    if (p->batch == 0 || p->dim == 0) return QA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int N = p->dstate;
    // up to sixteen states per lane: the per-row work (addresses, softplus, gate) is paid once per lane
    if (N <= 16) return launch_update<1>(*p, stream);
    if (N <= 32) return launch_update<2>(*p, stream);
    if (N <= 64) return launch_update<4>(*p, stream);
    if (N <= 128) return launch_update<8>(*p, stream);
    return launch_update<16>(*p, stream);
}

extern "C" int qa_mamba1_decode_step(const QaConvParams* conv, const QaSsmUpdateParams* p, void* stream_) {
    using namespace qa;
    const int st = validate_update(p, false);
    if (st != QA_OK) return st;
    if (!conv) return QA_ERR_NULL;
    if (p->batch == 0 && conv->batch == 0) return QA_OK;
    if (!conv->x || !conv->weight || !conv->conv_state) return QA_ERR_NULL;
    if (conv->width < 2 || conv->width > 4) return QA_ERR_SHAPE;
    if (conv->conv_state_len != conv->width && conv->conv_state_len != conv->width - 1) return QA_ERR_SHAPE;
    if (conv->batch != p->batch || conv->dim != p->dim) return QA_ERR_SHAPE;
    // one lane per (batch, channel) row carries both steps: one head, at most sixteen states, per-tensor scales
    if (p->nheads != 1 || p->dstate > 16 || p->nhead_groups > 0) return QA_ERR_UNSUPPORTED;
    if (p->batch == 0 || p->dim == 0) return QA_OK;
    return launch_update<1>(*p, static_cast<hipStream_t>(stream_), conv);
}
