// Mamba2 quantized SSD chunk scan for any head dimension (<= 256), state count and chunk length, and for tensors
// without 16-byte alignment: the shapes the matrix-core kernels of ssd.hip are not built for.
//
// Same stages, same arithmetic and the same fp16 rounding points as there (quamba/triton/quant_ssd_combined.py
// :61-77, grouped :146-162; the kernels restated are named at each stage) and the same matrix instructions, on 64-wide
// tiles in every dimension that pass through LDS with everything past an edge set to zero there; loads are bounded,
// and byte-wise unless sizes and addresses allow words or 16-byte pieces, so that nothing depends on a size being a
// multiple of anything:
//   cumsum      dt = clamp(softplus(s_dt q_dt + dt_bias)), dA_cs = within-chunk cumsum(dt * A)
//   state       S_c[p,n] = sum_k f16(x^[k,p]) f16(B^[k,n] (exp(dA_last - dA_k) dt_k));  P_{c+1} = exp(dA_last) P_c + S_c,
//               f16(P_c) stored as the state entering chunk c; final state fp32 / int8
//   chunk_scan  y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) f16(P_c[p,n])
//                      + sum_{k<=m} f16(((s_C s_B) (q_C[m,:] . q_B[k,:])) exp(dA_m - dA_k) dt_k) f16(x^[k,p])
//                      + x^[m,p] D, optional z gate, fp16 out
// All sums are fp32 (v_mfma_f32_16x16x32_f16 on fp16-rounded operands); the integer contraction of C and B is exact
// (v_mfma_i32_16x16x64_i8).
#include "qa_common.hpp"
#include "ssd_common.hpp"

namespace qa {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kT = 64;            // tile edge: steps, states, channels of the chunk scan
constexpr int kThreads = 256;

__device__ __forceinline__ float f16r(float v) { return static_cast<float>(static_cast<_Float16>(v)); }

// ---------------------------------------------------------------------------------------------
// Stage 1 (quamba/triton/quant_chunk_cumsum.py:56-70).  One wave per (batch, chunk, head): every lane takes
// ceil(chunk_size / 64) consecutive steps, then an inclusive scan across the lanes.  Steps past the end of the
// sequence have dt = 0.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void ssd_general_cumsum_kernel(QaSsdParams p, float* dt_out, float* dA_out, float* xs_out, int32_t* srow_out, int nc) {
    const int lane = threadIdx.x & 63;
    const unsigned idx = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (idx >= static_cast<unsigned>(p.batch) * static_cast<unsigned>(nc) * static_cast<unsigned>(p.nheads)) return;
    const int h = static_cast<int>(idx % static_cast<unsigned>(p.nheads));
    const int c = static_cast<int>((idx / static_cast<unsigned>(p.nheads)) % static_cast<unsigned>(nc));
    const int b = static_cast<int>(idx / (static_cast<unsigned>(p.nheads) * static_cast<unsigned>(nc)));
    const int Q = p.chunk_size, E = (Q + 63) / 64;
    if (b == 0 && c == 0) ssd_write_channel_tables(p, h, lane, xs_out, srow_out);
    const float A = -expf(*p.A_log_scale * static_cast<float>(p.A_log[h]));
    const float s_dt = p.dt_is_fp32 ? 0.0f : *p.dt_scale;
    const float bias = (!p.dt_is_fp32 && p.dt_bias) ? __half2float(static_cast<const __half*>(p.dt_bias)[h]) : 0.0f;
    float* dt_row = dt_out + ((static_cast<int64_t>(b) * p.nheads + h) * nc + c) * Q;
    float* dA_row = dA_out + ((static_cast<int64_t>(b) * p.nheads + h) * nc + c) * Q;
    float local = 0.0f;
    for (int e = 0; e < E; ++e) {
        const int k = lane * E + e;
        if (k >= Q) break;
        const int t = c * Q + k;
        float v = 0.0f;
        if (t < p.seqlen) {
            const int64_t di = (static_cast<int64_t>(b) * p.seqlen + t) * p.nheads + h;
            if (p.dt_is_fp32) {
                v = static_cast<const float*>(p.dt)[di];
            } else {
                v = s_dt * static_cast<float>(static_cast<const int8_t*>(p.dt)[di]) + bias;
                if (p.dt_softplus) v = v <= 20.0f ? log1pf(expf(v)) : v;
                v = fminf(fmaxf(v, p.dt_min), p.dt_max);
            }
        }
        dt_row[k] = v;
        local += v * A;
    }
    float incl = local;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    const float before = incl - local;
    // second pass over the lane's own steps (it wrote them itself)
    float run = 0.0f;
    for (int e = 0; e < E; ++e) {
        const int k = lane * E + e;
        if (k >= Q) break;
        run += dt_row[k] * A;
        dA_row[k] = before + run;
    }
}

// what the tensors' sizes and addresses allow (chosen on the host)
constexpr int kVecCodes = 1;      // B, C: rows of 16-byte pieces
constexpr int kVecX = 2;          // x: four channels per aligned word
constexpr int kVecState = 4;      // entering state: rows of 16-byte pieces
constexpr int kVecB4 = 8;         // B: four states per aligned word

// 64 steps x 64 columns of int8 codes (x: channels, B: states; rows `row_step` bytes apart, `width` columns in all,
// the tile's first column col0) become fp16 values in LDS, transposed to [column][step]: a thread takes four steps
// of four columns.  value(code, local column, local step) does the arithmetic; steps from `steps` on and columns from
// `width` on are zero.
template <typename F>
__device__ __forceinline__ void stage_transposed(_Float16 (*dst)[kT + 8], const int8_t* rows0, int64_t row_step, int steps, int col0,
                                                 int width, bool words, int tid, F&& value) {
    const int kb = tid / 16, cq = tid % 16, col = col0 + 4 * cq;
    uint32_t w[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int k = 4 * kb + r;
        w[r] = 0u;
        if (k < steps && col < width) {
            const int8_t* src = rows0 + k * row_step + col;
            if (words && col + 4 <= width) {
                w[r] = *reinterpret_cast<const uint32_t*>(src);
            } else {
                for (int e = 0; e < 4 && col + e < width; ++e) w[r] |= static_cast<uint32_t>(static_cast<uint8_t>(src[e])) << (8 * e);
            }
        }
    }
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
        v4h v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = static_cast<_Float16>(value(static_cast<float>(static_cast<int8_t>((w[r] >> (8 * cc)) & 0xffu)), 4 * cq + cc, 4 * kb + r));
        *reinterpret_cast<v4h*>(&dst[4 * cq + cc][4 * kb]) = v;
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 2, 3 and 6 (quamba/triton/quant_chunk_state.py:76-89, quant_state_passing.py:60-83, quant_ssm_states.py
// :43,119).  A workgroup of four waves per (batch, head, 64 channels, 64 states) walks the chunks in order with its
// part of the running state in registers: a wave owns sixteen states and all 64 channels (four accumulator tiles
// of v_mfma_f32_16x16x32_f16: a lane holds channels 16 j + 4 (lane / 16) + r, state lane % 16).  The chunk's
// operands pass through LDS in tiles of 64 steps, rounded to fp16 and transposed to [channel][step] and
// [state][step]; everything past an edge is zero there.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void ssd_general_state_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws, __half* prev, const float* xs_ws,
                                                                     const int32_t* srow_ws, int nc, int vec) {
    __shared__ __attribute__((aligned(16))) _Float16 xt[kT][kT + 8];      // x^ [channel][step]
    __shared__ __attribute__((aligned(16))) _Float16 bt[kT][kT + 8];      // B^ w [state][step]
    __shared__ float wk[kT];
    __shared__ float xs[kT];
    __shared__ int32_t srow[kT];
    const int P = p.headdim, N = p.dstate, Q = p.chunk_size, H = p.nheads, G = p.ngroups, L = p.seqlen;
    const int ptiles = (P + kT - 1) / kT, ntiles = (N + kT - 1) / kT;
    const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned idx = blockIdx.x;
    const int n0 = static_cast<int>(idx % ntiles) * kT; idx /= ntiles;
    const int p0 = static_cast<int>(idx % ptiles) * kT; idx /= ptiles;
    const int h = static_cast<int>(idx % H);
    const int b = static_cast<int>(idx / H);
    int g, hg;
    ssd_group_of(p, h, g, hg);
    const float sB = p.nhead_groups > 0 ? p.B_scale[g] : p.B_scale[0];
    if (tid < kT) {
        xs[tid] = p0 + tid < P ? xs_ws[h * P + p0 + tid] : 0.0f;
        srow[tid] = p0 + tid < P ? srow_ws[h * P + p0 + tid] : 0;
    }
    const int64_t rows0 = (static_cast<int64_t>(b) * H + h) * nc;
    const int64_t xstep = static_cast<int64_t>(H) * P, bstep = static_cast<int64_t>(G) * N;
    v4f run[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) run[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    for (int c = 0; c < nc; ++c) {
        const int t0 = c * Q;
        const int lim = min(Q, L - t0);
        const float* dA_row = dA_ws + (rows0 + c) * Q;
        const float* dt_row = dt_ws + (rows0 + c) * Q;
        const float dA_last = dA_row[Q - 1];
        const int8_t* xrow0 = p.x + ((static_cast<int64_t>(b) * L + t0) * H + h) * P;
        const int8_t* Brow0 = p.B + ((static_cast<int64_t>(b) * L + t0) * G + g) * N;
        v4f acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        for (int k0 = 0; k0 < lim; k0 += kT) {
            __syncthreads();                                       // the tile before is consumed (first pass: xs is written)
            if (tid < kT) wk[tid] = k0 + tid < lim ? ssd_exp(dA_last - dA_row[k0 + tid]) * dt_row[k0 + tid] : 0.0f;
            __syncthreads();
            stage_transposed(xt, xrow0 + k0 * xstep, xstep, lim - k0, p0, P, (vec & kVecX) != 0, tid,
                             [&](float q, int col, int) { return xs[col] * q; });
            stage_transposed(bt, Brow0 + k0 * bstep, bstep, lim - k0, n0, N, (vec & kVecB4) != 0, tid,
                             [&](float q, int, int k) { return (sB * q) * wk[k]; });
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (k0 + 32 * ks < lim) {
                    const v8h bf = *reinterpret_cast<const v8h*>(&bt[16 * wave + l16][32 * ks + 8 * lq]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const v8h xf = *reinterpret_cast<const v8h*>(&xt[16 * j + l16][32 * ks + 8 * lq]);
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, bf, acc[j], 0, 0, 0);
                    }
                }
            }
        }
        // P <- exp(dA_last) P + S
        const float decay = ssd_exp(dA_last);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) run[j][r] = decay * run[j][r] + acc[j][r];
        if (c + 1 < nc) {
            // the state entering chunk c + 1, in fp16 as the reference keeps it
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int pp = p0 + 16 * j + 4 * lq + r, nn = n0 + 16 * wave + l16;
                    if (pp < P && nn < N) prev[(((static_cast<int64_t>(b) * nc + c + 1) * H + h) * P + pp) * N + nn] = __float2half(run[j][r]);
                }
        }
    }

    if (p.final_states) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int pp = p0 + 16 * j + 4 * lq + r, nn = n0 + 16 * wave + l16;
                if (pp < P && nn < N) {
                    const int64_t fo = ((static_cast<int64_t>(b) * H + h) * P + pp) * N + nn;
                    if (p.final_state_is_fp32) static_cast<float*>(p.final_states)[fo] = run[j][r];
                    else static_cast<int8_t*>(p.final_states)[fo] = ssd_quantize_state(p, srow[pp - p0], nn, run[j][r]);
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 4 and 5 (quamba/triton/quant_bmm_chunk.py:60-66, quant_chunk_scan.py:96-171).  A workgroup of four waves per
// (batch, chunk, head, 64 rows m, 64 channels p); a wave owns sixteen rows and all 64 channels (four accumulator
// tiles of v_mfma_f32_16x16x32_f16: a lane holds rows 4 (lane / 16) + r, channel 16 j + lane % 16).
// Term 1 walks the states in tiles of 64: C^ converted in registers from the codes in LDS, the entering state as rows
// of channels.  Term 2 walks the steps k up to the diagonal in tiles of 64: v_mfma_i32_16x16x64_i8 forms the tile's
// integer (C B^T)^T from the codes (exact), a lane turns its four steps of a row into fp16 weights, the wave passes
// them through its own rows of LDS into operand order, and x^ waits there transposed ([channel][step]).
// Everything past an edge (rows, steps, states, channels) is zero in LDS, so the products need no bounds.
// ---------------------------------------------------------------------------------------------
struct GeneralScanSmem {
    // 16 pad bytes per row: the sixteen rows of an operand read fall into different banks
    __attribute__((aligned(16))) int8_t cq[kT][kT + 16];         // C codes of the rows m, one tile of 64 states
    __attribute__((aligned(16))) int8_t bq[kT][kT + 16];         // B codes of the steps k
    __attribute__((aligned(16))) _Float16 wt[kT][kT + 8];        // weights [row m][step k]
    __attribute__((aligned(16))) _Float16 xt[kT][kT + 8];        // term 2: x^ [channel][step k]; term 1: entering state [channel][state]
    float dA_m[kT], dA_k[kT], dt_k[kT], xs[kT], Dv[kT];
};

__global__ __launch_bounds__(kThreads) void ssd_general_chunk_scan_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws, const __half* prev,
                                                                          const float* xs_ws, int nc, int vec) {
    __shared__ GeneralScanSmem sm;
    const int P = p.headdim, N = p.dstate, Q = p.chunk_size, H = p.nheads, G = p.ngroups, L = p.seqlen;
    const int ptiles = (P + kT - 1) / kT, mtiles = (Q + kT - 1) / kT;
    const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned idx = blockIdx.x;
    const int p0 = static_cast<int>(idx % ptiles) * kT; idx /= ptiles;
    const int m0 = static_cast<int>(idx % mtiles) * kT; idx /= mtiles;
    const int h = static_cast<int>(idx % H); idx /= H;
    const int c = static_cast<int>(idx % nc);
    const int b = static_cast<int>(idx / nc);
    const int t0 = c * Q;
    const int lim = min(Q, L - t0);
    if (m0 >= lim) return;                                         // (the whole workgroup: nothing of this tile exists)
    int g, hg;
    ssd_group_of(p, h, g, hg);
    const bool grouped = p.nhead_groups > 0;
    const float sC = grouped ? p.C_scale[g] : p.C_scale[0];
    const float cb_scale = sC * (grouped ? p.B_scale[g] : p.B_scale[0]);
    const float* dA_row = dA_ws + ((static_cast<int64_t>(b) * H + h) * nc + c) * Q;
    const float* dt_row = dt_ws + ((static_cast<int64_t>(b) * H + h) * nc + c) * Q;
    const int8_t* xrow0 = p.x + ((static_cast<int64_t>(b) * L + t0) * H + h) * P;          // step k: + k H P
    const int8_t* Brow0 = p.B + ((static_cast<int64_t>(b) * L + t0) * G + g) * N;          // step k: + k G N
    const int8_t* Crow0 = p.C + ((static_cast<int64_t>(b) * L + t0) * G + g) * N;
    const int64_t xstep = static_cast<int64_t>(H) * P, cstep = static_cast<int64_t>(G) * N;

    if (tid < kT) {
        const int pp = p0 + tid;
        sm.xs[tid] = pp < P ? xs_ws[h * P + pp] : 0.0f;
        sm.Dv[tid] = (!p.D || pp >= P) ? 0.0f : *p.D_scale * static_cast<float>(p.D_has_hdim ? p.D[h * P + pp] : p.D[h]);
        sm.dA_m[tid] = dA_row[min(m0 + tid, Q - 1)];
    }

    // 64 rows x 64 codes of B or C (rows from `first`, states from n0) into LDS: a thread moves one 16-byte piece
    auto stage_codes = [&](int8_t (*dst)[kT + 16], const int8_t* rows0, int first, int n0) {
        const int r = tid / 4, q = tid % 4, row = first + r, n = n0 + 16 * q;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < lim && n < N) {
            const int8_t* src = rows0 + row * cstep + n;
            if ((vec & kVecCodes) && n + 16 <= N) {
                v = *reinterpret_cast<const uint4*>(src);
            } else {
                uint32_t w[4] = {0u, 0u, 0u, 0u};
                for (int e = 0; e < 16 && n + e < N; ++e) w[e / 4] |= static_cast<uint32_t>(static_cast<uint8_t>(src[e])) << (8 * (e % 4));
                v = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
        *reinterpret_cast<uint4*>(&dst[r][16 * q]) = v;
    };

    v4f acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // term 1: C^ (rows m) x the state entering the chunk (rows p); zero for the first chunk
    if (c > 0) {
        const __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * P * N;
        for (int n0 = 0; n0 < N; n0 += kT) {
            __syncthreads();                                       // the tile before is consumed
            stage_codes(sm.cq, Crow0, m0, n0);
            {
                // the entering state of 64 channels x 64 states: a thread moves sixteen states of one channel
                const int r = tid / 4, q = tid % 4, pp = p0 + r, n = n0 + 16 * q;
                uint4 v0 = make_uint4(0u, 0u, 0u, 0u), v1 = v0;
                if (pp < P && n < N) {
                    const __half* src = pst + static_cast<int64_t>(pp) * N + n;
                    if ((vec & kVecState) && n + 16 <= N) {
                        v0 = *reinterpret_cast<const uint4*>(src);
                        v1 = *reinterpret_cast<const uint4*>(src + 8);
                    } else {
                        uint32_t w[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
                        for (int e = 0; e < 16 && n + e < N; ++e) w[e / 2] |= static_cast<uint32_t>(__half_as_ushort(src[e])) << (16 * (e % 2));
                        v0 = make_uint4(w[0], w[1], w[2], w[3]);
                        v1 = make_uint4(w[4], w[5], w[6], w[7]);
                    }
                }
                *reinterpret_cast<uint4*>(&sm.xt[r][16 * q]) = v0;
                *reinterpret_cast<uint4*>(&sm.xt[r][16 * q + 8]) = v1;
            }
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const uint2 cw = *reinterpret_cast<const uint2*>(&sm.cq[16 * wave + l16][32 * ks + 8 * lq]);
                v8h cf;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    cf[e] = static_cast<_Float16>(sC * static_cast<float>(static_cast<int8_t>((cw.x >> (8 * e)) & 0xffu)));
                    cf[4 + e] = static_cast<_Float16>(sC * static_cast<float>(static_cast<int8_t>((cw.y >> (8 * e)) & 0xffu)));
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v8h pf = *reinterpret_cast<const v8h*>(&sm.xt[16 * j + l16][32 * ks + 8 * lq]);
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cf, pf, acc[j], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float em = ssd_exp(sm.dA_m[16 * wave + 4 * lq + r]);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j][r] *= em;
        }
    }

    // term 2: steps k <= m, tiles of 64 steps up to the one that holds the last row's diagonal
    const int k_end = min(m0 + kT, lim);
    const int m_last = m0 + 16 * wave + 15;                        // the wave's last row
    for (int k0 = 0; k0 < k_end; k0 += kT) {
        __syncthreads();                                           // the tiles before are consumed
        if (tid < kT) {
            const int k = k0 + tid;
            sm.dA_k[tid] = dA_row[min(k, Q - 1)];
            sm.dt_k[tid] = k < lim ? dt_row[k] : 0.0f;
        }
        // x^ of 64 steps x 64 channels, transposed (xs was written before the first barrier of this kernel)
        stage_transposed(sm.xt, xrow0 + k0 * xstep, xstep, lim - k0, p0, P, (vec & kVecX) != 0, tid,
                         [&](float q, int col, int) { return sm.xs[col] * q; });
        // integer (C B^T)^T of the wave's rows: block kb holds steps 16 kb + 4 (lane / 16) + r of row lane % 16
        v4i cb[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) cb[kb] = v4i{0, 0, 0, 0};
        for (int n0 = 0; n0 < N; n0 += kT) {
            if (n0 > 0) __syncthreads();
            stage_codes(sm.cq, Crow0, m0, n0);
            stage_codes(sm.bq, Brow0, k0, n0);
            __syncthreads();
            const v4i co = *reinterpret_cast<const v4i*>(&sm.cq[16 * wave + l16][16 * lq]);
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) {
                if (k0 + 16 * kb <= m_last) {                      // (blocks wholly above the diagonal stay zero)
                    const v4i bo = *reinterpret_cast<const v4i*>(&sm.bq[16 * kb + l16][16 * lq]);
                    cb[kb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bo, co, cb[kb], 0, 0, 0);
                }
            }
        }
        // the weights, rounded to fp16 where the reference rounds them, into the wave's own rows of LDS
        {
            const int m = m0 + 16 * wave + l16;
            const float dAm = sm.dA_m[16 * wave + l16];
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) {
                v4h wv;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int kk = 16 * kb + 4 * lq + r;
                    const float w = ((cb_scale * static_cast<float>(cb[kb][r])) * ssd_exp(dAm - sm.dA_k[kk])) * sm.dt_k[kk];
                    wv[r] = (k0 + kk <= m && m < lim) ? static_cast<_Float16>(w) : static_cast<_Float16>(0.0f);
                }
                *reinterpret_cast<v4h*>(&sm.wt[16 * wave + l16][16 * kb + 4 * lq]) = wv;
            }
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            if (k0 + 32 * ks <= m_last) {
                const v8h wf = *reinterpret_cast<const v8h*>(&sm.wt[16 * wave + l16][32 * ks + 8 * lq]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v8h xf = *reinterpret_cast<const v8h*>(&sm.xt[16 * j + l16][32 * ks + 8 * lq]);
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, xf, acc[j], 0, 0, 0);
                }
            }
        }
    }

    // skip term, gate, fp16 out: acc[j][r] is row 16 wave + 4 (lane / 16) + r, channel 16 j + lane % 16
    const float z_scale = p.z ? *p.z_scale : 0.0f;
    __half* out = static_cast<__half*>(p.out) + ((static_cast<int64_t>(b) * L + t0) * H + h) * P;
    const int8_t* zrow0 = p.z ? p.z + ((static_cast<int64_t>(b) * L + t0) * H + h) * P : nullptr;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = m0 + 16 * wave + 4 * lq + r;
        if (m >= lim) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int pl = 16 * j + l16, pp = p0 + pl;
            if (pp >= P) continue;
            float y = acc[j][r];
            if (p.D) y += (sm.xs[pl] * static_cast<float>(xrow0[m * xstep + pp])) * sm.Dv[pl];
            if (p.z) {
                const float zv = z_scale * static_cast<float>(zrow0[m * xstep + pp]);
                y *= zv * __builtin_amdgcn_rcpf(1.0f + ssd_exp(-zv));
            }
            out[m * xstep + pp] = __float2half(y);
        }
    }
}

}  // namespace

int ssd_general_grid_check(const QaSsdParams& p) {
    const int64_t nc = (static_cast<int64_t>(p.seqlen) + p.chunk_size - 1) / p.chunk_size;
    const int64_t scan = static_cast<int64_t>(p.batch) * nc * p.nheads * ((p.chunk_size + kT - 1) / kT) * ((p.headdim + kT - 1) / kT);
    const int64_t state = static_cast<int64_t>(p.batch) * p.nheads * ((p.headdim + kT - 1) / kT) * ((p.dstate + kT - 1) / kT);
    // one-dimensional grids; the cumsum kernel numbers its (batch, chunk, head) items in 32 bits
    if (scan > 0x7fffffffLL || state > 0x7fffffffLL) return QA_ERR_SHAPE;
    return QA_OK;
}

void ssd_general_launch(const QaSsdParams& p, float* dt_ws, float* dA_ws, __half* prev_ws, float* xs_ws, int32_t* srow_ws, int nc,
                        hipStream_t stream) {
    const int64_t bch = static_cast<int64_t>(p.batch) * nc * p.nheads;
    const int64_t scan = bch * ((p.chunk_size + kT - 1) / kT) * ((p.headdim + kT - 1) / kT);
    const int64_t state = static_cast<int64_t>(p.batch) * p.nheads * ((p.headdim + kT - 1) / kT) * ((p.dstate + kT - 1) / kT);
    hipLaunchKernelGGL(ssd_general_cumsum_kernel, dim3(static_cast<unsigned>((bch + 3) / 4)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, xs_ws, srow_ws, nc);
    int vec = 0;
    if (p.dstate % 16 == 0 && aligned16(p.B) && aligned16(p.C)) vec |= kVecCodes;
    if (p.headdim % 4 == 0 && aligned4(p.x)) vec |= kVecX;
    if (p.dstate % 8 == 0) vec |= kVecState;                       // (the workspace itself is 256-byte aligned)
    if (p.dstate % 4 == 0 && aligned4(p.B)) vec |= kVecB4;
    hipLaunchKernelGGL(ssd_general_state_kernel, dim3(static_cast<unsigned>(state)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, prev_ws, xs_ws, srow_ws,
                       nc, vec);
    hipLaunchKernelGGL(ssd_general_chunk_scan_kernel, dim3(static_cast<unsigned>(scan)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, prev_ws, xs_ws, nc, vec);
}

}  // namespace qa
