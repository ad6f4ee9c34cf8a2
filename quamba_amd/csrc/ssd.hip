// Mamba2 quantized SSD chunk scan (prefill) for gfx950.
//
// Stages and arithmetic follow the reference's Triton pipeline (quamba/triton/quant_ssd_combined.py
// :61-77, grouped :146-162); see each kernel for the file it restates.  fp16 operands rounded where the
// reference rounds them, fp32 accumulation, as there; the one pure int8 contraction (C B^T) runs on the
// int8 matrix cores inside the chunk scan and stays in fp32 registers.
//   cumsum      dt = clamp(softplus(s_dt q_dt + dt_bias)), dA_cs = within-chunk cumsum(dt * A)
//   state       S_c[p,n] = sum_k f16(x^[k,p]) f16(B^[k,n] exp(dA_last - dA_k) dt_k)   (fp16 MFMA)
//               P_0 = 0, P_{c+1} = exp(dA_last,c) P_c + S_c in registers; P_c stored in fp16; final state fp32 / int8
//   chunk_scan  CB[m,k] = (s_C s_B) * sum_n q_C[m,n] q_B[k,n]                       (int8 MFMA, at and below the diagonal)
//               y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) f16(P_c[p,n]) + sum_{k<=m} f16(CB[m,k] e^{dA_m-dA_k} dt_k) f16(x^[k,p])
//               + D x^[m,p], optional z gate, fp16 out                               (fp16 MFMA)
// Both fp16 contractions over the time index need x (and B) with time as the fastest-moving index,
// while memory has channels fastest; the tiles are transposed once on the way into LDS and then read as
// 16-byte MFMA operands.
#include <atomic>
#include <mutex>

#include "qa_common.hpp"
#include "ssd_common.hpp"

namespace qa {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kP = 64;          // head dimension of these kernels
__device__ __forceinline__ float fexp(float x) { return ssd_exp(x); }
__device__ __forceinline__ int8_t byte_of(uint32_t w, int j) { return static_cast<int8_t>((w >> (8 * j)) & 0xffu); }

// ---------------------------------------------------------------------------------------------
// Stage 1 (quamba/triton/quant_chunk_cumsum.py:56-70).  One wave per (batch, chunk, head): every
// lane processes chunk_size/64 consecutive steps, then an inclusive scan across the lanes.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ssd_cumsum_kernel(QaSsdParams p, float* dt_out, float* dA_out, float* xs_out, int32_t* srow_out, int nc) {
    const int lane = threadIdx.x & 63;
    // the item is the same for a whole wave and below 2^31 (the host checks): its decomposition is 32-bit arithmetic on
    // a uniform value instead of 64-bit divisions in every lane
    const unsigned idx = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (idx >= static_cast<unsigned>(p.batch) * static_cast<unsigned>(nc) * static_cast<unsigned>(p.nheads)) return;
    const int h = static_cast<int>(idx % static_cast<unsigned>(p.nheads));
    const int c = static_cast<int>((idx / static_cast<unsigned>(p.nheads)) % static_cast<unsigned>(nc));
    const int b = static_cast<int>(idx / (static_cast<unsigned>(p.nheads) * static_cast<unsigned>(nc)));
    const int Q = p.chunk_size, E = Q / 64;            // Q in {64, 128, 256}
    if (b == 0 && c == 0) ssd_write_channel_tables(p, h, lane, xs_out, srow_out);
    const float A = -expf(*p.A_log_scale * static_cast<float>(p.A_log[h]));
    const float s_dt = p.dt_is_fp32 ? 0.0f : *p.dt_scale;
    const float bias = (!p.dt_is_fp32 && p.dt_bias) ? __half2float(static_cast<const __half*>(p.dt_bias)[h]) : 0.0f;
    float dtv[4], run[4];
    float local = 0.0f;
    for (int e = 0; e < E; ++e) {
        const int t = c * Q + lane * E + e;
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
        dtv[e] = v;
        local += v * A;
        run[e] = local;
    }
    // exclusive prefix of the lane totals
    float incl = local;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    const float before = incl - local;
    float* dt_row = dt_out + ((static_cast<int64_t>(b) * p.nheads + h) * nc + c) * Q + lane * E;
    float* dA_row = dA_out + ((static_cast<int64_t>(b) * p.nheads + h) * nc + c) * Q + lane * E;
    for (int e = 0; e < E; ++e) {
        dt_row[e] = dtv[e];
        dA_row[e] = before + run[e];
    }
}

// ---------------------------------------------------------------------------------------------
// The fp16 contractions run on v_mfma_f32_16x16x32_f16 with the operands rounded to fp16 where the reference
// rounds them, so that the products agree and only the order of the fp32 sums differs:
//   S_c[p,n] = sum_k f16(x^[k,p]) f16(B^[k,n] exp(dA_last - dA_k) dt_k);   P_{c+1} = exp(dA_last) P_c + S_c
//   y[m,p]   = exp(dA_m) sum_n f16(C^[m,n]) f16(P_c[p,n])                                  (term 1)
//            + sum_{k<=m} f16(CB[m,k] exp(dA_m - dA_k) dt_k) f16(x^[k,p])                  (term 2)
//            + x^[m,p] D, optional z gate, fp16 out
// Both contractions over the time index need x with time as the fastest-moving index, while memory has channels
// fastest.  A thread transposes 4x4 blocks on the way into LDS: four dword loads (sixteen lanes cover the 64
// bytes of a row), four 8-byte stores.  The rows of the transposed tile are kept in the order
//   slot(p) = 16 (p % 4) + p / 4
// so that the sixteen lanes of one store write sixteen neighbouring rows (all banks, instead of every fourth row)
// and an MFMA tile, sixteen neighbouring rows, holds the channels p = 4 i + tile (i = 0..15): a lane then owns
// four neighbouring channels of an output row, which leave as one 8-byte store without passing through LDS.
// int8 values enter as biased bytes u = q + 128 (one xor per dword): s q = fma(u, s, -128 s) exactly, with the
// byte-to-float conversion in a single instruction.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ v4f mfma16(v8h a, v8h b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ float ubyte_of(uint32_t w, int j) { return static_cast<float>((w >> (8 * j)) & 0xffu); }
constexpr uint32_t kBias = 0x80808080u;
__device__ __forceinline__ uint32_t word_of(const uint4& v, int d) { return d == 0 ? v.x : d == 1 ? v.y : d == 2 ? v.z : v.w; }
__device__ __forceinline__ float lane_of(const float4& v, int d) { return d == 0 ? v.x : d == 1 ? v.y : d == 2 ? v.z : v.w; }

// A thread's share of a chunk's x tile, steps 4 kb .. 4 kb + 3 of channels 16 pb .. 16 pb + 15 (four 16-byte loads,
// biased bytes), goes to the transposed fp16 tile: sixteen 8-byte stores, rows in slot order.
template <int XP>
__device__ __forceinline__ void stage_x_share(_Float16 (*xt)[XP], const uint4 (&xr)[4], const float* xs, int pb, int kb) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const float4 s4 = *reinterpret_cast<const float4*>(xs + 16 * pb + 4 * d);
        const uint32_t w0 = word_of(xr[0], d) ^ kBias, w1 = word_of(xr[1], d) ^ kBias, w2 = word_of(xr[2], d) ^ kBias, w3 = word_of(xr[3], d) ^ kBias;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const float sc = lane_of(s4, cc), nsc = -128.0f * sc;
            v4h v;
            v[0] = static_cast<_Float16>(__builtin_fmaf(ubyte_of(w0, cc), sc, nsc));
            v[1] = static_cast<_Float16>(__builtin_fmaf(ubyte_of(w1, cc), sc, nsc));
            v[2] = static_cast<_Float16>(__builtin_fmaf(ubyte_of(w2, cc), sc, nsc));
            v[3] = static_cast<_Float16>(__builtin_fmaf(ubyte_of(w3, cc), sc, nsc));
            *reinterpret_cast<v4h*>(&xt[cc * 16 + 4 * pb + d][kb * 4]) = v;          // row slot(16 pb + 4 d + cc)
        }
    }
}

// Workgroup L of a launch whose units (things that share operands through L2) should stay on one XCD: L -> XCD
// L % 8, position L / 8 there; `parts` consecutive positions are the parts of one (unit, head).
__device__ __forceinline__ void unit_head_part(int linear, int units, int hpg, int parts, int& unit, int& head_in_group, int& part) {
    if (units % 8 == 0) {
        const int xcd = linear % 8, pos = linear / 8;
        part = pos % parts;
        unit = (pos / parts / hpg) * 8 + xcd;
        head_in_group = (pos / parts) % hpg;
    } else {
        part = linear % parts;
        unit = linear / parts / hpg;
        head_in_group = (linear / parts) % hpg;
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 2, 3 and 6 (quamba/triton/quant_chunk_state.py:76-89, quant_state_passing.py:60-83, quant_ssm_states.py
// :43,119): a workgroup of four waves per (batch, head, 64 state columns) walks the chunks in order with its part
// of the running state P (64 x 64 of headdim x dstate, fp32) in registers; the fp32 chunk states never travel
// through memory.  A wave owns 16 columns n and all rows p.  Its B operand, f16((s_B q_B[k,n]) w_k) with the
// per-head weight w_k = exp(dA_last - dA_k) dt_k, is built in registers from the transposed int8 B tile in LDS
// (rows n of 4-byte-aligned pitch with an odd number of dwords: conflict-free for the transposing dword stores
// and for the operand reads); its A operand is the transposed x tile.  The tiles of chunk c+1 are fetched into
// registers while chunk c is multiplied.  The state entering chunk c >= 1 is stored as fp16, rows in slot order.
// ---------------------------------------------------------------------------------------------
template <int Q>
struct StateSmem {
    static constexpr int XP = Q + 8;        // halves per row of the transposed x tile
    static constexpr int BP = Q + 4;        // bytes per row of the transposed B tile
    __attribute__((aligned(16))) _Float16 xt[kP][XP];
    __attribute__((aligned(16))) int8_t b8[64][BP];
    __attribute__((aligned(16))) float w[Q];
    __attribute__((aligned(16))) float xs[kP];    // x scale per channel
    int32_t srow[kP];                             // the channel's row of the grouped state scales
};

template <int N, int Q>
__global__ __launch_bounds__(256, 3) void ssd_state_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws, __half* prev, const float* xs_ws,
                                                          const int32_t* srow_ws, int nc) {
    using S = StateSmem<Q>;
    extern __shared__ __attribute__((aligned(16))) unsigned char ssd_smem_raw[];
    S& sm = *reinterpret_cast<S*>(ssd_smem_raw);
    constexpr int kThreads = 256;
    constexpr int PARTS = N / 64;                                 // workgroups per (batch, head)
    static_assert(Q <= kThreads, "a thread stages at most one share of the chunk's tiles");

    const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);    // the same in every lane: kept in a scalar register
    // a head of 64 s channels runs as s heads of 64 that share the head's step sizes, decay and skip weight: H, h count
    // those; hp is the head itself and ch0 the first of its channels this workgroup covers
    const int split = p.headdim / kP;
    const int G = p.ngroups, H = p.nheads * split, L = p.seqlen;
    int unit, hig, part;
    unit_head_part(blockIdx.x, p.batch * G, H / G, PARTS, unit, hig, part);
    const int h = (unit % G) * (H / G) + hig;
    const int hp = h / split, ch0 = (h % split) * kP;
    const int b = unit / G;
    const int g = hp / (p.nheads / G);
    const bool grouped = p.nhead_groups > 0;
    const float sB = grouped ? p.B_scale[g] : p.B_scale[0];
    const float nsB = -128.0f * sB;
    const uint32_t xrow = static_cast<uint32_t>(H) * kP;          // bytes between steps of x
    const uint32_t brow = static_cast<uint32_t>(G) * N;           // bytes between steps of B
    const int64_t rows0 = (static_cast<int64_t>(b) * p.nheads + hp) * nc;
    // this thread's share of a chunk's tiles: steps 4 kb .. 4 kb + 3, sixteen columns from 16 pb (of x: channels; of
    // B: state columns of this workgroup's part)
    const int pb = tid % 4, kb = tid / 4;
    const bool mine = Q == 256 || tid < Q;
    const uint32_t voff_x = static_cast<uint32_t>(4 * kb) * xrow + 16 * pb, voff_b = static_cast<uint32_t>(4 * kb) * brow + 16 * pb;
    if (tid < kP) {
        sm.xs[tid] = xs_ws[hp * p.headdim + ch0 + tid];
        sm.srow[tid] = srow_ws[hp * p.headdim + ch0 + tid];
    }
    uint4 xr[4], br[4];
    float r_dt = 0.0f, r_dA = 0.0f, r_last = 0.0f;
    int valid_loaded = Q;                                         // steps of the chunk whose tiles are in xr / br
    // One path for whole and ragged chunks: rows past the end of the sequence read the last row (the loads stay inside
    // the tensors) and are zeroed when the chunk is staged.  With a second, ragged path beside it the compiler merges
    // the two sets of destination registers by copies right behind the loads, i.e. waits for them where they are issued.
    auto load_chunk = [&](int c) {
        const int t0 = c * Q;
        const int valid = min(Q, L - t0);
        valid_loaded = valid;
        // uniform row addresses plus one per-thread offset: the address arithmetic stays in scalar registers
        const int8_t* xsrc = p.x + (static_cast<int64_t>(b) * L + t0) * xrow + static_cast<int64_t>(h) * kP;
        const int8_t* bsrc = p.B + (static_cast<int64_t>(b) * L + t0) * brow + static_cast<int64_t>(g) * N + part * 64;
        if (mine) {
            const uint32_t last_x = static_cast<uint32_t>(valid - 1) * xrow + 16 * pb, last_b = static_cast<uint32_t>(valid - 1) * brow + 16 * pb;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                xr[r] = *reinterpret_cast<const uint4*>(xsrc + static_cast<uint64_t>(min(voff_x + static_cast<uint32_t>(r) * xrow, last_x)));
                br[r] = *reinterpret_cast<const uint4*>(bsrc + static_cast<uint64_t>(min(voff_b + static_cast<uint32_t>(r) * brow, last_b)));
            }
        }
        const float* dA_row = dA_ws + (rows0 + c) * Q;
        r_last = dA_row[Q - 1];
        if (Q == kThreads || tid < Q) {
            r_dt = dt_ws[(rows0 + c) * Q + tid];
            r_dA = dA_row[tid];
        }
    };
    auto stage_chunk = [&]() {
        if (mine) {
            if (valid_loaded < Q) {
                // ragged last chunk: steps past the end of the sequence count as zero
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (4 * kb + r >= valid_loaded) xr[r] = br[r] = make_uint4(0u, 0u, 0u, 0u);
                }
            }
            stage_x_share<S::XP>(sm.xt, xr, sm.xs, pb, kb);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                // 4x4 byte transpose: rows k (registers) x columns n (bytes) -> rows n x bytes k
                const uint32_t r0 = word_of(br[0], d) ^ kBias, r1 = word_of(br[1], d) ^ kBias, r2 = word_of(br[2], d) ^ kBias, r3 = word_of(br[3], d) ^ kBias;
                const uint32_t lo01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);   // r0.b0 r1.b0 r0.b1 r1.b1
                const uint32_t hi01 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);   // r0.b2 r1.b2 r0.b3 r1.b3
                const uint32_t lo23 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
                const uint32_t hi23 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
                const int n4 = 16 * pb + 4 * d;
                *reinterpret_cast<uint32_t*>(&sm.b8[n4 + 0][kb * 4]) = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
                *reinterpret_cast<uint32_t*>(&sm.b8[n4 + 1][kb * 4]) = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
                *reinterpret_cast<uint32_t*>(&sm.b8[n4 + 2][kb * 4]) = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
                *reinterpret_cast<uint32_t*>(&sm.b8[n4 + 3][kb * 4]) = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
            }
        }
        if (tid < Q) sm.w[tid] = fexp(r_last - r_dA) * r_dt;        // weight of step k in the chunk's state
    };

    // the running state: columns n = 64 part + 16 wave + lane % 16; tile j, register r: channel p = 4 (4 (lane / 16) + r) + j
    const int n_col = part * 64 + 16 * wave + l16;
    v4f run[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) run[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    load_chunk(0);
    __syncthreads();                                              // the table of x scales
    stage_chunk();
    float dA_last = r_last;                                       // of the chunk about to be multiplied
    __syncthreads();

    for (int c = 0; c < nc; ++c) {
        const bool more = c + 1 < nc;
        // in flight during the products.  Unconditional (the last chunk is requested once more and never staged): a
        // conditional request leaves the tile registers with two possible sources, which the compiler merges by
        // copies right behind the loads, i.e. by waiting for them where they are issued
        load_chunk(min(c + 1, nc - 1));
        __builtin_amdgcn_sched_barrier(0);                         // (the scheduler would sink the requests below the products)
        v4f accs[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) accs[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < Q / 32; ++ks) {
            const int k0 = 32 * ks + 8 * lq;
            const uint32_t b0 = *reinterpret_cast<const uint32_t*>(&sm.b8[16 * wave + l16][k0]);
            const uint32_t b1 = *reinterpret_cast<const uint32_t*>(&sm.b8[16 * wave + l16][k0 + 4]);
            const float4 w0 = *reinterpret_cast<const float4*>(&sm.w[k0]), w1 = *reinterpret_cast<const float4*>(&sm.w[k0 + 4]);
            v8h fx[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) fx[j] = *reinterpret_cast<const v8h*>(&sm.xt[j * 16 + l16][k0]);
            const float wk[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
            v8h bw;
#pragma unroll
            for (int e = 0; e < 8; ++e) bw[e] = static_cast<_Float16>(__builtin_fmaf(ubyte_of(e < 4 ? b0 : b1, e & 3), sB, nsB) * wk[e]);
#pragma unroll
            for (int j = 0; j < 4; ++j) accs[j] = mfma16(fx[j], bw, accs[j]);
        }
        // P <- exp(dA_last) P + S
        const float decay = fexp(dA_last);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) run[j][r] = decay * run[j][r] + accs[j][r];
        if (more) {
            // the state entering chunk c + 1, in fp16 as the reference keeps it, rows in slot order
            __half* pst = prev + (((static_cast<int64_t>(b) * nc + c + 1) * H + h) * kP) * N + n_col;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) pst[(j * 16 + 4 * lq + r) * N] = __float2half(run[j][r]);
        }
        __syncthreads();                                           // every wave has read this chunk's tiles
        if (more) {
            stage_chunk();
            dA_last = r_last;
        }
        __syncthreads();
    }

    // final state in the requested form
    if (p.final_states) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int pp = 4 * (4 * lq + r) + j;
                const int64_t fo = ((static_cast<int64_t>(b) * H + h) * kP + pp) * N + n_col;
                const float sv = run[j][r];
                if (p.final_state_is_fp32) {
                    static_cast<float*>(p.final_states)[fo] = sv;
                } else {
                    static_cast<int8_t*>(p.final_states)[fo] = ssd_quantize_state(p, sm.srow[pp], n_col, sv);
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 4 and 5 (quamba/triton/quant_bmm_chunk.py:60-66, quant_chunk_scan.py:96-171): a workgroup of eight waves
// per (batch, chunk, head).  A wave owns whole 16-row m-tiles with all 64 channels, a long and a short causal range
// each (with sixteen tiles: 15 - w and w), the long one first.
// C B^T never exists in memory: the chunk's B codes sit in LDS, a lane holds 32 codes of its row of C, and
// v_mfma_i32_16x16x64_i8 forms (C B^T)^T in 16 x 16 blocks - exact integers, times s_C s_B in fp32, the value
// the reference's bmm kernel stores.  A block comes out with a lane per row m and four consecutive steps k, which
// is how the next product wants its first operand: two blocks (steps 4 q .. 4 q + 3 and 16 + 4 q .. 16 + 4 q + 3
// of a 32-step piece, q = lane / 16) are the eight values of a lane, and the x operand is read from LDS in the
// same order (the order of the summation index is free as long as both operands agree).  The same codes of C,
// dequantised to fp16, are the first operand of term 1; a lane's codes are states 64 i + 16 q .. + 15, and the
// entering state is read in that order.  Below the diagonal the decay factors into exp(dA_m - R) (one exp per
// lane and piece) and exp(R - dA_k) dt_k (a table per workgroup) with R = dA at the last step of the piece, so
// that both exponents are <= 0; on the piece that holds the diagonal it is computed per element, in the
// reference's order.  After the prologue a wave reads global memory only for the bytes of the skip term and gate.
// With 128 states and chunks of 256 steps two workgroups fit a CU's LDS only if the entering state and the upper
// half of the B codes share their 16 KB: term 1 of both tiles runs first, then the B codes (held in registers
// since the prologue) take the state's place.
// ---------------------------------------------------------------------------------------------
template <int N, int Q>
struct ScanSmem {
    static constexpr bool ALIAS = N == 128 && Q == 256;
    static constexpr int XP = Q + 8;        // halves per row of the transposed x tile
    static constexpr int NCH = N / 8;       // 16-byte pieces per row of the entering state
    static constexpr int SWZ = (NCH < 16 ? NCH : 16) - 1;
    static constexpr int BSWZ = (N / 16 < 8 ? N / 16 : 8) - 1;
    static constexpr int BROWS = ALIAS ? Q / 2 : Q;
    __attribute__((aligned(16))) _Float16 xt[kP][XP];
    // rows without padding: piece c of row r sits at position c ^ (r & SWZ), so that the sixteen rows of an operand
    // read fall into different banks
    __attribute__((aligned(16))) _Float16 prev[kP][N];
    __attribute__((aligned(16))) int8_t bq[BROWS][N];   // B codes; 16-byte piece c of row k at position c ^ (k & BSWZ)
    __attribute__((aligned(16))) float dt[Q];
    __attribute__((aligned(16))) float dA[Q];
    __attribute__((aligned(16))) float gk[Q];   // exp(dA[end of the 32-step piece] - dA_k) dt_k
    __attribute__((aligned(16))) float xs[kP];  // x scale per channel
    __attribute__((aligned(16))) float Dv[kP];  // skip weight per channel
    __attribute__((aligned(16))) float gate[256];   // SiLU(z_scale code) of the gate's 256 codes, indexed by the code's byte
    static_assert(!ALIAS || sizeof(_Float16) * kP * N == static_cast<size_t>(Q / 2) * N, "the upper B rows take exactly the state's place");
    // row k of the B codes
    __device__ __forceinline__ int8_t* brow(int k) {
        if (ALIAS && k >= BROWS) return reinterpret_cast<int8_t*>(&prev[0][0]) + (k - BROWS) * N;
        return bq[k];
    }
};

constexpr int scan_waves_of(int Q) { return Q / 16 < 8 ? Q / 16 : 8; }

template <int N, int Q>
__global__ __launch_bounds__(64 * scan_waves_of(Q), 4) void ssd_chunk_scan_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws,
                                                                                const __half* prev, const float* xs_ws, int nc) {
    using S = ScanSmem<N, Q>;
    extern __shared__ __attribute__((aligned(16))) unsigned char ssd_smem_raw[];
    S& sm = *reinterpret_cast<S*>(ssd_smem_raw);
    constexpr int kWaves = scan_waves_of(Q);
    constexpr int kThreads = 64 * kWaves;
    constexpr int NMT = Q / 16;                                   // 16-row m-tiles of a chunk
    constexpr int TILES = NMT / kWaves;                           // per wave: 2 (Q 256), 1 (Q 128, 64)
    constexpr int PPC = kP * N / 8;                               // 16-byte pieces of the entering state
    constexpr int PB = PPC / kThreads;
    constexpr int BPC = Q * N / 16;                               // 16-byte pieces of the B codes
    constexpr int BB = BPC / kThreads;
    constexpr int BB_NOW = S::ALIAS ? BB / 2 : BB;                // pieces a thread writes in the prologue
    static_assert(Q <= kThreads, "a thread stages at most one share of the x tile");
    static_assert(PPC % kThreads == 0 && BPC % kThreads == 0 && (!S::ALIAS || BB % 2 == 0), "whole shares per thread");
    static_assert(TILES <= 2, "a long and a short tile per wave");

    const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);    // the same in every lane: kept in a scalar register
    // (H, h, hp, ch0 as in the state kernel: heads of 64 s channels run as s heads of 64)
    const int split = p.headdim / kP;
    const int G = p.ngroups, H = p.nheads * split, L = p.seqlen;
    // the heads of one (batch, chunk, ssd group) read the same B and C codes: they go to one XCD
    int unit, hig, part;
    unit_head_part(blockIdx.x, p.batch * nc * G, H / G, 1, unit, hig, part);
    const int h = (unit % G) * (H / G) + hig;
    const int hp = h / split, ch0 = (h % split) * kP;
    const int c = (unit / G) % nc;
    const int b = unit / (G * nc);
    const int g = hp / (p.nheads / G);
    const bool grouped = p.nhead_groups > 0;
    const float sC = grouped ? p.C_scale[g] : p.C_scale[0];
    const float cb_scale = sC * (grouped ? p.B_scale[g] : p.B_scale[0]);
    const int t0 = c * Q;
    const int lim = min(Q, L - t0);
    const uint32_t xrow = static_cast<uint32_t>(H) * kP;          // bytes between steps of x
    const uint32_t crow = static_cast<uint32_t>(G) * N;           // bytes between steps of B and C
    const int8_t* xbase = p.x + (static_cast<int64_t>(b) * L + t0) * xrow + static_cast<int64_t>(h) * kP;
    const int8_t* zbase = p.z + (static_cast<int64_t>(b) * L + t0) * xrow + static_cast<int64_t>(h) * kP;       // only read if p.z
    const int8_t* Bbase = p.B + (static_cast<int64_t>(b) * L + t0) * crow + static_cast<int64_t>(g) * N;
    const int8_t* Cbase = p.C + (static_cast<int64_t>(b) * L + t0) * crow + static_cast<int64_t>(g) * N;
    const float D_scale = p.D ? *p.D_scale : 0.0f;
    const float z_scale = p.z ? *p.z_scale : 0.0f;
    __half* out = static_cast<__half*>(p.out) + (static_cast<int64_t>(b) * L + t0) * xrow + static_cast<int64_t>(h) * kP;

    // tile s of this wave
    auto tile_of = [&](int s) { return (s & 1) == 0 ? NMT - 1 - 8 * (s / 2) - wave : 8 * ((TILES - 1 - s) / 2) + wave; };

    // codes of C of this lane's rows: states 64 i + 16 q .. + 15 (rows past the end of the sequence read the last
    // row; nothing of theirs is stored)
    v4i cq[TILES][N / 64];
    v4i r_b[BB];
    {
        // Prologue: every global read is issued before the first LDS write, so that the workgroup waits for memory
        // once.
        float r_dt = 0.0f, r_dA = 0.0f, r_end = 0.0f;
        if (tid < Q) {
            const int64_t row = ((static_cast<int64_t>(b) * p.nheads + hp) * nc + c) * Q;
            r_dt = dt_ws[row + tid];
            r_dA = dA_ws[row + tid];
            r_end = dA_ws[row + (tid | 31)];
        }
        // (the first chunk has no entering state: its slot of the workspace is read all the same and never used)
        v4i r_prev[PB];
        const __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * kP * N;
#pragma unroll
        for (int i = 0; i < PB; ++i) r_prev[i] = *reinterpret_cast<const v4i*>(pst + (tid + i * kThreads) * 8);
        // the chunk's B codes
#pragma unroll
        for (int i = 0; i < BB; ++i) {
            const int piece = tid + i * kThreads, k = piece / (N / 16), col = piece % (N / 16);
            r_b[i] = *reinterpret_cast<const v4i*>(Bbase + static_cast<uint32_t>(min(k, lim - 1)) * crow + 16 * col);
        }
#pragma unroll
        for (int s = 0; s < TILES; ++s) {
            const int8_t* cp = Cbase + static_cast<uint32_t>(min(tile_of(s) * 16 + l16, lim - 1)) * crow + 16 * lq;
#pragma unroll
            for (int i = 0; i < N / 64; ++i) cq[s][i] = *reinterpret_cast<const v4i*>(cp + 64 * i);
        }
        // (requested last: the compiler moves the loaded words into other registers right behind these loads, i.e.
        // waits for them here, and everything else is then already on its way)
        // this thread's share of the x tile: steps 4 kb .. 4 kb + 3, channels 16 pb .. 16 pb + 15
        const int pb = tid % 4, kb = tid / 4;
        const bool mine = Q == kThreads || tid < Q;
        // (one path for whole and ragged chunks: rows past the end of the sequence read the last row and are zeroed
        // when the tile is staged; with a second path beside it the compiler merges the two sets of destination
        // registers by copies right behind the loads and so waits for them before the requests below are issued)
        uint4 xr[4];
        if (mine) {
            const uint32_t last_x = static_cast<uint32_t>(lim - 1) * xrow + 16 * pb, voff_x = static_cast<uint32_t>(4 * kb) * xrow + 16 * pb;
#pragma unroll
            for (int r = 0; r < 4; ++r) xr[r] = *reinterpret_cast<const uint4*>(xbase + static_cast<uint64_t>(min(voff_x + static_cast<uint32_t>(r) * xrow, last_x)));
        }
        if (tid < kP) {
            sm.xs[tid] = xs_ws[hp * p.headdim + ch0 + tid];
            sm.Dv[tid] = !p.D ? 0.0f : D_scale * static_cast<float>(p.D_has_hdim ? p.D[hp * p.headdim + ch0 + tid] : p.D[hp]);
        }
        if (p.z) {
            // the gate has 256 possible values: evaluated once per workgroup, looked up per output
            for (int i = tid; i < 256; i += kThreads) {
                const float zv = z_scale * static_cast<float>(static_cast<int8_t>(i));
                sm.gate[i] = zv * __builtin_amdgcn_rcpf(1.0f + fexp(-zv));
            }
        }
        __syncthreads();                                           // the tables per channel (and every load above has landed)

        if (tid < Q) {
            sm.dt[tid] = r_dt;
            sm.dA[tid] = r_dA;
            sm.gk[tid] = fexp(r_end - r_dA) * r_dt;
        }
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const int piece = tid + i * kThreads, pr = piece / (N / 8), col = (piece % (N / 8)) * 8;
            *reinterpret_cast<v4i*>(&sm.prev[pr][col ^ ((pr & S::SWZ) * 8)]) = r_prev[i];
        }
#pragma unroll
        for (int i = 0; i < BB_NOW; ++i) {
            const int piece = tid + i * kThreads, k = piece / (N / 16), col = piece % (N / 16);
            *reinterpret_cast<v4i*>(sm.brow(k) + (col ^ (k & S::BSWZ)) * 16) = r_b[i];
        }
        if (mine) {
            if (lim < Q) {
                // ragged last chunk: steps past the end of the sequence count as zero
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (4 * kb + r >= lim) xr[r] = make_uint4(0u, 0u, 0u, 0u);
                }
            }
            stage_x_share<S::XP>(sm.xt, xr, sm.xs, pb, kb);
        }
    }
    __syncthreads();

    // term 1 of every tile of the wave: C^ (rows m) x entering state (rows p), zero for the first chunk
    v4f acc[TILES][4];
#pragma unroll
    for (int s = 0; s < TILES; ++s) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[s][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        if (c > 0) {
            const int m0 = tile_of(s) * 16;
#pragma unroll
            for (int ks = 0; ks < N / 32; ++ks) {
                const uint32_t w0 = static_cast<uint32_t>(cq[s][ks / 2][2 * (ks % 2)]), w1 = static_cast<uint32_t>(cq[s][ks / 2][2 * (ks % 2) + 1]);
                v8h cf;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    cf[e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(w0, e)));
                    cf[4 + e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(w1, e)));
                }
                const int n0 = 64 * (ks / 2) + 16 * lq + 8 * (ks % 2);     // the states of those eight codes
                v8h fs[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) fs[j] = *reinterpret_cast<const v8h*>(&sm.prev[j * 16 + l16][n0 ^ ((l16 & S::SWZ) * 8)]);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[s][j] = mfma16(cf, fs[j], acc[s][j]);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float em = fexp(sm.dA[m0 + 4 * lq + r]);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[s][j][r] *= em;
            }
        }
    }
    if constexpr (S::ALIAS) {
        __syncthreads();                                           // everyone is done with the entering state
#pragma unroll
        for (int i = BB_NOW; i < BB; ++i) {
            const int piece = tid + i * kThreads, k = piece / (N / 16), col = piece % (N / 16);
            *reinterpret_cast<v4i*>(sm.brow(k) + (col ^ (k & S::BSWZ)) * 16) = r_b[i];
        }
        __syncthreads();
    }

#pragma unroll
    for (int s = 0; s < TILES; ++s) {
        // the most pieces a tile in position s can have (position 0 holds the longest tiles)
        const int max_tile = (s & 1) == 0 ? NMT - 1 - 8 * (s / 2) : 8 * ((TILES - 1 - s) / 2) + kWaves - 1;
        const int max_nks = (max_tile + 2) / 2;
        const int mt = tile_of(s);
        const int m0 = mt * 16;
        const int nks = (mt + 2) / 2;                               // 32-step pieces that reach row m0 + 15; the last holds the diagonal
        const int m_row = m0 + l16;                                 // row of this lane's first operands
        const float dA_m = sm.dA[m_row];
        // skip-term operands of this lane's four output rows
        // (requested now, used in the epilogue: nothing there waits for memory)
        uint32_t xq[4], zq[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t at = static_cast<uint32_t>(min(m0 + 4 * lq + r, lim - 1)) * xrow + 4 * l16;
            xq[r] = *reinterpret_cast<const uint32_t*>(xbase + at);
            if (p.z) zq[r] = *reinterpret_cast<const uint32_t*>(zbase + at);
        }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (ks < max_nks && ks < nks) {
                // steps of this lane's eight values: ka .. ka + 3 and ka + 16 .. ka + 19
                const int ka = 32 * ks + 4 * lq;
                // (C B^T)^T for the two 16-step blocks of the piece
                v4i cbi[2];
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const int k = 32 * ks + 16 * blk + l16;
                    const int8_t* brow = sm.brow(32 * ks + 16 * blk) + l16 * N;
                    cbi[blk] = v4i{0, 0, 0, 0};
#pragma unroll
                    for (int i = 0; i < N / 64; ++i) {
                        const v4i bo = *reinterpret_cast<const v4i*>(brow + (((4 * i + lq) ^ (k & S::BSWZ)) * 16));
                        cbi[blk] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bo, cq[s][i], cbi[blk], 0, 0, 0);
                    }
                }
                v8h fx[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v4h x0 = *reinterpret_cast<const v4h*>(&sm.xt[j * 16 + l16][ka]);
                    const v4h x1 = *reinterpret_cast<const v4h*>(&sm.xt[j * 16 + l16][ka + 16]);
                    fx[j] = v8h{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                }
                float cv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) cv[e] = static_cast<float>(cbi[e / 4][e % 4]);
                float wv[8];
                if (ks + 1 < nks) {
                    const float4 g0 = *reinterpret_cast<const float4*>(&sm.gk[ka]), g1 = *reinterpret_cast<const float4*>(&sm.gk[ka + 16]);
                    const float gk[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
                    const float e_m = cb_scale * fexp(dA_m - sm.dA[32 * ks + 31]);      // the scale of C B^T rides with the row's decay
#pragma unroll
                    for (int e = 0; e < 8; ++e) wv[e] = cv[e] * (e_m * gk[e]);
                } else {
                    // the piece with the diagonal: steps after row m do not count
                    const float4 a0 = *reinterpret_cast<const float4*>(&sm.dA[ka]), a1 = *reinterpret_cast<const float4*>(&sm.dA[ka + 16]);
                    const float4 d0 = *reinterpret_cast<const float4*>(&sm.dt[ka]), d1 = *reinterpret_cast<const float4*>(&sm.dt[ka + 16]);
                    const float ak[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                    const float dk[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int k = ka + 16 * (e / 4) + e % 4;
                        wv[e] = ((k <= m_row ? cb_scale * cv[e] : 0.0f) * fexp(fminf(dA_m - ak[e], 0.0f))) * dk[e];
                    }
                }
                v8h fl;
#pragma unroll
                for (int e = 0; e < 8; ++e) fl[e] = static_cast<_Float16>(wv[e]);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[s][j] = mfma16(fl, fx[j], acc[s][j]);
            }
        }
        // Epilogue: acc[s][j][r] is row m0 + 4 (lane / 16) + r, channel 4 (lane % 16) + j
        const float4 xs4 = *reinterpret_cast<const float4*>(&sm.xs[4 * l16]), Dv4 = *reinterpret_cast<const float4*>(&sm.Dv[4 * l16]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + 4 * lq + r;
            if (m < lim) {
                float y[4] = {acc[s][0][r], acc[s][1][r], acc[s][2][r], acc[s][3][r]};
                if (p.D) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) y[j] += __builtin_fmaf(ubyte_of(xq[r] ^ kBias, j), lane_of(xs4, j), -128.0f * lane_of(xs4, j)) * lane_of(Dv4, j);
                }
                if (p.z) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) y[j] *= sm.gate[(zq[r] >> (8 * j)) & 0xffu];
                }
                v4h o;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = static_cast<_Float16>(y[j]);
                *reinterpret_cast<v4h*>(out + static_cast<uint32_t>(m) * xrow + 4 * l16) = o;
            }
        }
    }
}

int validate(const QaSsdParams* p) {
    if (!p) return QA_ERR_NULL;
    if (p->batch < 0 || p->seqlen < 0 || p->nheads < 1 || p->ngroups < 1 || p->nheads % p->ngroups != 0) return QA_ERR_SHAPE;
    if (p->batch > 0 && p->seqlen > 0) {                          // (no steps: the tensors may be null)
        if (!p->x || !p->dt || !p->A_log || !p->B || !p->C || !p->out) return QA_ERR_NULL;
        if (!p->x_scale || !p->A_log_scale || !p->B_scale || !p->C_scale) return QA_ERR_NULL;
        if (!p->dt_is_fp32 && !p->dt_scale) return QA_ERR_NULL;
        if ((p->D && !p->D_scale) || (p->z && !p->z_scale)) return QA_ERR_NULL;
        if (p->final_states && !p->final_state_is_fp32 && !p->state_scale) return QA_ERR_NULL;
        if (p->nhead_groups > 0 && (!p->x_head_group_range || !p->x_dim_group_range || p->ndim_groups < 1)) return QA_ERR_NULL;
    }
    // what the general kernels take; the matrix-core kernels cover a subset (ssd_fast_shape)
    if (p->headdim < 1 || p->headdim > 256 || p->dstate < 1 || p->dstate > 1024 || p->chunk_size < 1 || p->chunk_size > 1024) return QA_ERR_UNSUPPORTED;
    const int64_t nc = (static_cast<int64_t>(p->seqlen) + p->chunk_size - 1) / p->chunk_size;
    if (ssd_fast_shape(*p)) {
        // every launch is a one-dimensional grid: one workgroup per (batch, chunk, head) or per (batch, head, 64 states)
        const int64_t heads = static_cast<int64_t>(p->nheads) * (p->headdim / 64);       // heads of 64 channels
        if (static_cast<int64_t>(p->batch) * nc * heads > 0x7fffffffLL) return QA_ERR_SHAPE;
        if (static_cast<int64_t>(p->batch) * heads * (p->dstate / 64) > 0x7fffffffLL) return QA_ERR_SHAPE;
    } else {
        const int st = ssd_general_grid_check(*p);
        if (st != QA_OK) return st;
    }
    return QA_OK;
}

}  // namespace
}  // namespace qa

extern "C" int64_t qa_ssd_workspace_bytes(const QaSsdParams* p) {
    if (qa::validate(p) != QA_OK) return 0;
    return qa::ssd_workspace_layout(*p).total;
}

extern "C" int qa_ssd_chunk_scan_fwd(const QaSsdParams* p, void* stream_) {
    using namespace qa;
    const int st = validate(p);
    if (st != QA_OK) return st;
    if (p->batch == 0) return QA_OK;
    if (p->seqlen == 0) {
        // no steps: the state after them is the zero state the scan starts from
        const int64_t states = static_cast<int64_t>(p->batch) * p->nheads * p->headdim * p->dstate;
        return fill_zero(p->final_states, states * (p->final_state_is_fp32 ? 4 : 1), static_cast<hipStream_t>(stream_));
    }
    const SsdWorkspace ws = ssd_workspace_layout(*p);
    if (!p->workspace) return QA_ERR_NULL;
    if (p->workspace_bytes < ws.total || (reinterpret_cast<uintptr_t>(p->workspace) & 255u)) return QA_ERR_STRIDE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    uint8_t* base = static_cast<uint8_t*>(p->workspace);
    float* dt_ws = reinterpret_cast<float*>(base + ws.dt);
    float* dA_ws = reinterpret_cast<float*>(base + ws.dA);
    const int nc = (p->seqlen + p->chunk_size - 1) / p->chunk_size;
    const int64_t bch = static_cast<int64_t>(p->batch) * nc * p->nheads;

    __half* prev_ws = reinterpret_cast<__half*>(base + ws.prev);
    float* xs_ws = reinterpret_cast<float*>(base + ws.xs);
    int32_t* srow_ws = reinterpret_cast<int32_t*>(base + ws.srow);
    if (!ssd_fast_shape(*p)) {
        ssd_general_launch(*p, dt_ws, dA_ws, prev_ws, xs_ws, srow_ws, nc, stream);
        return check_launch();
    }
    hipLaunchKernelGGL(ssd_cumsum_kernel, dim3(static_cast<unsigned>((bch + 3) / 4)), dim3(256), 0, stream, *p, dt_ws,
                       dA_ws, xs_ws, srow_ws, nc);
    const int heads64 = p->nheads * (p->headdim / 64);          // the kernels see a head of 64 s channels as s heads of 64
    const dim3 hgrid(static_cast<unsigned>(p->batch * heads64 * (p->dstate / 64)));
    int status = QA_OK;
    // more LDS than a kernel gets by default: raise the limit (idempotent)
    auto lds_ok = [&](const void* kernel, size_t lds) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) == hipSuccess) return true;
        status = check_launch();
        if (status == QA_OK) status = QA_ERR_LAUNCH;
        return false;
    };
    auto launch = [&](auto state_kernel, size_t state_lds, auto scan_kernel, size_t scan_lds, int scan_threads) {
        if (!lds_ok(reinterpret_cast<const void*>(state_kernel), state_lds) || !lds_ok(reinterpret_cast<const void*>(scan_kernel), scan_lds)) return;
        hipLaunchKernelGGL(state_kernel, hgrid, dim3(256), state_lds, stream, *p, dt_ws, dA_ws, prev_ws, xs_ws, srow_ws, nc);
        hipLaunchKernelGGL(scan_kernel, dim3(static_cast<unsigned>(bch * (p->headdim / 64))), dim3(scan_threads), scan_lds, stream, *p, dt_ws, dA_ws, prev_ws, xs_ws, nc);
    };
#define QA_SSD_LAUNCH(N_, Q_) launch(ssd_state_kernel<N_, Q_>, sizeof(StateSmem<Q_>), ssd_chunk_scan_kernel<N_, Q_>, \
                                     sizeof(ScanSmem<N_, Q_>), 64 * scan_waves_of(Q_))
    if (p->dstate == 128) {
        if (p->chunk_size == 256) QA_SSD_LAUNCH(128, 256);
        else if (p->chunk_size == 128) QA_SSD_LAUNCH(128, 128);
        else QA_SSD_LAUNCH(128, 64);
    } else {
        if (p->chunk_size == 256) QA_SSD_LAUNCH(64, 256);
        else if (p->chunk_size == 128) QA_SSD_LAUNCH(64, 128);
        else QA_SSD_LAUNCH(64, 64);
    }
#undef QA_SSD_LAUNCH
    if (status != QA_OK) return status;
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// The same scan for callers that cannot allocate (code under HIP graph capture, serving loops and harnesses that
// forbid hipMalloc): the workspace is a fixed array in the device image instead of a caller's buffer.  Every GPU
// holds its own copy of the array at its own address, so the address is looked up once per device, with that
// device current, and kept.  In host code the array's name is only a handle for that lookup, never a pointer.
// ---------------------------------------------------------------------------------------------
namespace qa {
namespace {
constexpr int64_t kStaticScratchBytes = QA_SSD_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
}  // namespace
}  // namespace qa

static __device__ __align__(256) unsigned char scratch[qa::kStaticScratchBytes];

namespace qa {
namespace {
std::mutex g_scratch_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (null: the runtime refused the lookup).
void* static_scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr) return ptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (ptr) return ptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        set_last_hip_error(static_cast<int>(e));
        return nullptr;
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    return ptr;
}
}  // namespace
}  // namespace qa

extern "C" int qa_ssd_chunk_scan_fwd_noalloc(const QaSsdParams* p, void* stream_) {
    using namespace qa;
    const int st = validate(p);
    if (st != QA_OK) return st;
    if (p->batch == 0 || p->seqlen == 0) return qa_ssd_chunk_scan_fwd(p, stream_);      // (nothing needs a workspace)
    if (ssd_workspace_layout(*p).total > kStaticScratchBytes) return QA_ERR_SCRATCH;
    void* ptr = static_scratch_of_current_device();
    if (!ptr) return QA_ERR_LAUNCH;
    QaSsdParams q = *p;
    q.workspace = ptr;
    q.workspace_bytes = kStaticScratchBytes;
    return qa_ssd_chunk_scan_fwd(&q, stream_);
}
