// Mamba2 quantized SSD chunk scan (prefill) for gfx950.
//
// Stages and arithmetic follow the reference's Triton pipeline (quamba/triton/quant_ssd_combined.py
// :61-77, grouped :146-162); see each kernel for the file it restates.  fp16 operands, fp32
// accumulation, as there; the one pure int8 contraction (C B^T) runs on the int8 matrix cores.
//   cumsum      dt = clamp(softplus(s_dt q_dt + dt_bias)), dA_cs = within-chunk cumsum(dt * A)
//   cb          CB[m,k] = (s_C s_B) * sum_n q_C[m,n] q_B[k,n]                       (int8 MFMA, lower tiles)
//   state       S_c[p,n] = sum_k f16(x^[k,p] exp(dA_last - dA_k) dt_k) f16(B^[k,n])   (fp16 MFMA; the reference
//               rounds B^ times the weight instead, the difference is inside the fp16 tolerance)
//               P_0 = 0, P_{c+1} = exp(dA_last,c) P_c + S_c in registers; P_c stored in fp16; final state fp32 / int8
//   chunk_scan  y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) P_c[p,n] + sum_{k<=m} f16(CB[m,k] e^{dA_m-dA_k} dt_k) f16(x^[k,p])
//               + D x^[m,p], optional z gate, fp16 out                               (fp16 MFMA; C B^T is held
//               in fp16 and meets its decay factor in a packed fp16 multiply)
// Both fp16 contractions over the time index need x (and B) with time as the fastest-moving index,
// while memory has channels fastest; x tiles are transposed once on the way into LDS (4x4 blocks:
// four dword loads, four 8-byte LDS stores) and then read as 16-byte MFMA operands, B is packed in
// operand order once per ssd group.
#include <atomic>
#include <mutex>

#include "qa_common.hpp"

namespace qa {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kP = 64;          // head dimension this build supports
constexpr float kLog2e = 1.44269504088896341f;
// C B^T is kept in fp16 divided by 16 (exact), so that products of full-range int8 rows stay inside
// the fp16 range; the factor returns with the decay table.
constexpr float kCbShift = 0.0625f, kCbUnshift = 16.0f;

__device__ __forceinline__ float fexp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }
// orders a wave's own LDS writes before its later LDS reads (wave-private scratch needs no workgroup barrier)
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ int8_t byte_of(uint32_t w, int j) { return static_cast<int8_t>((w >> (8 * j)) & 0xffu); }

struct Ws {            // workspace sections (byte offsets), see qa_ssd_workspace_bytes
    int64_t dt, dA, cb, prev, final_f32, c16, bt16, total;
};

__host__ __device__ inline int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }

__host__ __device__ inline Ws ws_layout(const QaSsdParams& p) {
    const int64_t nc = (p.seqlen + p.chunk_size - 1) / p.chunk_size;
    const int64_t B = p.batch, H = p.nheads, Q = p.chunk_size, G = p.ngroups, P = p.headdim, N = p.dstate;
    Ws w;
    int64_t off = 0;
    w.dt = off; off = align256(off + B * H * nc * Q * 4);
    w.dA = off; off = align256(off + B * H * nc * Q * 4);
    w.cb = off; off = align256(off + B * nc * G * Q * Q * 2);
    w.prev = off; off = align256(off + B * nc * H * P * N * 2);
    w.final_f32 = off; off = align256(off + B * H * P * N * 4);
    w.c16 = off; off = align256(off + B * static_cast<int64_t>(p.seqlen) * G * N * 2);
    w.bt16 = off; off = align256(off + B * nc * G * N * Q * 2);
    w.total = off;
    return w;
}

// Workgroups are handed to the eight XCDs (each with an L2 of its own) in turn by linear index.  The
// heads of one ssd group share the packed B operand and neighbouring heads share the 128-byte lines
// of x, so in the state kernel the heads of one (batch, group) unit get linear indices that land on one
// XCD: index L -> XCD L % 8, position L / 8 there -> unit (L / 8) / hpg * 8 + L % 8, head (L / 8) % hpg
// of the group.  Needs a unit count that is a multiple of eight; otherwise the natural order
// (unit-major) is kept.  (The chunk scan measured the same either way and keeps the natural order.)
__device__ __forceinline__ void unit_and_head(int linear, int units, int hpg, int& unit, int& head_in_group) {
    if (units % 8 == 0) {
        const int xcd = linear % 8, pos = linear / 8;
        unit = (pos / hpg) * 8 + xcd;
        head_in_group = pos % hpg;
    } else {
        unit = linear / hpg;
        head_in_group = linear % hpg;
    }
}

// x scale of channel p of head h (per-tensor, or looked up from the cumulative group ranges,
// quamba/triton/quant_chunk_state.py:202-214)
__device__ __forceinline__ void group_of(const QaSsdParams& p, int h, int& g, int& hg) {
    const int hpg = p.nheads / p.ngroups;
    g = h / hpg;
    hg = 0;
    if (p.nhead_groups > 0) {
        for (int j = 0; j < p.nhead_groups; ++j) hg += (h % hpg) >= p.x_head_group_range[g * p.nhead_groups + j] ? 1 : 0;
        hg = min(hg, p.nhead_groups - 1);
    }
}
__device__ __forceinline__ int dim_group_of(const QaSsdParams& p, int g, int hg, int ch) {
    const int32_t* dr = p.x_dim_group_range + (g * p.nhead_groups + hg) * p.ndim_groups;
    int dg = 0;
    for (int j = 0; j < p.ndim_groups; ++j) dg += ch >= dr[j] ? 1 : 0;
    return min(dg, p.ndim_groups - 1);
}
__device__ __forceinline__ float x_scale_of(const QaSsdParams& p, int g, int hg, int ch) {
    if (p.nhead_groups == 0) return p.x_scale[0];
    return p.x_scale[(g * p.nhead_groups + hg) * p.ndim_groups + dim_group_of(p, g, hg, ch)];
}

// ---------------------------------------------------------------------------------------------
// Stage 1 (quamba/triton/quant_chunk_cumsum.py:56-70).  One wave per (batch, chunk, head): every
// lane processes chunk_size/64 consecutive steps, then an inclusive scan across the lanes.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ssd_cumsum_kernel(QaSsdParams p, float* dt_out, float* dA_out, int nc) {
    const int lane = threadIdx.x & 63;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (idx >= static_cast<int64_t>(p.batch) * nc * p.nheads) return;
    const int h = static_cast<int>(idx % p.nheads);
    const int c = static_cast<int>((idx / p.nheads) % nc);
    const int b = static_cast<int>(idx / (static_cast<int64_t>(p.nheads) * nc));
    const int Q = p.chunk_size, E = Q / 64;            // Q in {64, 128, 256}
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
// Stage 4 (quamba/triton/quant_bmm_chunk.py:60-66): one wave per 64x64 tile of CB, lower tiles only.
// Both operands are rows of dstate int8 values, i.e. already MFMA operands.  The diagonal tiles also
// write their C rows dequantised to fp16 (f16(s_C * q_C)): every head of the group multiplies those
// rows with its entering state in the chunk scan, which then reads them ready-made.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void ssd_cb_kernel(QaSsdParams p, __half* cb_out, __half* c16_out, int nc) {
    const int Q = p.chunk_size, N = p.dstate, G = p.ngroups;
    const int nt = Q / 64;
    // blockIdx.x enumerates lower-triangular tile pairs (mt >= kt)
    int mt = 0, rem = blockIdx.x;
    while (rem > mt) { rem -= mt + 1; ++mt; }
    const int kt = rem;
    if (mt >= nt) return;
    const int bcg = blockIdx.y;
    const int g = bcg % G, c = (bcg / G) % nc, b = bcg / (G * nc);
    const int lane = threadIdx.x, frow = lane & 31, fhalf = lane >> 5;
    const int t0 = c * Q;
    const int lim = min(Q, p.seqlen - t0);
    const float sC = p.nhead_groups > 0 ? p.C_scale[g] : p.C_scale[0];
    const float scale = sC * (p.nhead_groups > 0 ? p.B_scale[g] : p.B_scale[0]);

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    // every operand piece of the tile pair is requested before the first product: one memory round trip
    constexpr int KSMAX = 4;                                  // dstate 128
    const int nks = N / 32;
    v4i fc[KSMAX][2], fb[KSMAX][2];
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = mt * 64 + i * 32 + frow, k = kt * 64 + i * 32 + frow;
            const bool on = ks < nks;
            fc[ks][i] = (on && m < lim) ? *reinterpret_cast<const v4i*>(p.C + ((static_cast<int64_t>(b) * p.seqlen + t0 + m) * G + g) * N + ks * 32 + fhalf * 16)
                                        : v4i{0, 0, 0, 0};
            fb[ks][i] = (on && k < lim) ? *reinterpret_cast<const v4i*>(p.B + ((static_cast<int64_t>(b) * p.seqlen + t0 + k) * G + g) * N + ks * 32 + fhalf * 16)
                                        : v4i{0, 0, 0, 0};
        }
    }
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
        if (ks >= nks) break;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = mt * 64 + i * 32 + frow;
            if (mt == kt && m < lim) {
                v8h lo, hi;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    lo[e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(static_cast<uint32_t>(fc[ks][i][e >> 2]), e & 3)));
                    hi[e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(static_cast<uint32_t>(fc[ks][i][2 + (e >> 2)]), e & 3)));
                }
                __half* dst = c16_out + ((static_cast<int64_t>(b) * p.seqlen + t0 + m) * G + g) * N + ks * 32 + fhalf * 16;
                *reinterpret_cast<v8h*>(dst) = lo;
                *reinterpret_cast<v8h*>(dst + 8) = hi;
            }
        }
        // B rows as the first operand: the products come out with a lane per row m of C B^T and four
        // consecutive columns k per register group, which leave as 8-byte pieces
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks][j], fc[ks][i], acc[i][j], 0, 0, 0);
    }
    // acc[i][j]: lane holds row m = mt*64 + i*32 + (lane & 31), register r column k = kt*64 + j*32 + 8*(r/4) + 4*(lane/32) + r%4
    __half* tile = cb_out + ((static_cast<int64_t>(b) * nc + c) * G + g) * Q * Q;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = mt * 64 + i * 32 + frow;
                const int k = kt * 64 + j * 32 + 8 * q + 4 * fhalf;
                v4h o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = static_cast<_Float16>((scale * static_cast<float>(acc[i][j][4 * q + e])) * kCbShift);
                *reinterpret_cast<v4h*>(tile + static_cast<int64_t>(m) * Q + k) = o;
            }
}

// ---------------------------------------------------------------------------------------------
// B operand of the chunk-state product, packed once per (batch, chunk, ssd group) for every head of
// the group: f16(s_B q_B[k, n]) stored fragment-major, so that a wave's 16-byte-per-lane operand of
// n-tile nt and k-step ks is one contiguous kilobyte:
//   element (n, k) -> (((n/32) * (Q/16) + k/16) * 64 + ((k%16)/8) * 32 + n%32) * 8 + k%8
// One workgroup per (batch, chunk, group, n-tile); the 32 columns of the tile pass through LDS.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ssd_bpack_kernel(QaSsdParams p, __half* bt16, int nc) {
    constexpr int QMAX = 256, PITCH = 36;
    __shared__ __attribute__((aligned(16))) int8_t s_b[QMAX * PITCH];
    const int Q = p.chunk_size, N = p.dstate, G = p.ngroups, NT = N / 32;
    const int nt = blockIdx.x % NT;
    const int bcg = blockIdx.x / NT;
    const int g = bcg % G, c = (bcg / G) % nc, b = bcg / (G * nc);
    const int tid = threadIdx.x;
    const int t0 = c * Q;
    const int lim = min(Q, p.seqlen - t0);
    const float sB = p.nhead_groups > 0 ? p.B_scale[g] : p.B_scale[0];
    // rows k of the tile: 32 bytes each, two 16-byte pieces
    for (int piece = tid; piece < Q * 2; piece += 256) {
        const int k = piece >> 1, half = piece & 1;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (k < lim) v = *reinterpret_cast<const uint4*>(p.B + ((static_cast<int64_t>(b) * p.seqlen + t0 + k) * G + g) * N + nt * 32 + half * 16);
        uint32_t* dst = reinterpret_cast<uint32_t*>(s_b + k * PITCH + half * 16);
        dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    }
    __syncthreads();
    __half* out = bt16 + (static_cast<int64_t>(bcg) * NT + nt) * (Q / 16) * 64 * 8;
    for (int piece = tid; piece < (Q / 16) * 64; piece += 256) {
        const int ks = piece >> 6, lane = piece & 63, frow = lane & 31, fhalf = lane >> 5;
        v8h o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = static_cast<_Float16>(sB * static_cast<float>(s_b[(ks * 16 + fhalf * 8 + e) * PITCH + frow]));
        *reinterpret_cast<v8h*>(out + static_cast<int64_t>(piece) * 8) = o;
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 2, 3 and 6 in one pass (quamba/triton/quant_chunk_state.py:76-89, quant_state_passing.py
// :60-83, quant_ssm_states.py:43,119): one workgroup per (batch, head) walks the chunks in order and
// keeps the running state P (headdim x dstate, fp32) in registers, in the layout of the MFMA
// accumulators:
//   S_c[p,n] = sum_k f16(x^[k,p] w_k) f16(B^[k,n]),  w_k = exp(dA_last - dA_k) dt_k
//   store f16(P) as the state entering chunk c;  P = exp(dA_last) P + S_c
// The per-head weight w_k is applied to x (64 columns) rather than to B (dstate columns), so the B
// operand is the same for every head of a group and comes ready-made from ssd_bpack_kernel; the
// fp32 chunk states never travel through memory.  The x tile of chunk c+1 is fetched into registers
// before the products of chunk c are issued.
// Wave w owns n-tile w and both p-tiles (dstate 128) or n-tile w&1 and p-tile w>>1 (dstate 64).
// ---------------------------------------------------------------------------------------------
template <int N, int Q>
__global__ __launch_bounds__(256, 2) void ssd_state_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws,
                                                        const __half* bt16, __half* prev, float* final_ws, int nc) {
    constexpr int PITCH = Q + 8, NT = N / 32, PTW = NT == 4 ? 2 : 1, nks = Q / 16;
    constexpr int XB = (Q / 4) * (kP / 4) / 256;               // 4x4 blocks of the x tile per thread
    __shared__ __attribute__((aligned(16))) _Float16 s_xt[kP * PITCH];
    __shared__ __attribute__((aligned(16))) float s_w[2][Q];
    __shared__ float s_xs[kP];
    constexpr int kPatchPitch = 40;                            // halves; rows stay 16-byte aligned
    __shared__ __attribute__((aligned(16))) _Float16 s_patch[4 * 32 * kPatchPitch];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, frow = lane & 31, fhalf = lane >> 5;
    int unit, hig;
    unit_and_head(blockIdx.x, p.batch * p.ngroups, p.nheads / p.ngroups, unit, hig);
    const int h = (unit % p.ngroups) * (p.nheads / p.ngroups) + hig;
    const int b = unit / p.ngroups;
    const int G = p.ngroups, H = p.nheads;
    int g, hg;
    group_of(p, h, g, hg);
    if (tid < kP) s_xs[tid] = x_scale_of(p, g, hg, tid);
    const int ntile = NT == 4 ? wave : (wave & 1);
    const int pt0 = NT == 4 ? 0 : (wave >> 1);
    const int64_t row_stride = static_cast<int64_t>(H) * kP;
    const int64_t rows0 = (static_cast<int64_t>(b) * H + h) * nc;

    uint32_t xr[XB][4];
    auto load_x = [&](int c) {
        const int t0 = c * Q;
        const int valid = min(Q, p.seqlen - t0);
        const int8_t* src = p.x + ((static_cast<int64_t>(b) * p.seqlen + t0) * H + h) * kP;
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int id = tid + i * 256, kb = id / (kP / 4), cb = id % (kP / 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int k = kb * 4 + r;
                // rows past the end of the sequence read the last valid row and are zeroed (no branch)
                const uint32_t v = *reinterpret_cast<const uint32_t*>(src + min(k, valid - 1) * row_stride + cb * 4);
                xr[i][r] = k < valid ? v : 0u;
            }
        }
    };
    // s_w[c & 1][k] = exp(dA_last - dA_k) dt_k, in two halves so that the loads are issued an MFMA
    // phase before their values are needed
    float w_dt = 0.0f, w_dA = 0.0f, w_last = 0.0f;
    auto weights_load = [&](int c) {
        const float* dt_row = dt_ws + (rows0 + c) * Q;
        const float* dA_row = dA_ws + (rows0 + c) * Q;
        w_last = dA_row[Q - 1];
        if (Q == 256 || tid < Q) {
            w_dt = dt_row[tid];
            w_dA = dA_row[tid];
        }
    };
    auto weights_store = [&](int c) {
        if (Q == 256 || tid < Q) s_w[c & 1][tid] = fexp(w_last - w_dA) * w_dt;
    };
    auto store_x = [&](int c) {
        const float* w = s_w[c & 1];
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int id = tid + i * 256, kb = id / (kP / 4), cb = id % (kP / 4);
            const float4 wk = *reinterpret_cast<const float4*>(w + kb * 4);
            const float wr[4] = {wk.x, wk.y, wk.z, wk.w};
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const float cs = s_xs[cb * 4 + cc];
                v4h o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = static_cast<_Float16>((cs * static_cast<float>(byte_of(xr[i][r], cc))) * wr[r]);
                *reinterpret_cast<v4h*>(s_xt + (cb * 4 + cc) * PITCH + kb * 4) = o;
            }
        }
    };
    v8h fb[nks];
    auto load_b = [&](int c) {
        const __half* src = bt16 + (((static_cast<int64_t>(b) * nc + c) * G + g) * NT + ntile) * nks * 512 + lane * 8;
#pragma unroll
        for (int ks = 0; ks < nks; ++ks) fb[ks] = *reinterpret_cast<const v8h*>(src + ks * 512);
    };

    v16f run[PTW], acc[PTW];
#pragma unroll
    for (int j = 0; j < PTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) { run[j][r] = 0.0f; acc[j][r] = 0.0f; }

    load_x(0);
    weights_load(0);
    load_b(0);
    weights_store(0);
    float dA_last = w_last;                                    // of the chunk being multiplied
    __syncthreads();                                           // s_xs, s_w[0]
    store_x(0);
    __syncthreads();

    for (int c = 0; c < nc; ++c) {
        const bool more = c + 1 < nc;
        if (more) {
            weights_load(c + 1);                               // requests return in order: the one needed first goes first
            load_x(c + 1);
        }
#pragma unroll
        for (int ks = 0; ks < nks; ++ks) {
#pragma unroll
            for (int j = 0; j < PTW; ++j) {
                const v8h fx = *reinterpret_cast<const v8h*>(s_xt + ((pt0 + j) * 32 + frow) * PITCH + ks * 16 + fhalf * 8);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx, fb[ks], acc[j], 0, 0, 0);
            }
        }
        if (more) load_b(c + 1);                               // in flight during the update and the staging below
        // the state entering chunk c, then the recurrence.  Lane holds column n = ntile*32 + lane%32 and,
        // in register r, row p = pt*32 + 8*(r/4) + 4*(lane/32) + r%4.
        // The 32 x 32 tile passes through a wave-private LDS patch so that it leaves as 16-byte pieces.
        const float decay = fexp(dA_last);
        __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * kP * N + ntile * 32;
        _Float16* patch = s_patch + wave * (32 * kPatchPitch);
#pragma unroll
        for (int j = 0; j < PTW; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                patch[(8 * (r / 4) + 4 * fhalf + (r % 4)) * kPatchPitch + frow] = static_cast<_Float16>(run[j][r]);
                run[j][r] = decay * run[j][r] + acc[j][r];
                acc[j][r] = 0.0f;
            }
            wave_sync();
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int row = q * 16 + (lane >> 2), piece = lane & 3;
                const uint4 v = *reinterpret_cast<const uint4*>(patch + row * kPatchPitch + piece * 8);
                *reinterpret_cast<uint4*>(pst + ((pt0 + j) * 32 + row) * N + piece * 8) = v;
            }
            wave_sync();
        }
        if (more) {
            weights_store(c + 1);
            dA_last = w_last;
        }
        __syncthreads();                                       // every wave is done with this chunk's x tile; s_w written
        if (more) store_x(c + 1);
        __syncthreads();
    }

    // final state: fp32 copy for the caller's workspace, and the requested output form
#pragma unroll
    for (int j = 0; j < PTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int pp = (pt0 + j) * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
            const int n = ntile * 32 + frow;
            const int64_t fo = ((static_cast<int64_t>(b) * H + h) * kP + pp) * N + n;
            const float sv = run[j][r];
            if (final_ws) final_ws[fo] = sv;
            if (p.final_states) {
                if (p.final_state_is_fp32) {
                    static_cast<float*>(p.final_states)[fo] = sv;
                } else {
                    float sc, K;
                    if (p.nhead_groups > 0) {
                        const int dg = dim_group_of(p, g, hg, pp);
                        sc = p.state_scale[((g * p.nhead_groups + hg) * p.ndim_groups + dg) * N + n];
                        K = 1e6f;
                    } else {
                        sc = p.state_scale[0];
                        K = 1e2f;
                    }
                    const float s16 = __half2float(__float2half(sv));      // the reference hands fp16 states to the quantiser
                    static_cast<int8_t*>(p.final_states)[fo] = sat8_rne((s16 * K) / (sc * K));
                }
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Stage 5 (quamba/triton/quant_chunk_scan.py:96-171): one workgroup per (batch, chunk, head), four
// waves; each wave owns whole 32-row m-tiles (paired small/large so the causal work balances).
// Everything a tile reads from global memory - its C rows, its rows of C B^T (fp16, all k-steps of the
// causal range) and the x / z bytes of the epilogue - is requested at the top of the tile, so the
// memory latency is paid once per tile instead of once per k-step.
// ---------------------------------------------------------------------------------------------
template <int N, int Q>
__global__ __launch_bounds__(256, 2) void ssd_chunk_scan_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws,
                                                                const __half* cb_ws, const __half* prev, const __half* c16, int nc) {
    constexpr int WAVES = 4, PITCH = Q + 8, PPITCH = N + 8, kThreads = 64 * WAVES;
    constexpr int kScratch = 512;      // floats per wave: the decay table (Q halves) or an 8 x 64 piece of the output tile
    constexpr int NMT = Q / 32, PER_WAVE = NMT / WAVES > 0 ? NMT / WAVES : 1, KSMAX = Q / 16;
    __shared__ __attribute__((aligned(16))) _Float16 s_xt[kP * PITCH];
    __shared__ __attribute__((aligned(16))) _Float16 s_prev[kP * PPITCH];     // entering state, rows p
    __shared__ __attribute__((aligned(16))) float s_dt[Q];
    __shared__ __attribute__((aligned(16))) float s_dA[Q];
    __shared__ __attribute__((aligned(16))) float s_g[WAVES * kScratch];
    __shared__ float s_xs[kP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, frow = lane & 31, fhalf = lane >> 5;
    const int h = blockIdx.x % p.nheads;
    const int c = (blockIdx.x / p.nheads) % nc;
    const int b = blockIdx.x / (p.nheads * nc);
    const int G = p.ngroups, H = p.nheads;
    int g, hg;
    group_of(p, h, g, hg);
    const int t0 = c * Q;
    const int lim = min(Q, p.seqlen - t0);
    const int64_t row_base = (static_cast<int64_t>(b) * H + h) * nc + c;
    const __half* cb = cb_ws + ((static_cast<int64_t>(b) * nc + c) * G + g) * Q * Q;
    const int64_t row_stride = static_cast<int64_t>(H) * kP;
    const int erow = lane >> 3, ecol = (lane & 7) * 8;       // epilogue: row within a piece of 8, first of 8 columns
    const int64_t tile_base = (static_cast<int64_t>(b) * p.seqlen + t0) * row_stride + static_cast<int64_t>(h) * kP + ecol;

    // Per-tile operands that come from global memory: this lane's pieces of its C row (term 1), of its
    // row of C B^T (term 2, every k-step of the causal range) and the x / z bytes of the epilogue.  They
    // are requested one tile ahead: the first tile's together with the prologue's reads, the next
    // tile's piece by piece as the current tile lets go of the registers.
    // tile order 0, NMT-1, 1, NMT-2, ...: wave w takes entries w*PER_WAVE + s
    auto tile_of = [&](int s) {
        const int entry = wave * PER_WAVE + s;
        return (entry & 1) ? NMT - 1 - (entry >> 1) : (entry >> 1);
    };
    v8h c_frag[N / 16], cbf[KSMAX];
    uint2 xq[4], zq[4];
    auto c_ptr = [&](int mt, int ks) {
        return c16 + ((static_cast<int64_t>(b) * p.seqlen + t0 + min(mt * 32 + frow, lim - 1)) * G + g) * N + ks * 16 + fhalf * 8;
    };
    auto cb_ptr = [&](int mt, int ks) { return cb + static_cast<int64_t>(mt * 32 + frow) * Q + fhalf * 8 + ks * 16; };
    auto load_xz = [&](int mt, int q) {
        const int64_t at = tile_base + min(mt * 32 + 8 * q + erow, lim - 1) * row_stride;
        xq[q] = p.D ? *reinterpret_cast<const uint2*>(p.x + at) : make_uint2(0u, 0u);
        zq[q] = p.z ? *reinterpret_cast<const uint2*>(p.z + at) : make_uint2(0u, 0u);
    };
    // skip-term and gate parameters: requested with everything else, used in the epilogue
    const float D_scale = p.D ? *p.D_scale : 0.0f;
    const float z_scale = p.z ? *p.z_scale : 0.0f;
    int8_t e_Dq[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) e_Dq[e] = p.D ? p.D[p.D_has_hdim ? h * kP + ecol + e : h] : int8_t(0);
    if (wave * PER_WAVE < NMT) {
        const int mt = tile_of(0);
#pragma unroll
        for (int ks = 0; ks < N / 16; ++ks) c_frag[ks] = *reinterpret_cast<const v8h*>(c_ptr(mt, ks));
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks)
            if (ks < 2 * (mt + 1)) cbf[ks] = *reinterpret_cast<const v8h*>(cb_ptr(mt, ks));
#pragma unroll
        for (int q = 0; q < 4; ++q) load_xz(mt, q);
    }
    {
        // Prologue: every global read is issued before the first LDS write, so that the workgroup waits
        // for memory once.  x is transposed on the way (4x4 blocks: four dword loads, four 8-byte stores).
        static_assert(Q <= kThreads, "one step per thread");
        constexpr int XB = (Q / 4) * (kP / 4) / kThreads, PB = kP * N / 8 / kThreads;
        float r_dt = 0.0f, r_dA = 0.0f;
        if (Q == kThreads || tid < Q) {
            r_dt = dt_ws[row_base * Q + tid];
            r_dA = dA_ws[row_base * Q + tid];
        }
        const __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * kP * N;
        uint4 r_prev[PB];
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const int piece = tid + i * kThreads, pr = piece / (N / 8), col = (piece % (N / 8)) * 8;
            r_prev[i] = *reinterpret_cast<const uint4*>(pst + pr * N + col);
        }
        const int8_t* xsrc = p.x + ((static_cast<int64_t>(b) * p.seqlen + t0) * H + h) * kP;
        const int64_t xstride = static_cast<int64_t>(H) * kP;
        const int cb4 = tid % (kP / 4);                      // the same four columns in every block of this thread
        uint32_t xr[XB][4];
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int kb = (tid + i * kThreads) / (kP / 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int k = kb * 4 + r;
                const uint32_t v = *reinterpret_cast<const uint32_t*>(xsrc + min(k, lim - 1) * xstride + cb4 * 4);
                xr[i][r] = k < lim ? v : 0u;
            }
        }
        float cs[4];
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) cs[cc] = x_scale_of(p, g, hg, cb4 * 4 + cc);
        if (tid < kP) s_xs[tid] = x_scale_of(p, g, hg, tid);

        if (Q == kThreads || tid < Q) {
            s_dt[tid] = r_dt;
            s_dA[tid] = r_dA;
        }
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const int piece = tid + i * kThreads, pr = piece / (N / 8), col = (piece % (N / 8)) * 8;
            *reinterpret_cast<uint4*>(s_prev + pr * PPITCH + col) = r_prev[i];
        }
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int kb = (tid + i * kThreads) / (kP / 4);
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                v4h o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = static_cast<_Float16>(cs[cc] * static_cast<float>(byte_of(xr[i][r], cc)));
                *reinterpret_cast<v4h*>(s_xt + (cb4 * 4 + cc) * PITCH + kb * 4) = o;
            }
        }
    }
    __syncthreads();

    __half* out = static_cast<__half*>(p.out);
    float e_Dv[8];                                           // D of the eight columns this lane writes
#pragma unroll
    for (int e = 0; e < 8; ++e) e_Dv[e] = D_scale * static_cast<float>(e_Dq[e]);

#pragma unroll
    for (int s = 0; s < PER_WAVE; ++s) {
        if (wave * PER_WAVE + s >= NMT) break;
        const int mt = tile_of(s);
        const bool has_next = s + 1 < PER_WAVE;
        const int mt_next = has_next ? tile_of(s + 1) : 0;
        const int nks_next = has_next ? 2 * (mt_next + 1) : 0;
        const int m_lane = mt * 32 + frow;                 // row of this lane's A operands
        const int nks = 2 * (mt + 1);                      // k-steps of the causal range
        const int n_off = 2 * mt;                          // of which entirely before the tile
        v16f acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

        // Decay factors.  The cumulative dA decreases along the chunk, so with ref = dA at the first row
        // of this m-tile, exp(dA_m - dA_k) = exp(dA_m - ref) * exp(ref - dA_k) for every k before the
        // tile, both factors <= 1.  The k factor (times dt_k, times the power of two that C B^T was
        // stored without) is tabulated once per tile by the wave, in fp16; the row factor is applied to
        // the accumulator after the off-diagonal k-steps, together with term 1 (whose decay exp(dA_m) =
        // exp(ref) * exp(dA_m - ref)).  Only the two diagonal k-steps evaluate the decay per element.
        // acc = E_m * (exp(ref) * T1 + sum_{k < m0} (CB * G_k) x_k) + diagonal.
        const int m0 = mt * 32;
        const float ref = s_dA[m0];
        _Float16* g_tab = reinterpret_cast<_Float16*>(s_g + wave * kScratch);
        for (int k = lane; k < m0; k += 64) g_tab[k] = static_cast<_Float16>((fexp(ref - s_dA[k]) * s_dt[k]) * kCbUnshift);
        wave_sync();

        // term 1: C^ (rows m, dstate contiguous) x entering state (rows p, dstate contiguous, staged in LDS)
        const bool row_ok = m_lane < lim;
#pragma unroll
        for (int ks = 0; ks < N / 16; ++ks) {
            v8h fc = c_frag[ks];
            if (has_next) c_frag[ks] = *reinterpret_cast<const v8h*>(c_ptr(mt_next, ks));
            if (!row_ok) {
#pragma unroll
                for (int e = 0; e < 8; ++e) fc[e] = static_cast<_Float16>(0.0f);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const v8h fs = *reinterpret_cast<const v8h*>(s_prev + (j * 32 + frow) * PPITCH + ks * 16 + fhalf * 8);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fc, fs, acc[j], 0, 0, 0);
            }
        }
        const float e_ref = fexp(ref);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            acc[0][r] *= e_ref;
            acc[1][r] *= e_ref;
        }
        // term 2.  The LDS operands of k-step ks+1 (decay table piece, two x fragments) are requested before
        // the products of k-step ks; the addresses are valid for every ks, so the requests need no condition.
        v8h gh_n = *reinterpret_cast<const v8h*>(g_tab + fhalf * 8);
        v8h fx_n[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) fx_n[j] = *reinterpret_cast<const v8h*>(s_xt + (j * 32 + frow) * PITCH + fhalf * 8);
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks) {
            const v8h gh = gh_n;
            const v8h fx_c[2] = {fx_n[0], fx_n[1]};
            if (ks + 1 < KSMAX) {
                const int k1 = (ks + 1) * 16 + fhalf * 8;
                gh_n = *reinterpret_cast<const v8h*>(g_tab + k1);
#pragma unroll
                for (int j = 0; j < 2; ++j) fx_n[j] = *reinterpret_cast<const v8h*>(s_xt + (j * 32 + frow) * PITCH + k1);
            }
            if (ks < nks) {
                const int k0 = ks * 16 + fhalf * 8;
                v8h fl;
                if (ks < n_off) {
                    fl = cbf[ks] * gh;
                } else {
                    if (ks == n_off) {
                        // leaving the off-diagonal part: apply the row factors once
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float em = fexp(s_dA[m0 + 8 * (r / 4) + 4 * fhalf + (r % 4)] - ref);
                            acc[0][r] *= em;
                            acc[1][r] *= em;
                        }
                    }
                    const float dA_m = s_dA[m_lane];
                    const float4 dA0 = *reinterpret_cast<const float4*>(s_dA + k0), dA1 = *reinterpret_cast<const float4*>(s_dA + k0 + 4);
                    const float4 dt0 = *reinterpret_cast<const float4*>(s_dt + k0), dt1 = *reinterpret_cast<const float4*>(s_dt + k0 + 4);
                    const float dAk[8] = {dA0.x, dA0.y, dA0.z, dA0.w, dA1.x, dA1.y, dA1.z, dA1.w};
                    const float dtk[8] = {dt0.x, dt0.y, dt0.z, dt0.w, dt1.x, dt1.y, dt1.z, dt1.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int k = k0 + e;
                        const float cbv = static_cast<float>(cbf[ks][e]) * kCbUnshift;
                        const float wv = (cbv * fexp(dA_m - dAk[e])) * dtk[e];
                        fl[e] = static_cast<_Float16>(k <= m_lane ? wv : 0.0f);
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fl, fx_c[j], acc[j], 0, 0, 0);
            }
            if (ks < nks_next) cbf[ks] = *reinterpret_cast<const v8h*>(cb_ptr(mt_next, ks));
        }
        wave_sync();                                    // the table is done with: its space now carries the output tile
        // Epilogue.  In the accumulators a lane holds one column p and 16 rows; memory wants rows of 64
        // contiguous columns.  The tile passes through the wave's scratch eight rows at a time (registers
        // 4q..4q+3 of both accumulators are rows 8q + 4*(lane/32) + 0..3), after which lane l holds row
        // l/8 and the eight columns 8*(l%8)..+7: the skip term and the gate use the 8 bytes fetched at
        // the top of the tile, the output is one 16-byte store.
        float* o_tab = s_g + wave * kScratch;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) o_tab[(4 * fhalf + t) * 64 + j * 32 + frow] = acc[j][4 * q + t];
            wave_sync();
            const int m = mt * 32 + 8 * q + erow;
            const float4 y0 = *reinterpret_cast<const float4*>(o_tab + erow * 64 + ecol);
            const float4 y1 = *reinterpret_cast<const float4*>(o_tab + erow * 64 + ecol + 4);
            wave_sync();                                // the next piece overwrites the scratch
            const uint2 xb = xq[q], zb = zq[q];
            if (has_next) load_xz(mt_next, q);
            if (m < lim) {
                float y[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
                const int64_t at = tile_base + m * row_stride;
                if (p.D) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = static_cast<float>(byte_of(e < 4 ? xb.x : xb.y, e & 3));
                        y[e] += (s_xs[ecol + e] * xv) * e_Dv[e];
                    }
                }
                if (p.z) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float zv = z_scale * static_cast<float>(byte_of(e < 4 ? zb.x : zb.y, e & 3));
                        y[e] *= zv * __builtin_amdgcn_rcpf(1.0f + fexp(-zv));
                    }
                }
                v8h o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<_Float16>(y[e]);
                *reinterpret_cast<v8h*>(out + at) = o;
            }
        }
    }
}

int validate(const QaSsdParams* p) {
    if (!p || !p->x || !p->dt || !p->A_log || !p->B || !p->C || !p->out) return QA_ERR_NULL;
    if (!p->x_scale || !p->A_log_scale || !p->B_scale || !p->C_scale) return QA_ERR_NULL;
    if (!p->dt_is_fp32 && !p->dt_scale) return QA_ERR_NULL;
    if ((p->D && !p->D_scale) || (p->z && !p->z_scale)) return QA_ERR_NULL;
    if (p->final_states && !p->final_state_is_fp32 && !p->state_scale) return QA_ERR_NULL;
    if (p->nhead_groups > 0 && (!p->x_head_group_range || !p->x_dim_group_range || p->ndim_groups < 1)) return QA_ERR_NULL;
    if (p->batch < 0 || p->seqlen < 0 || p->nheads < 1 || p->ngroups < 1 || p->nheads % p->ngroups != 0) return QA_ERR_SHAPE;
    if (p->headdim != kP) return QA_ERR_UNSUPPORTED;
    if (p->dstate != 64 && p->dstate != 128) return QA_ERR_UNSUPPORTED;
    if (p->chunk_size != 64 && p->chunk_size != 128 && p->chunk_size != 256) return QA_ERR_UNSUPPORTED;
    if (!aligned16(p->x) || !aligned16(p->B) || !aligned16(p->C) || !aligned16(p->out)) return QA_ERR_STRIDE;
    if (p->z && (reinterpret_cast<uintptr_t>(p->z) & 7u)) return QA_ERR_STRIDE;      // the gate is read 8 bytes at a time
    return QA_OK;
}

}  // namespace
}  // namespace qa

extern "C" int64_t qa_ssd_workspace_bytes(const QaSsdParams* p) {
    if (qa::validate(p) != QA_OK) return 0;
    return qa::ws_layout(*p).total;
}

extern "C" int qa_ssd_chunk_scan_fwd(const QaSsdParams* p, void* stream_) {
    using namespace qa;
    const int st = validate(p);
    if (st != QA_OK) return st;
    if (p->batch == 0 || p->seqlen == 0) return QA_OK;
    const Ws ws = ws_layout(*p);
    if (!p->workspace) return QA_ERR_NULL;
    if (p->workspace_bytes < ws.total || (reinterpret_cast<uintptr_t>(p->workspace) & 255u)) return QA_ERR_STRIDE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    uint8_t* base = static_cast<uint8_t*>(p->workspace);
    float* dt_ws = reinterpret_cast<float*>(base + ws.dt);
    float* dA_ws = reinterpret_cast<float*>(base + ws.dA);
    __half* cb_ws = reinterpret_cast<__half*>(base + ws.cb);
    __half* prev = reinterpret_cast<__half*>(base + ws.prev);
    float* final_ws = reinterpret_cast<float*>(base + ws.final_f32);
    __half* c16_ws = reinterpret_cast<__half*>(base + ws.c16);
    const int nc = (p->seqlen + p->chunk_size - 1) / p->chunk_size;
    const int64_t bch = static_cast<int64_t>(p->batch) * nc * p->nheads;
    if (bch > 0x7fffffffLL || static_cast<int64_t>(p->batch) * nc * p->ngroups > 65535) return QA_ERR_SHAPE;

    hipLaunchKernelGGL(ssd_cumsum_kernel, dim3(static_cast<unsigned>((bch + 3) / 4)), dim3(256), 0, stream, *p, dt_ws,
                       dA_ws, nc);
    const int nt = p->chunk_size / 64;
    hipLaunchKernelGGL(ssd_cb_kernel, dim3(nt * (nt + 1) / 2, p->batch * nc * p->ngroups), dim3(64), 0, stream, *p, cb_ws, c16_ws, nc);
    __half* bt16_ws = reinterpret_cast<__half*>(base + ws.bt16);
    const int64_t bcg_tiles = static_cast<int64_t>(p->batch) * nc * p->ngroups * (p->dstate / 32);
    if (bcg_tiles > 0x7fffffffLL) return QA_ERR_SHAPE;
    hipLaunchKernelGGL(ssd_bpack_kernel, dim3(static_cast<unsigned>(bcg_tiles)), dim3(256), 0, stream, *p, bt16_ws, nc);
    const dim3 hgrid(static_cast<unsigned>(p->batch * p->nheads));
    auto launch_state = [&](auto kernel) { hipLaunchKernelGGL(kernel, hgrid, dim3(256), 0, stream, *p, dt_ws, dA_ws, bt16_ws, prev, final_ws, nc); };
    if (p->dstate == 128) {
        if (p->chunk_size == 256) launch_state(ssd_state_kernel<128, 256>);
        else if (p->chunk_size == 128) launch_state(ssd_state_kernel<128, 128>);
        else launch_state(ssd_state_kernel<128, 64>);
    } else {
        if (p->chunk_size == 256) launch_state(ssd_state_kernel<64, 256>);
        else if (p->chunk_size == 128) launch_state(ssd_state_kernel<64, 128>);
        else launch_state(ssd_state_kernel<64, 64>);
    }
    const dim3 sgrid(static_cast<unsigned>(bch));
    auto launch_scan = [&](auto kernel) { hipLaunchKernelGGL(kernel, sgrid, dim3(256), 0, stream, *p, dt_ws, dA_ws, cb_ws, prev, c16_ws, nc); };
    if (p->dstate == 128) {
        if (p->chunk_size == 256) launch_scan(ssd_chunk_scan_kernel<128, 256>);
        else if (p->chunk_size == 128) launch_scan(ssd_chunk_scan_kernel<128, 128>);
        else launch_scan(ssd_chunk_scan_kernel<128, 64>);
    } else {
        if (p->chunk_size == 256) launch_scan(ssd_chunk_scan_kernel<64, 256>);
        else if (p->chunk_size == 128) launch_scan(ssd_chunk_scan_kernel<64, 128>);
        else launch_scan(ssd_chunk_scan_kernel<64, 64>);
    }
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
    if (p->batch == 0 || p->seqlen == 0) return QA_OK;
    if (ws_layout(*p).total > kStaticScratchBytes) return QA_ERR_SCRATCH;
    void* ptr = static_scratch_of_current_device();
    if (!ptr) return QA_ERR_LAUNCH;
    QaSsdParams q = *p;
    q.workspace = ptr;
    q.workspace_bytes = kStaticScratchBytes;
    return qa_ssd_chunk_scan_fwd(&q, stream_);
}
