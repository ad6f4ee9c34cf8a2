// Mamba2 quantized SSD chunk scan (prefill) for gfx950.
//
// Stages and arithmetic follow the reference's Triton pipeline (quamba/triton/quant_ssd_combined.py
// :61-77, grouped :146-162); see each kernel for the file it restates.  fp16 operands, fp32
// accumulation, as there; the one pure int8 contraction (C B^T) runs on the int8 matrix cores.
//   cumsum      dt = clamp(softplus(s_dt q_dt + dt_bias)), dA_cs = within-chunk cumsum(dt * A)
//   cb          CB[m,k] = (s_C s_B) * sum_n q_C[m,n] q_B[k,n]                       (int8 MFMA, lower tiles)
//   chunk_state S_c[p,n] = sum_k f16(x^[k,p]) f16(B^[k,n] exp(dA_last - dA_k) dt_k)   (fp16 MFMA)
//   passing     P_0 = 0, P_{c+1} = exp(dA_last,c) P_c + S_c; P_c kept in fp16; final state fp32 / int8
//   chunk_scan  y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) P_c[p,n] + sum_{k<=m} f16(CB[m,k] e^{dA_m-dA_k} dt_k) f16(x^[k,p])
//               + D x^[m,p], optional z gate, fp16 out                               (fp16 MFMA)
// Both fp16 contractions over the time index need x (and B) with time as the fastest-moving index,
// while memory has channels fastest; the tiles are transposed once on the way into LDS (4x4 blocks:
// four dword loads, four 8-byte LDS stores) and then read as 16-byte MFMA operands.
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

__device__ __forceinline__ float fexp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }
// orders a wave's own LDS writes before its later LDS reads (wave-private scratch needs no workgroup barrier)
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ int8_t byte_of(uint32_t w, int j) { return static_cast<int8_t>((w >> (8 * j)) & 0xffu); }

struct Ws {            // workspace sections (byte offsets), see qa_ssd_workspace_bytes
    int64_t dt, dA, cb, states, prev, final_f32, c16, total;
};

__host__ __device__ inline int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }

__host__ __device__ inline Ws ws_layout(const QaSsdParams& p) {
    const int64_t nc = (p.seqlen + p.chunk_size - 1) / p.chunk_size;
    const int64_t B = p.batch, H = p.nheads, Q = p.chunk_size, G = p.ngroups, P = p.headdim, N = p.dstate;
    Ws w;
    int64_t off = 0;
    w.dt = off; off = align256(off + B * H * nc * Q * 4);
    w.dA = off; off = align256(off + B * H * nc * Q * 4);
    w.cb = off; off = align256(off + B * nc * G * Q * Q * 4);
    w.states = off; off = align256(off + B * nc * H * P * N * 4);
    w.prev = off; off = align256(off + B * nc * H * P * N * 2);
    w.final_f32 = off; off = align256(off + B * H * P * N * 4);
    w.c16 = off; off = align256(off + B * static_cast<int64_t>(p.seqlen) * G * N * 2);
    w.total = off;
    return w;
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
__global__ __launch_bounds__(64) void ssd_cb_kernel(QaSsdParams p, float* cb_out, __half* c16_out, int nc) {
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
    for (int ks = 0; ks < N / 32; ++ks) {
        v4i fc[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = mt * 64 + i * 32 + frow, k = kt * 64 + i * 32 + frow;
            fc[i] = m < lim ? *reinterpret_cast<const v4i*>(p.C + ((static_cast<int64_t>(b) * p.seqlen + t0 + m) * G + g) * N + ks * 32 + fhalf * 16)
                            : v4i{0, 0, 0, 0};
            fb[i] = k < lim ? *reinterpret_cast<const v4i*>(p.B + ((static_cast<int64_t>(b) * p.seqlen + t0 + k) * G + g) * N + ks * 32 + fhalf * 16)
                            : v4i{0, 0, 0, 0};
            if (mt == kt && m < lim) {
                v8h lo, hi;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    lo[e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(static_cast<uint32_t>(fc[i][e >> 2]), e & 3)));
                    hi[e] = static_cast<_Float16>(sC * static_cast<float>(byte_of(static_cast<uint32_t>(fc[i][2 + (e >> 2)]), e & 3)));
                }
                __half* dst = c16_out + ((static_cast<int64_t>(b) * p.seqlen + t0 + m) * G + g) * N + ks * 32 + fhalf * 16;
                *reinterpret_cast<v8h*>(dst) = lo;
                *reinterpret_cast<v8h*>(dst + 8) = hi;
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fc[i], fb[j], acc[i][j], 0, 0, 0);
    }
    // acc[i][j]: lane holds column k = kt*64 + j*32 + (lane & 31), register r row m = mt*64 + i*32 + 8*(r/4) + 4*(lane/32) + r%4
    float* tile = cb_out + ((static_cast<int64_t>(b) * nc + c) * G + g) * Q * Q;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = mt * 64 + i * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
                const int k = kt * 64 + j * 32 + frow;
                tile[static_cast<int64_t>(m) * Q + k] = scale * static_cast<float>(acc[i][j][r]);
            }
}

// ---------------------------------------------------------------------------------------------
// Transposing stage: dst[col][k] (fp16, `pitch` halves per row) <- src rows k (int8, `row_stride`
// bytes apart, NC columns), k in [0, KC).  value = f16((col_scale[col] * q) * k_scale[k]) when
// K_SCALE, else f16(col_scale[col] * q).  Rows k >= k_valid read as zero.
// ---------------------------------------------------------------------------------------------
template <int NC, bool K_SCALE>
__device__ __forceinline__ void stage_transposed(_Float16* dst, int pitch, const int8_t* src, int64_t row_stride,
                                                 int KC, int k_valid, const float* col_scale, const float* k_scale,
                                                 int tid, int nthreads) {
    constexpr int CB = NC / 4;
    for (int id = tid; id < (KC / 4) * CB; id += nthreads) {
        const int kb = id / CB, cb = id % CB;
        uint32_t w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int k = kb * 4 + r;
            w[r] = k < k_valid ? *reinterpret_cast<const uint32_t*>(src + k * row_stride + cb * 4) : 0u;
        }
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const float cs = col_scale[cb * 4 + cc];
            v4h o;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = cs * static_cast<float>(byte_of(w[r], cc));
                if (K_SCALE) v *= k_scale[kb * 4 + r];
                o[r] = static_cast<_Float16>(v);
            }
            *reinterpret_cast<v4h*>(dst + (cb * 4 + cc) * pitch + kb * 4) = o;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Stage 2 (quamba/triton/quant_chunk_state.py:76-89): one workgroup per (batch, chunk, head).
// S[p,n] = sum_k XT[p][k] * BT[n][k]; 4 waves, wave w owns p-tile w&1 and n-tiles 2*(w>>1)..+1 (of 32).
// The chunk is consumed in passes of 128 steps.
// ---------------------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256) void ssd_chunk_state_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws,
                                                              float* states, int nc) {
    constexpr int KC = 128, PITCH = KC + 8, NT = N / 64;      // NT n-tiles per wave
    __shared__ __attribute__((aligned(16))) _Float16 s_xt[kP * PITCH];
    __shared__ __attribute__((aligned(16))) _Float16 s_bt[N * PITCH];
    __shared__ float s_w[KC];
    __shared__ float s_xs[kP];
    __shared__ float s_bs[N];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, frow = lane & 31, fhalf = lane >> 5;
    const int h = blockIdx.x % p.nheads;
    const int c = (blockIdx.x / p.nheads) % nc;
    const int b = blockIdx.x / (p.nheads * nc);
    const int Q = p.chunk_size, G = p.ngroups, H = p.nheads;
    int g, hg;
    group_of(p, h, g, hg);
    const int t0 = c * Q;
    const int lim = min(Q, p.seqlen - t0);
    const float* dt_row = dt_ws + ((static_cast<int64_t>(b) * H + h) * nc + c) * Q;
    const float* dA_row = dA_ws + ((static_cast<int64_t>(b) * H + h) * nc + c) * Q;
    const float dA_last = dA_row[Q - 1];
    if (tid < kP) s_xs[tid] = x_scale_of(p, g, hg, tid);
    const float sB = p.nhead_groups > 0 ? p.B_scale[g] : p.B_scale[0];
    for (int i = tid; i < N; i += 256) s_bs[i] = sB;

    const int pt = wave & 1, nt0 = (wave >> 1) * NT;
    v16f acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

    for (int k0 = 0; k0 < Q; k0 += KC) {
        const int kc = min(KC, Q - k0);
        __syncthreads();                       // previous pass fully consumed (and scale tables written)
        if (tid < KC) s_w[tid] = tid < kc ? fexp(dA_last - dA_row[k0 + tid]) * dt_row[k0 + tid] : 0.0f;
        __syncthreads();
        const int valid = max(0, min(kc, lim - k0));
        stage_transposed<kP, false>(s_xt, PITCH, p.x + ((static_cast<int64_t>(b) * p.seqlen + t0 + k0) * H + h) * kP,
                                    static_cast<int64_t>(H) * kP, KC, valid, s_xs, nullptr, tid, 256);
        stage_transposed<N, true>(s_bt, PITCH, p.B + ((static_cast<int64_t>(b) * p.seqlen + t0 + k0) * G + g) * N,
                                  static_cast<int64_t>(G) * N, KC, valid, s_bs, s_w, tid, 256);
        __syncthreads();
        for (int ks = 0; ks < KC / 16; ++ks) {
            const v8h fx = *reinterpret_cast<const v8h*>(s_xt + (pt * 32 + frow) * PITCH + ks * 16 + fhalf * 8);
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const v8h fb = *reinterpret_cast<const v8h*>(s_bt + ((nt0 + j) * 32 + frow) * PITCH + ks * 16 + fhalf * 8);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx, fb, acc[j], 0, 0, 0);
            }
        }
    }
    // acc[j]: lane holds column n = (nt0+j)*32 + (lane & 31); register r row p = pt*32 + 8*(r/4) + 4*(lane/32) + r%4
    float* out = states + ((static_cast<int64_t>(b) * nc + c) * H + h) * kP * N;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int pp = pt * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
            out[pp * N + (nt0 + j) * 32 + frow] = acc[j][r];
        }
}

// ---------------------------------------------------------------------------------------------
// Stages 3 and 6 (quamba/triton/quant_state_passing.py:60-83, quant_ssm_states.py:43,119): one
// thread per state element, sequential over chunks.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ssd_state_passing_kernel(QaSsdParams p, const float* dA_ws, const float* states,
                                                                __half* prev, float* final_ws, int nc) {
    const int N = p.dstate, H = p.nheads, Q = p.chunk_size;
    const int64_t per_head = static_cast<int64_t>(kP) * N;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(p.batch) * H * per_head) return;
    const int e = static_cast<int>(idx % per_head);
    const int h = static_cast<int>((idx / per_head) % H);
    const int b = static_cast<int>(idx / (per_head * H));
    float s = 0.0f;
    // the chunk states do not depend on the running state: fetch eight chunks at a time, then recur
    constexpr int kBlock = 8;
    const int64_t c_stride = static_cast<int64_t>(H) * per_head;
    const int64_t off0 = (static_cast<int64_t>(b) * nc * H + h) * per_head + e;
    const float* dA_last_p = dA_ws + (static_cast<int64_t>(b) * H + h) * nc * Q + Q - 1;
    for (int c0 = 0; c0 < nc; c0 += kBlock) {
        float st[kBlock], da[kBlock];
#pragma unroll
        for (int i = 0; i < kBlock; ++i) {
            const int c = min(c0 + i, nc - 1);
            st[i] = states[off0 + c * c_stride];
            da[i] = dA_last_p[static_cast<int64_t>(c) * Q];
        }
#pragma unroll
        for (int i = 0; i < kBlock; ++i) {
            if (c0 + i < nc) {
                prev[off0 + (c0 + i) * c_stride] = __float2half(s);
                s = expf(da[i]) * s + st[i];
            }
        }
    }
    const int64_t fo = (static_cast<int64_t>(b) * H + h) * per_head + e;
    if (final_ws) final_ws[fo] = s;
    if (p.final_states) {
        if (p.final_state_is_fp32) {
            static_cast<float*>(p.final_states)[fo] = s;
        } else {
            const int pp = e / N, n = e % N;
            float sc, K;
            if (p.nhead_groups > 0) {
                int g, hg;
                group_of(p, h, g, hg);
                const int dg = dim_group_of(p, g, hg, pp);
                sc = p.state_scale[((g * p.nhead_groups + hg) * p.ndim_groups + dg) * N + n];
                K = 1e6f;
            } else {
                sc = p.state_scale[0];
                K = 1e2f;
            }
            const float s16 = __half2float(__float2half(s));      // the reference hands fp16 states to the quantiser
            static_cast<int8_t*>(p.final_states)[fo] = sat8_rne((s16 * K) / (sc * K));
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Stage 5 (quamba/triton/quant_chunk_scan.py:96-171): one workgroup per (batch, chunk, head);
// each wave owns whole 32-row m-tiles (paired small/large so the causal work balances).
// ---------------------------------------------------------------------------------------------
template <int N, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES == 8 ? 4 : 1) void ssd_chunk_scan_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws,
                                                             const float* cb_ws, const __half* prev, const __half* c16, int nc) {
    constexpr int QMAX = 256, PITCH = QMAX + 8, PPITCH = N + 8, kThreads = 64 * WAVES;
    constexpr int kScratch = 512;      // floats per wave: the decay table (QMAX) or an 8 x 64 piece of the output tile
    __shared__ __attribute__((aligned(16))) _Float16 s_xt[kP * PITCH];
    __shared__ __attribute__((aligned(16))) _Float16 s_prev[kP * PPITCH];     // entering state, rows p
    __shared__ __attribute__((aligned(16))) float s_dt[QMAX];
    __shared__ __attribute__((aligned(16))) float s_dA[QMAX];
    __shared__ __attribute__((aligned(16))) float s_g[WAVES * kScratch];          // per wave: decay * dt of earlier steps
    __shared__ float s_xs[kP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, frow = lane & 31, fhalf = lane >> 5;
    const int h = blockIdx.x % p.nheads;
    const int c = (blockIdx.x / p.nheads) % nc;
    const int b = blockIdx.x / (p.nheads * nc);
    const int Q = p.chunk_size, G = p.ngroups, H = p.nheads;
    int g, hg;
    group_of(p, h, g, hg);
    const int t0 = c * Q;
    const int lim = min(Q, p.seqlen - t0);
    const int64_t row_base = (static_cast<int64_t>(b) * H + h) * nc + c;
    for (int i = tid; i < Q; i += kThreads) {
        s_dt[i] = dt_ws[row_base * Q + i];
        s_dA[i] = dA_ws[row_base * Q + i];
    }
    if (tid < kP) s_xs[tid] = x_scale_of(p, g, hg, tid);
    {
        const __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * kP * N;
        for (int piece = tid; piece < kP * N / 8; piece += kThreads) {
            const int pr = piece / (N / 8), col = (piece % (N / 8)) * 8;
            *reinterpret_cast<uint4*>(s_prev + pr * PPITCH + col) = *reinterpret_cast<const uint4*>(pst + pr * N + col);
        }
    }
    __syncthreads();
    stage_transposed<kP, false>(s_xt, PITCH, p.x + ((static_cast<int64_t>(b) * p.seqlen + t0) * H + h) * kP,
                                static_cast<int64_t>(H) * kP, Q, lim, s_xs, nullptr, tid, kThreads);
    __syncthreads();

    const float* cb = cb_ws + ((static_cast<int64_t>(b) * nc + c) * G + g) * Q * Q;
    const float D_scale = p.D ? *p.D_scale : 0.0f;
    const float z_scale = p.z ? *p.z_scale : 0.0f;
    const int nmt = Q / 32;
    const int per_wave = max(1, nmt / WAVES);
    float e_Dv[8];                                           // D of the eight columns this lane writes
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int pp = (lane & 7) * 8 + e;
        e_Dv[e] = p.D ? D_scale * static_cast<float>(p.D[p.D_has_hdim ? h * kP + pp : h]) : 0.0f;
    }

    for (int s = 0; s < per_wave; ++s) {
        // tile order 0, nmt-1, 1, nmt-2, ...: wave w takes entries w*per_wave + s
        const int entry = wave * per_wave + s;
        if (entry >= nmt) break;
        const int mt = (entry & 1) ? nmt - 1 - (entry >> 1) : (entry >> 1);
        const int m_lane = mt * 32 + frow;                 // row of this lane's A operands
        v16f acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

        // Loads of this tile that do not depend on each other go out first: the lane's pieces of its
        // C row (term 1) and the first two k-steps of its CB row (term 2).
        const __half* c_row = c16 + ((static_cast<int64_t>(b) * p.seqlen + t0 + m_lane) * G + g) * N;
        v8h c_frag[N / 16];
#pragma unroll
        for (int ks = 0; ks < N / 16; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) c_frag[ks][e] = static_cast<_Float16>(0.0f);
            if (m_lane < lim) c_frag[ks] = *reinterpret_cast<const v8h*>(c_row + ks * 16 + fhalf * 8);
        }
        const float* cb_row = cb + static_cast<int64_t>(m_lane) * Q + fhalf * 8;
        const int nks = 2 * (mt + 1);
        constexpr int kAhead = 2;
        float4 pre[kAhead][2];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            if (a < nks) {
                pre[a][0] = *reinterpret_cast<const float4*>(cb_row + a * 16);
                pre[a][1] = *reinterpret_cast<const float4*>(cb_row + a * 16 + 4);
            }
        }

        // term 1: C^ (rows m, dstate contiguous) x entering state (rows p, dstate contiguous, staged in LDS)
#pragma unroll
        for (int ks = 0; ks < N / 16; ++ks) {
            const v8h fc = c_frag[ks];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const v8h fs = *reinterpret_cast<const v8h*>(s_prev + (j * 32 + frow) * PPITCH + ks * 16 + fhalf * 8);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fc, fs, acc[j], 0, 0, 0);
            }
        }
        // Decay factors.  The cumulative dA decreases along the chunk, so with ref = dA at the first row
        // of this m-tile, exp(dA_m - dA_k) = exp(dA_m - ref) * exp(ref - dA_k) for every k before the
        // tile, both factors <= 1.  The k factor (times dt_k) is tabulated once per tile by the wave; the
        // row factor is applied to the accumulator after the off-diagonal k-steps, together with term 1
        // (whose decay exp(dA_m) = exp(ref) * exp(dA_m - ref)).  Only the two diagonal k-steps evaluate
        // the decay per element.  acc = E_m * (exp(ref) * T1 + sum_{k < m0} (CB * G_k) x_k) + diagonal.
        const int m0 = mt * 32;
        const float ref = s_dA[m0];
        float* g_tab = s_g + wave * kScratch;
        for (int k = lane; k < m0; k += 64) g_tab[k] = fexp(ref - s_dA[k]) * s_dt[k];
        wave_sync();
        const float e_ref = fexp(ref);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            acc[0][r] *= e_ref;
            acc[1][r] *= e_ref;
        }
        const int n_off = 2 * mt;                       // k-steps entirely before the tile
        for (int ks = 0; ks < nks; ks += kAhead) {
#pragma unroll
            for (int a = 0; a < kAhead; ++a) {
                const int kk = ks + a;
                if (kk >= nks) break;                   // nks is even, kept for safety
                const float4 c0 = pre[a][0], c1 = pre[a][1];
                if (kk + kAhead < nks) {
                    pre[a][0] = *reinterpret_cast<const float4*>(cb_row + (kk + kAhead) * 16);
                    pre[a][1] = *reinterpret_cast<const float4*>(cb_row + (kk + kAhead) * 16 + 4);
                }
                const int k0 = kk * 16 + fhalf * 8;
                const float cbv[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
                v8h fl;
                if (kk < n_off) {
                    const float4 g0 = *reinterpret_cast<const float4*>(g_tab + k0), g1 = *reinterpret_cast<const float4*>(g_tab + k0 + 4);
                    const float gk[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) fl[e] = static_cast<_Float16>(cbv[e] * gk[e]);
                } else {
                    if (kk == n_off) {
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
                        const float wv = (cbv[e] * fexp(dA_m - dAk[e])) * dtk[e];
                        fl[e] = static_cast<_Float16>(k <= m_lane ? wv : 0.0f);
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const v8h fx = *reinterpret_cast<const v8h*>(s_xt + (j * 32 + frow) * PITCH + k0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fl, fx, acc[j], 0, 0, 0);
                }
            }
        }
        wave_sync();                                    // the table is done with: its space now carries the output tile
        // Epilogue.  In the accumulators a lane holds one column p and 16 rows; memory wants rows of 64
        // contiguous columns.  The tile passes through the wave's scratch eight rows at a time (registers
        // 4q..4q+3 of both accumulators are rows 8q + 4*(lane/32) + 0..3), after which lane l holds row
        // l/8 and the eight columns 8*(l%8)..+7: skip term and gate read 8 bytes, the output is one
        // 16-byte store.
        const int64_t row_stride = static_cast<int64_t>(H) * kP;
        const int erow = lane >> 3, ecol = (lane & 7) * 8;
        const int64_t tile_base = (static_cast<int64_t>(b) * p.seqlen + t0) * row_stride + static_cast<int64_t>(h) * kP + ecol;
        __half* out = static_cast<__half*>(p.out);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) g_tab[(4 * fhalf + t) * 64 + j * 32 + frow] = acc[j][4 * q + t];
            wave_sync();
            const int m = mt * 32 + 8 * q + erow;
            const float4 y0 = *reinterpret_cast<const float4*>(g_tab + erow * 64 + ecol);
            const float4 y1 = *reinterpret_cast<const float4*>(g_tab + erow * 64 + ecol + 4);
            wave_sync();                                // the next piece overwrites the scratch
            if (m < lim) {
                float y[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
                const int64_t at = tile_base + m * row_stride;
                if (p.D) {
                    const uint2 xr = *reinterpret_cast<const uint2*>(p.x + at);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = static_cast<float>(byte_of(e < 4 ? xr.x : xr.y, e & 3));
                        y[e] += (s_xs[ecol + e] * xv) * e_Dv[e];
                    }
                }
                if (p.z) {
                    const uint2 zr = *reinterpret_cast<const uint2*>(p.z + at);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float zv = z_scale * static_cast<float>(byte_of(e < 4 ? zr.x : zr.y, e & 3));
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
    float* cb_ws = reinterpret_cast<float*>(base + ws.cb);
    float* states = reinterpret_cast<float*>(base + ws.states);
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
    if (p->dstate == 128) {
        hipLaunchKernelGGL(ssd_chunk_state_kernel<128>, dim3(static_cast<unsigned>(bch)), dim3(256), 0, stream, *p, dt_ws, dA_ws,
                           states, nc);
    } else {
        hipLaunchKernelGGL(ssd_chunk_state_kernel<64>, dim3(static_cast<unsigned>(bch)), dim3(256), 0, stream, *p, dt_ws, dA_ws,
                           states, nc);
    }
    const int64_t elems = static_cast<int64_t>(p->batch) * p->nheads * kP * p->dstate;
    hipLaunchKernelGGL(ssd_state_passing_kernel, dim3(static_cast<unsigned>((elems + 255) / 256)), dim3(256), 0, stream, *p,
                       dA_ws, states, prev, final_ws, nc);
    // four waves per workgroup, m-tiles paired small/large per wave (eight waves with one tile each measured slower)
    const dim3 sgrid(static_cast<unsigned>(bch));
    if (p->dstate == 128) hipLaunchKernelGGL((ssd_chunk_scan_kernel<128, 4>), sgrid, dim3(256), 0, stream, *p, dt_ws, dA_ws, cb_ws, prev, c16_ws, nc);
    else hipLaunchKernelGGL((ssd_chunk_scan_kernel<64, 4>), sgrid, dim3(256), 0, stream, *p, dt_ws, dA_ws, cb_ws, prev, c16_ws, nc);
    return check_launch();
}
