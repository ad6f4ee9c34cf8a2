// Mamba2 quantized SSD chunk scan for any head dimension (<= 256), state count and chunk length, and for tensors
// without 16-byte alignment: the shapes the matrix-core kernels of ssd.hip are not built for.
//
// Same stages, same arithmetic and the same fp16 rounding points as there (quamba/triton/quant_ssd_combined.py
// :61-77, grouped :146-162; the kernels restated are named at each stage), on the vector ALUs with 64-wide tiles in
// every dimension and byte-wise loads, so that nothing depends on a size being a multiple of anything:
//   cumsum      dt = clamp(softplus(s_dt q_dt + dt_bias)), dA_cs = within-chunk cumsum(dt * A)
//   state       S_c[p,n] = sum_k f16(x^[k,p]) f16(B^[k,n] (exp(dA_last - dA_k) dt_k));  P_{c+1} = exp(dA_last) P_c + S_c,
//               f16(P_c) stored as the state entering chunk c; final state fp32 / int8
//   chunk_scan  y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) f16(P_c[p,n])
//                      + sum_{k<=m} f16(((s_C s_B) (q_C[m,:] . q_B[k,:])) exp(dA_m - dA_k) dt_k) f16(x^[k,p])
//                      + x^[m,p] D, optional z gate, fp16 out
// All sums are fp32; the integer contraction of C and B is exact (v_dot4_i32_i8).
#include "qa_common.hpp"
#include "ssd_common.hpp"

namespace qa {
namespace {

constexpr int kT = 64;            // tile edge: steps, states, channels of the chunk scan
constexpr int kTP = 32;           // channels per workgroup of the state kernel
constexpr int kThreads = 256;

__device__ __forceinline__ float f16r(float v) { return static_cast<float>(static_cast<_Float16>(v)); }

// ---------------------------------------------------------------------------------------------
// Stage 1 (quamba/triton/quant_chunk_cumsum.py:56-70).  One wave per (batch, chunk, head): every lane takes
// ceil(chunk_size / 64) consecutive steps, then an inclusive scan across the lanes.  Steps past the end of the
// sequence have dt = 0.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void ssd_general_cumsum_kernel(QaSsdParams p, float* dt_out, float* dA_out, int nc) {
    const int lane = threadIdx.x & 63;
    const unsigned idx = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (idx >= static_cast<unsigned>(p.batch) * static_cast<unsigned>(nc) * static_cast<unsigned>(p.nheads)) return;
    const int h = static_cast<int>(idx % static_cast<unsigned>(p.nheads));
    const int c = static_cast<int>((idx / static_cast<unsigned>(p.nheads)) % static_cast<unsigned>(nc));
    const int b = static_cast<int>(idx / (static_cast<unsigned>(p.nheads) * static_cast<unsigned>(nc)));
    const int Q = p.chunk_size, E = (Q + 63) / 64;
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

// ---------------------------------------------------------------------------------------------
// Stages 2, 3 and 6 (quamba/triton/quant_chunk_state.py:76-89, quant_state_passing.py:60-83, quant_ssm_states.py
// :43,119).  A workgroup per (batch, head, 32 channels, 64 states) walks the chunks in order with its part of the
// running state in registers (a thread: two channels x four states); the chunk's operands pass through LDS in tiles
// of 64 steps, already rounded to fp16 and widened again.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void ssd_general_state_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws, __half* prev, int nc) {
    __shared__ __attribute__((aligned(16))) float xh[kT][kTP];
    __shared__ __attribute__((aligned(16))) float bw[kT][kT];
    __shared__ float wk[kT];
    __shared__ float xs[kTP];
    const int P = p.headdim, N = p.dstate, Q = p.chunk_size, H = p.nheads, G = p.ngroups, L = p.seqlen;
    const int ptiles = (P + kTP - 1) / kTP, ntiles = (N + kT - 1) / kT;
    const int tid = threadIdx.x, tp = tid / 16, tn = tid % 16;
    unsigned idx = blockIdx.x;
    const int n0 = static_cast<int>(idx % ntiles) * kT; idx /= ntiles;
    const int p0 = static_cast<int>(idx % ptiles) * kTP; idx /= ptiles;
    const int h = static_cast<int>(idx % H);
    const int b = static_cast<int>(idx / H);
    int g, hg;
    ssd_group_of(p, h, g, hg);
    const float sB = p.nhead_groups > 0 ? p.B_scale[g] : p.B_scale[0];
    if (tid < kTP) xs[tid] = p0 + tid < P ? ssd_x_scale_of(p, g, hg, p0 + tid) : 0.0f;
    const int64_t rows0 = (static_cast<int64_t>(b) * H + h) * nc;
    float run[2][4] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};

    for (int c = 0; c < nc; ++c) {
        const int t0 = c * Q;
        const int lim = min(Q, L - t0);
        const float* dA_row = dA_ws + (rows0 + c) * Q;
        const float* dt_row = dt_ws + (rows0 + c) * Q;
        const float dA_last = dA_row[Q - 1];
        float acc[2][4] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
        for (int k0 = 0; k0 < lim; k0 += kT) {
            __syncthreads();                                       // the tile before is consumed (first pass: xs is written)
            if (tid < kT) wk[tid] = k0 + tid < lim ? ssd_exp(dA_last - dA_row[k0 + tid]) * dt_row[k0 + tid] : 0.0f;
            __syncthreads();
            for (int i = tid; i < kT * kTP; i += kThreads) {
                const int kk = i / kTP, pp = i % kTP;
                float v = 0.0f;
                if (k0 + kk < lim && p0 + pp < P) {
                    const int8_t q = p.x[((static_cast<int64_t>(b) * L + t0 + k0 + kk) * H + h) * P + p0 + pp];
                    v = f16r(xs[pp] * static_cast<float>(q));
                }
                xh[kk][pp] = v;
            }
            for (int i = tid; i < kT * kT; i += kThreads) {
                const int kk = i / kT, nn = i % kT;
                float v = 0.0f;
                if (k0 + kk < lim && n0 + nn < N) {
                    const int8_t q = p.B[((static_cast<int64_t>(b) * L + t0 + k0 + kk) * G + g) * N + n0 + nn];
                    v = f16r((sB * static_cast<float>(q)) * wk[kk]);
                }
                bw[kk][nn] = v;
            }
            __syncthreads();
            const int steps = min(kT, lim - k0);
            for (int kk = 0; kk < steps; ++kk) {
                const float2 xv = *reinterpret_cast<const float2*>(&xh[kk][2 * tp]);
                const float4 bv = *reinterpret_cast<const float4*>(&bw[kk][4 * tn]);
                acc[0][0] += xv.x * bv.x; acc[0][1] += xv.x * bv.y; acc[0][2] += xv.x * bv.z; acc[0][3] += xv.x * bv.w;
                acc[1][0] += xv.y * bv.x; acc[1][1] += xv.y * bv.y; acc[1][2] += xv.y * bv.z; acc[1][3] += xv.y * bv.w;
            }
        }
        // P <- exp(dA_last) P + S
        const float decay = ssd_exp(dA_last);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) run[i][j] = decay * run[i][j] + acc[i][j];
        if (c + 1 < nc) {
            // the state entering chunk c + 1, in fp16 as the reference keeps it
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int pp = p0 + 2 * tp + i, nn = n0 + 4 * tn + j;
                    if (pp < P && nn < N) prev[(((static_cast<int64_t>(b) * nc + c + 1) * H + h) * P + pp) * N + nn] = __float2half(run[i][j]);
                }
        }
    }

    if (p.final_states) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int pp = p0 + 2 * tp + i, nn = n0 + 4 * tn + j;
                if (pp < P && nn < N) {
                    const int64_t fo = ((static_cast<int64_t>(b) * H + h) * P + pp) * N + nn;
                    if (p.final_state_is_fp32) static_cast<float*>(p.final_states)[fo] = run[i][j];
                    else static_cast<int8_t*>(p.final_states)[fo] = ssd_quantize_state(p, g, hg, pp, nn, N, run[i][j]);
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Stages 4 and 5 (quamba/triton/quant_bmm_chunk.py:60-66, quant_chunk_scan.py:96-171).  A workgroup per (batch,
// chunk, head, 64 rows m, 64 channels p); a thread owns four rows and four channels.  Term 1 walks the states in
// tiles of 64; term 2 walks the steps k up to the diagonal in tiles of 64, forming the tile's integer C B^T itself
// (a thread: four rows m x four steps k, states in tiles of 64) and from it the fp16 weights.
// ---------------------------------------------------------------------------------------------
struct GeneralScanSmem {
    union {
        struct { float ct[kT][kT]; float pt[kT][kT]; } one;                                  // [state][row m], [state][channel]
        struct { float wt[kT][kT]; float xh[kT][kT]; uint32_t cq[kT][17]; uint32_t bq[kT][17]; } two;   // [step][row m], [step][channel]; codes, four to a word
    };
    float dA_m[kT], dA_k[kT], dt_k[kT], xs[kT], Dv[kT];
};

__global__ __launch_bounds__(kThreads) void ssd_general_chunk_scan_kernel(QaSsdParams p, const float* dt_ws, const float* dA_ws, const __half* prev, int nc) {
    __shared__ __attribute__((aligned(16))) GeneralScanSmem sm;
    const int P = p.headdim, N = p.dstate, Q = p.chunk_size, H = p.nheads, G = p.ngroups, L = p.seqlen;
    const int ptiles = (P + kT - 1) / kT, mtiles = (Q + kT - 1) / kT;
    const int tid = threadIdx.x, tm = tid / 16, tq = tid % 16;
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
        sm.xs[tid] = pp < P ? ssd_x_scale_of(p, g, hg, pp) : 0.0f;
        sm.Dv[tid] = (!p.D || pp >= P) ? 0.0f : *p.D_scale * static_cast<float>(p.D_has_hdim ? p.D[h * P + pp] : p.D[h]);
        sm.dA_m[tid] = dA_row[min(m0 + tid, Q - 1)];
    }
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

    // term 1: C^ (rows m) x the state entering the chunk (rows p); zero for the first chunk
    if (c > 0) {
        const __half* pst = prev + ((static_cast<int64_t>(b) * nc + c) * H + h) * P * N;
        for (int n0 = 0; n0 < N; n0 += kT) {
            __syncthreads();
            for (int i = tid; i < kT * kT; i += kThreads) {
                const int r = i / kT, nn = i % kT;
                float cv = 0.0f, pv = 0.0f;
                if (n0 + nn < N) {
                    if (m0 + r < lim) cv = f16r(sC * static_cast<float>(Crow0[(m0 + r) * cstep + n0 + nn]));
                    if (p0 + r < P) pv = __half2float(pst[static_cast<int64_t>(p0 + r) * N + n0 + nn]);
                }
                // (a thread's row r is a column here: the 16-byte pieces of a row are exchanged by the state's low bits,
                // so that the 64 states a wave writes do not all fall into one bank)
                sm.one.ct[nn][r ^ ((nn & 15) << 2)] = cv;
                sm.one.pt[nn][r ^ ((nn & 15) << 2)] = pv;
            }
            __syncthreads();
            const int states = min(kT, N - n0);
            for (int nn = 0; nn < states; ++nn) {
                const float4 cv = *reinterpret_cast<const float4*>(&sm.one.ct[nn][(4 * tm) ^ ((nn & 15) << 2)]);
                const float4 pv = *reinterpret_cast<const float4*>(&sm.one.pt[nn][(4 * tq) ^ ((nn & 15) << 2)]);
                const float cvv[4] = {cv.x, cv.y, cv.z, cv.w}, pvv[4] = {pv.x, pv.y, pv.z, pv.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] += cvv[i] * pvv[j];
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float em = ssd_exp(sm.dA_m[4 * tm + i]);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] *= em;
        }
    }

    // term 2: steps k <= m, tiles of 64 steps up to the one that holds the last row's diagonal
    const int k_end = min(m0 + kT, lim);
    for (int k0 = 0; k0 < k_end; k0 += kT) {
        __syncthreads();                                           // the tiles before are consumed
        if (tid < kT) {
            const int k = k0 + tid;
            sm.dA_k[tid] = dA_row[min(k, Q - 1)];
            sm.dt_k[tid] = k < lim ? dt_row[k] : 0.0f;
        }
        // integer C B^T of the tile: rows 4 tm .. + 3, steps 4 tq .. + 3
        int cb[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) cb[i][j] = 0;
        for (int n0 = 0; n0 < N; n0 += kT) {
            if (n0 > 0) __syncthreads();
            for (int i = tid; i < kT * 16; i += kThreads) {
                const int r = i / 16, w = i % 16;
                uint32_t cw = 0u, bwd = 0u;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int nn = n0 + 4 * w + e;
                    if (nn < N) {
                        if (m0 + r < lim) cw |= static_cast<uint32_t>(static_cast<uint8_t>(Crow0[(m0 + r) * cstep + nn])) << (8 * e);
                        if (k0 + r < lim) bwd |= static_cast<uint32_t>(static_cast<uint8_t>(Brow0[(k0 + r) * cstep + nn])) << (8 * e);
                    }
                }
                sm.two.cq[r][w] = cw;
                sm.two.bq[r][w] = bwd;
            }
            __syncthreads();
#pragma unroll 4
            for (int w = 0; w < 16; ++w) {
                uint32_t cw[4], bwd[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    cw[i] = sm.two.cq[4 * tm + i][w];
                    bwd[i] = sm.two.bq[4 * tq + i][w];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) cb[i][j] = __builtin_amdgcn_sdot4(static_cast<int>(cw[i]), static_cast<int>(bwd[j]), cb[i][j], false);
            }
        }
        // the weights, rounded to fp16 where the reference rounds them, as [step][row]; x^ as [step][channel]
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + 4 * tq + j;
            float wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + 4 * tm + i;
                wv[i] = (k <= m && m < lim)
                            ? f16r(((cb_scale * static_cast<float>(cb[i][j])) * ssd_exp(sm.dA_m[4 * tm + i] - sm.dA_k[4 * tq + j])) * sm.dt_k[4 * tq + j])
                            : 0.0f;
            }
            *reinterpret_cast<float4*>(&sm.two.wt[4 * tq + j][4 * tm]) = make_float4(wv[0], wv[1], wv[2], wv[3]);
        }
        for (int i = tid; i < kT * kT; i += kThreads) {
            const int kk = i / kT, pp = i % kT;
            float v = 0.0f;
            if (k0 + kk < lim && p0 + pp < P) v = f16r(sm.xs[pp] * static_cast<float>(xrow0[(k0 + kk) * xstep + p0 + pp]));
            sm.two.xh[kk][pp] = v;
        }
        __syncthreads();
        const int steps = min(kT, lim - k0);
        for (int kk = 0; kk < steps; ++kk) {
            const float4 wv = *reinterpret_cast<const float4*>(&sm.two.wt[kk][4 * tm]);
            const float4 xv = *reinterpret_cast<const float4*>(&sm.two.xh[kk][4 * tq]);
            const float wvv[4] = {wv.x, wv.y, wv.z, wv.w}, xvv[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += wvv[i] * xvv[j];
        }
    }

    // skip term, gate, fp16 out
    const float z_scale = p.z ? *p.z_scale : 0.0f;
    __half* out = static_cast<__half*>(p.out) + ((static_cast<int64_t>(b) * L + t0) * H + h) * P;
    const int8_t* zrow0 = p.z ? p.z + ((static_cast<int64_t>(b) * L + t0) * H + h) * P : nullptr;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + 4 * tm + i;
        if (m >= lim) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int pl = 4 * tq + j, pp = p0 + pl;
            if (pp >= P) continue;
            float y = acc[i][j];
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
    const int64_t state = static_cast<int64_t>(p.batch) * p.nheads * ((p.headdim + kTP - 1) / kTP) * ((p.dstate + kT - 1) / kT);
    // one-dimensional grids; the cumsum kernel numbers its (batch, chunk, head) items in 32 bits
    if (scan > 0x7fffffffLL || state > 0x7fffffffLL) return QA_ERR_SHAPE;
    return QA_OK;
}

void ssd_general_launch(const QaSsdParams& p, float* dt_ws, float* dA_ws, __half* prev_ws, int nc, hipStream_t stream) {
    const int64_t bch = static_cast<int64_t>(p.batch) * nc * p.nheads;
    const int64_t scan = bch * ((p.chunk_size + kT - 1) / kT) * ((p.headdim + kT - 1) / kT);
    const int64_t state = static_cast<int64_t>(p.batch) * p.nheads * ((p.headdim + kTP - 1) / kTP) * ((p.dstate + kT - 1) / kT);
    hipLaunchKernelGGL(ssd_general_cumsum_kernel, dim3(static_cast<unsigned>((bch + 3) / 4)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, nc);
    hipLaunchKernelGGL(ssd_general_state_kernel, dim3(static_cast<unsigned>(state)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, prev_ws, nc);
    hipLaunchKernelGGL(ssd_general_chunk_scan_kernel, dim3(static_cast<unsigned>(scan)), dim3(kThreads), 0, stream, p, dt_ws, dA_ws, prev_ws, nc);
}

}  // namespace qa
