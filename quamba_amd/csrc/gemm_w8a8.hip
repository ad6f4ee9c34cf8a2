// W8A8 GEMM on the int8 matrix cores with a fused scale epilogue.
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]            (int32, exact)
//   d[m,n]   = cast( s_a[m|0] * ( s_w[n|0] * float(acc) ) )     cast: fp16 RN, or int8 saturating with
//                                                               round-half-even (or half-away for the GEMV rule)
// Reference arithmetic: csrc/linear/quant_linear_fwd_kernel.cuh:63-130 (epilogue :85-109),
// csrc/linear/quant_linear_fwd_gemv_kernel.cuh:56-60 (roundf variant).
//
// Mapping for gfx950: a 2x2 grid of waves per workgroup, each wave owning TM x TN tiles of
// v_mfma_i32_32x32x32_i8 (32x32 outputs, 32 k-bytes per instruction, 16 bytes per lane per
// operand).  Both operands are K-contiguous in memory, so a 16-byte chunk of a row is exactly
// one lane's MFMA operand: tiles of BK = 64 bytes per row travel global -> registers -> LDS as
// 16-byte chunks, double-buffered, with the chunk index XOR-swizzled by the row so that the
// fragment reads (32 rows x one chunk) spread over all LDS banks without padding.
// The weight fragment is the MFMA "A" operand and the activation fragment the "B" operand, so a
// lane ends up with 4 consecutive output columns n for one row m; the epilogue scales, converts,
// stages the tile through LDS and writes full 16-byte pieces of output rows.
#include "qa_common.hpp"

namespace qa {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;            // k-bytes per LDS tile row
constexpr int kGemmThreads = 256;  // 4 waves, 2 (m) x 2 (n)

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 3); }

template <int TM, int TN>
struct GemmCfg {
    static constexpr int kBM = 2 * TM * 32;
    static constexpr int kBN = 2 * TN * 32;
    static constexpr int kAChunks = kBM * 4 / kGemmThreads;   // 16-byte chunks per thread per tile
    static constexpr int kWChunks = kBN * 4 / kGemmThreads;
    static constexpr int kStageBytes = (kBM + kBN) * kBK;
    static constexpr int kLdsBytes = 2 * kStageBytes;
};

template <int TM, int TN, int OUT>   // OUT: QA_OUT_I8 / QA_OUT_F16
__global__ __launch_bounds__(kGemmThreads) void gemm_w8a8_kernel(QaGemmW8A8Params p) {
    using Cfg = GemmCfg<TM, TN>;
    constexpr int BM = Cfg::kBM, BN = Cfg::kBN;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    // consecutive workgroups walk down m first so that neighbours share the same weight tile
    const int tiles_m = (p.m + BM - 1) / BM;
    const int m0 = (blockIdx.x % tiles_m) * BM;
    const int n0 = (blockIdx.x / tiles_m) * BN;

    uint4 ra[Cfg::kAChunks], rw[Cfg::kWChunks];

    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < Cfg::kAChunks; ++i) {
            const int id = tid + i * kGemmThreads;
            const int row = id >> 2, c = id & 3;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (m0 + row < p.m && k0 + c * 16 < p.k) {
                v = *reinterpret_cast<const uint4*>(p.a + static_cast<int64_t>(m0 + row) * p.lda + k0 + c * 16);
            }
            ra[i] = v;
        }
#pragma unroll
        for (int i = 0; i < Cfg::kWChunks; ++i) {
            const int id = tid + i * kGemmThreads;
            const int row = id >> 2, c = id & 3;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (n0 + row < p.n && k0 + c * 16 < p.k) {
                v = *reinterpret_cast<const uint4*>(p.w + static_cast<int64_t>(n0 + row) * p.ldw + k0 + c * 16);
            }
            rw[i] = v;
        }
    };
    auto store_tile = [&](int stage) {
        uint8_t* sa = lds + stage * Cfg::kStageBytes;
        uint8_t* sw = sa + BM * kBK;
#pragma unroll
        for (int i = 0; i < Cfg::kAChunks; ++i) {
            const int id = tid + i * kGemmThreads;
            const int row = id >> 2, c = id & 3;
            *reinterpret_cast<uint4*>(sa + row * kBK + swz(row, c) * 16) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < Cfg::kWChunks; ++i) {
            const int id = tid + i * kGemmThreads;
            const int row = id >> 2, c = id & 3;
            *reinterpret_cast<uint4*>(sw + row * kBK + swz(row, c) * 16) = rw[i];
        }
    };

    v16i acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int k_tiles = (p.k + kBK - 1) / kBK;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    const int frow = lane & 31;       // row inside a 32-row fragment
    const int fhalf = lane >> 5;      // which 16-byte half of the 32 k-bytes
    for (int kt = 0; kt < k_tiles; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < k_tiles) load_tile((kt + 1) * kBK);
        const uint8_t* sa = lds + stage * Cfg::kStageBytes + (wm * TM * 32) * kBK;
        const uint8_t* sw = lds + stage * Cfg::kStageBytes + BM * kBK + (wn * TN * 32) * kBK;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            v4i fa[TM], fw[TN];
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int row = j * 32 + frow;
                fa[j] = *reinterpret_cast<const v4i*>(sa + row * kBK + swz(row, kk * 2 + fhalf) * 16);
            }
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                const int row = i * 32 + frow;
                fw[i] = *reinterpret_cast<const v4i*>(sw + row * kBK + swz(row, kk * 2 + fhalf) * 16);
            }
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[i], fa[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < k_tiles) store_tile(stage ^ 1);
        __syncthreads();
    }

    // Epilogue.  In acc[i][j] lane l holds output row m = j*32 + (l & 31) and, in register r,
    // column n = i*32 + 8*(r/4) + 4*(l/32) + (r%4).
    constexpr int kElt = OUT == QA_OUT_I8 ? 1 : 2;
    constexpr int kPitch = TN * 32 * kElt + 16;          // bytes per staged row (+16: bank spread)
    static_assert(4 * 32 * kPitch <= Cfg::kLdsBytes, "epilogue staging does not fit");
    uint8_t* stg = lds + wave * (32 * kPitch);
    const int wave_m0 = m0 + wm * TM * 32, wave_n0 = n0 + wn * TN * 32;
    const bool vec_store = (p.ldd * kElt) % 16 == 0 && aligned16(p.d);
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = wave_m0 + j * 32 + frow;
        const float sa_m = p.use_alpha ? p.alpha : p.a_scale[p.a_scale_numel == 1 ? 0 : min(m, p.m - 1)];
#pragma unroll
        for (int i = 0; i < TN; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = i * 32 + 8 * q + 4 * fhalf;      // first of 4 consecutive columns
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int n = wave_n0 + nl + e;
                    const float accf = static_cast<float>(acc[i][j][q * 4 + e]);
                    if (p.use_alpha) {
                        v[e] = sa_m * accf;
                    } else {
                        const float sw_n = p.w_scale[p.w_scale_numel == 1 ? 0 : min(n, p.n - 1)];
                        // GEMV rule (round-half-away mode): the two scales are multiplied first
                        v[e] = p.round_mode == QA_ROUND_HALF_AWAY ? (sw_n * sa_m) * accf : sa_m * (sw_n * accf);
                    }
                }
                if (OUT == QA_OUT_I8) {
                    uint32_t packed = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int8_t r8 = p.round_mode == QA_ROUND_RNE ? sat8_rne(v[e]) : sat8_half_away(v[e]);
                        packed |= static_cast<uint32_t>(static_cast<uint8_t>(r8)) << (8 * e);
                    }
                    *reinterpret_cast<uint32_t*>(stg + frow * kPitch + nl) = packed;
                } else {
                    __half2 lo = __floats2half2_rn(v[0], v[1]), hi = __floats2half2_rn(v[2], v[3]);
                    uint2 pk;
                    pk.x = *reinterpret_cast<uint32_t*>(&lo);
                    pk.y = *reinterpret_cast<uint32_t*>(&hi);
                    *reinterpret_cast<uint2*>(stg + frow * kPitch + nl * 2) = pk;
                }
            }
        }
        __syncthreads();
        // 32 rows x (TN*32*kElt) bytes, 16 bytes per lane
        constexpr int kPiecesPerRow = TN * 32 * kElt / 16;
        for (int piece = lane; piece < 32 * kPiecesPerRow; piece += 64) {
            const int r = piece / kPiecesPerRow, cb = (piece % kPiecesPerRow) * 16;
            const int mm = wave_m0 + j * 32 + r;
            const int nn = wave_n0 + cb / kElt;
            if (mm >= p.m || nn >= p.n) continue;
            uint8_t* dst = static_cast<uint8_t*>(p.d) + (static_cast<int64_t>(mm) * p.ldd + nn) * kElt;
            const uint4 val = *reinterpret_cast<const uint4*>(stg + r * kPitch + cb);
            if (vec_store && nn + 16 / kElt <= p.n) {
                *reinterpret_cast<uint4*>(dst) = val;
            } else {
                const uint8_t* src = reinterpret_cast<const uint8_t*>(&val);
                const int nbytes = min(16, (p.n - nn) * kElt);
                for (int e = 0; e < nbytes; ++e) dst[e] = src[e];
            }
        }
        __syncthreads();
    }
}

template <int TM, int TN>
int launch_gemm(const QaGemmW8A8Params& p, hipStream_t stream) {
    using Cfg = GemmCfg<TM, TN>;
    const int64_t tiles = static_cast<int64_t>((p.m + Cfg::kBM - 1) / Cfg::kBM) * ((p.n + Cfg::kBN - 1) / Cfg::kBN);
    if (tiles > 0x7fffffffLL) return QA_ERR_SHAPE;
    if (p.out_type == QA_OUT_I8) {
        hipLaunchKernelGGL((gemm_w8a8_kernel<TM, TN, QA_OUT_I8>), dim3(static_cast<unsigned>(tiles)),
                           dim3(kGemmThreads), Cfg::kLdsBytes, stream, p);
    } else {
        hipLaunchKernelGGL((gemm_w8a8_kernel<TM, TN, QA_OUT_F16>), dim3(static_cast<unsigned>(tiles)),
                           dim3(kGemmThreads), Cfg::kLdsBytes, stream, p);
    }
    return check_launch();
}

}  // namespace
}  // namespace qa

extern "C" int qa_gemm_w8a8(const QaGemmW8A8Params* p, void* stream_) {
    using namespace qa;
    if (!p || !p->a || !p->w || !p->d) return QA_ERR_NULL;
    if (!p->use_alpha && (!p->a_scale || !p->w_scale)) return QA_ERR_NULL;
    if (p->m < 0 || p->n < 0 || p->k < 0) return QA_ERR_SHAPE;
    if (p->out_type != QA_OUT_I8 && p->out_type != QA_OUT_F16) return QA_ERR_UNSUPPORTED;
    if (!p->use_alpha && p->a_scale_numel != 1 && p->a_scale_numel != p->m) return QA_ERR_SHAPE;
    if (!p->use_alpha && p->w_scale_numel != 1 && p->w_scale_numel != p->n) return QA_ERR_SHAPE;
    // 16-byte operand chunks: the same alignment the reference's tensor-core path demands
    if (p->k % 16 != 0 || p->lda % 16 != 0 || p->ldw % 16 != 0 || !aligned16(p->a) || !aligned16(p->w)) return QA_ERR_STRIDE;
    if (p->lda < p->k || p->ldw < p->k || p->ldd < p->n) return QA_ERR_STRIDE;
    if (p->m == 0 || p->n == 0) return QA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t big_tiles = static_cast<int64_t>((p->m + 255) / 256) * ((p->n + 255) / 256);
    if (big_tiles >= 256) return launch_gemm<4, 4>(*p, stream);
    return launch_gemm<2, 2>(*p, stream);
}
