// W8A8 GEMM on the int8 matrix cores with a fused scale epilogue.
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]            (int32, exact)
//   d[m,n]   = cast( s_a[m|0] * ( s_w[n|0] * float(acc) ) )     cast: fp16 RN, or int8 saturating with
//                                                               round-half-even (or half-away for the GEMV rule)
// Reference arithmetic: csrc/linear/quant_linear_fwd_kernel.cuh:63-130 (epilogue :85-109),
// csrc/linear/quant_linear_fwd_gemv_kernel.cuh:56-60 (roundf variant).
// The tiling, LDS layout and epilogue are in gemm_core.hpp.
#include "gemm_core.hpp"

namespace qa {
namespace {

using namespace gemm;

template <int TM, int TN, int WGM, int WGN, int STAGES, int OUT, bool FLEX>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_w8a8_kernel(QaGemmW8A8Params p) {
    using C = Cfg<TM, TN, WGM, WGN, STAGES>;
    constexpr int BM = C::kBM, BN = C::kBN, WAVES = C::kWaves;
    static_assert(epilogue_lds_bytes<TM, TN, WAVES>() <= C::kLdsBytes, "epilogue staging does not fit");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    // consecutive workgroups walk down m first so that neighbours share the same weight tile
    const int tiles_m = (p.m + BM - 1) / BM;
    const int m0 = (blockIdx.x % tiles_m) * BM;
    const int n0 = (blockIdx.x / tiles_m) * BN;

    const v4i rsrc_a = make_rsrc(p.a, static_cast<int>((static_cast<int64_t>(p.m) - 1) * p.lda + p.k));
    const v4i rsrc_w = make_rsrc(p.w, static_cast<int>((static_cast<int64_t>(p.n) - 1) * p.ldw + p.k));
    const uint32_t lds_base = lds_offset_of(lds);

    TileLoader<C::kAInstr> load_a;
    TileLoader<C::kWInstr> load_w;
    load_a.template init<WAVES>(m0, p.m, p.lda, wave, lane);
    load_w.template init<WAVES>(n0, p.n, p.ldw, wave, lane);

    v16i acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int k_tiles = (p.k + kBK - 1) / kBK;
    auto issue = [&](int tile) {
        const uint32_t base = lds_base + (tile % STAGES) * C::kStageBytes;
        load_a.template issue<WAVES>(rsrc_a, tile * kBK, p.k, base, wave);
        load_w.template issue<WAVES>(rsrc_w, tile * kBK, p.k, base + BM * kBK, wave);
    };
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s);

    const int frow = lane & 31, fhalf = lane >> 5;
    for (int kt = 0; kt < k_tiles; ++kt) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * (C::kAInstr + C::kWInstr)));
        __syncthreads();
        issue(kt + STAGES - 1);          // past the end: every lane is out of range and stores zeros
        const uint8_t* stage = lds + (kt % STAGES) * C::kStageBytes;
        mma_tile<TM, TN>(stage + (wm * TM * 32) * kBK, stage + BM * kBK + (wn * TN * 32) * kBK, frow, fhalf, acc);
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    Epilogue e;
    e.row_scale = p.a_scale; e.col_scale = p.w_scale;
    e.row_numel = p.a_scale_numel; e.col_numel = p.w_scale_numel;
    e.use_alpha = p.use_alpha; e.alpha = p.alpha; e.round_mode = p.round_mode;
    e.ldd = p.ldd; e.d = p.d;
    epilogue<TM, TN, OUT, FLEX, false>(e, acc, lds, p.m, p.n, m0 + wm * TM * 32, n0 + wn * TN * 32, wave, lane);
}

template <int TM, int TN, int WGM, int WGN, int STAGES, int OUT, bool FLEX>
int launch_one(const QaGemmW8A8Params& p, hipStream_t stream) {
    using C = Cfg<TM, TN, WGM, WGN, STAGES>;
    const int64_t tiles = static_cast<int64_t>((p.m + C::kBM - 1) / C::kBM) * ((p.n + C::kBN - 1) / C::kBN);
    if (tiles > 0x7fffffffLL) return QA_ERR_SHAPE;
    auto kernel = gemm_w8a8_kernel<TM, TN, WGM, WGN, STAGES, OUT, FLEX>;
    if (C::kLdsBytes > 65536) {
        // allowing more than 64 KiB of dynamic LDS is a per-function attribute; setting it is idempotent
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                C::kLdsBytes) != hipSuccess) {
            return check_launch();
        }
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(C::kThreads), C::kLdsBytes, stream, p);
    return check_launch();
}

template <int TM, int TN, int WGM, int WGN, int STAGES, bool FLEX>
int launch_gemm(const QaGemmW8A8Params& p, hipStream_t stream) {
    return p.out_type == QA_OUT_I8 ? launch_one<TM, TN, WGM, WGN, STAGES, QA_OUT_I8, FLEX>(p, stream)
                                   : launch_one<TM, TN, WGM, WGN, STAGES, QA_OUT_F16, FLEX>(p, stream);
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
    // operands are addressed with 32-bit byte offsets inside a buffer descriptor
    if (static_cast<int64_t>(p->m) * p->lda >= 0x70000000LL || static_cast<int64_t>(p->n) * p->ldw >= 0x70000000LL) return QA_ERR_SHAPE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    // the single-row rules (host alpha, round-half-away) only ever come with tiny M
    if (p->use_alpha || p->round_mode != QA_ROUND_RNE) return launch_gemm<2, 2, 2, 2, 2, true>(*p, stream);
    const int64_t big_tiles = static_cast<int64_t>((p->m + 255) / 256) * ((p->n + 255) / 256);
    if (big_tiles >= 192) {
        // One workgroup per CU at a time: the launch runs in rounds of `cus` tiles, so a tile count
        // just above a multiple of the CU count wastes most of a round.  A 256x320 tile (same 8 waves,
        // 64x160 each) is taken when it needs fewer tile-rounds' worth of arithmetic.
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
            cus = 256;
        }
        auto cost = [&](int64_t bm, int64_t bn) {
            const int64_t tiles = ((p->m + bm - 1) / bm) * ((p->n + bn - 1) / bn);
            return ((tiles + cus - 1) / cus) * bm * bn;
        };
        if (cost(256, 320) < cost(256, 256)) return launch_gemm<2, 5, 4, 2, 2, false>(*p, stream);
        return launch_gemm<4, 2, 2, 4, 2, false>(*p, stream);                        // 256x256 tile, 8 waves
    }
    return launch_gemm<2, 2, 2, 2, 2, false>(*p, stream);                            // 128x128 tile, 4 waves
}
