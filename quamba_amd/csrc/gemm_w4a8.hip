// W4A8 GEMM: int8 activations x 4-bit weights with group-wise (128) fp16 scales or per-channel
// scaling, on the int8 matrix cores.
//
//   grouped:      w8[n,k] = int8( rne( (code - 8) * s_group[k/128, n] ) )      one fp16 FMA, one rounding
//   per-channel:  w8[n,k] = 16 * signed_nibble(code)
//   acc[m,n] = sum_k a[m,k] * w8[n,k] (int32);  d = cast( (float(acc) * s_channel[n]) * s_token[m|0] )
// Reference arithmetic: csrc/linear/marlin_qqq_gemm_kernel.cuh:125-178 (dequant), :744-749 (fp16
// epilogue), marlin_qqq_gemm_kernel_o8.cuh:107-116 (int8 epilogue, round-half-even saturating).
//
// Weight storage (this library's own): uint8 (N, K/2).  Each aligned group of 8 codes of a row is
// one 32-bit word whose byte i holds code[8w+i] in the low nibble and code[8w+4+i] in the high
// nibble, so that the fp16 exponent trick below yields the int8 bytes in k order.
// The expansion to int8 runs in registers on the way from global memory to LDS (once per
// workgroup, not once per wave): (word & 0x000f000f) | 0x6400_6400 is the half2 (1024+c0, 1024+c2);
// subtracting 1032 gives c-8 exactly; one packed FMA with the group scale and the constant 1152
// leaves rne((c-8)*s) + 128 in the low byte of each half; v_perm gathers four bytes and an XOR with
// 0x80 turns them into int8.  Everything else is the shared core in gemm_core.hpp.
#include "gemm_core.hpp"

namespace qa {
namespace {

using namespace gemm;

__device__ __forceinline__ uint32_t h2_bits(__half2 v) { return *reinterpret_cast<uint32_t*>(&v); }
__device__ __forceinline__ __half2 bits_h2(uint32_t v) { return *reinterpret_cast<__half2*>(&v); }

// 8 codes (one word) -> 8 int8 in k order (two words), grouped mode.
__device__ __forceinline__ uint2 expand_grouped(uint32_t p, __half2 s2) {
    const __half2 k1032 = bits_h2(0x64086408u);      // 1032, 1032
    const __half2 k16th = bits_h2(0x2c002c00u);      // 1/16
    const __half2 km72 = bits_h2(0xd480d480u);       // -72
    const __half2 k1152 = bits_h2(0x64806480u);      // 1152
    const uint32_t q = p >> 8;
    const __half2 a = __hsub2(bits_h2((p & 0x000f000fu) | 0x64006400u), k1032);            // c0-8, c2-8
    const __half2 b = __hfma2(bits_h2((p & 0x00f000f0u) | 0x64006400u), k16th, km72);      // c4-8, c6-8
    const __half2 c = __hsub2(bits_h2((q & 0x000f000fu) | 0x64006400u), k1032);            // c1-8, c3-8
    const __half2 d = __hfma2(bits_h2((q & 0x00f000f0u) | 0x64006400u), k16th, km72);      // c5-8, c7-8
    const uint32_t ra = h2_bits(__hfma2(a, s2, k1152)), rb = h2_bits(__hfma2(b, s2, k1152));
    const uint32_t rc = h2_bits(__hfma2(c, s2, k1152)), rd = h2_bits(__hfma2(d, s2, k1152));
    uint2 out;
    out.x = __builtin_amdgcn_perm(rc, ra, 0x06020400u) ^ 0x80808080u;    // k0 k1 k2 k3
    out.y = __builtin_amdgcn_perm(rd, rb, 0x06020400u) ^ 0x80808080u;    // k4 k5 k6 k7
    return out;
}

__device__ __forceinline__ uint2 expand_per_channel(uint32_t p) {
    uint2 out;
    out.x = (p << 4) & 0xf0f0f0f0u;
    out.y = p & 0xf0f0f0f0u;
    return out;
}

template <int TM, int TN, int WGM, int WGN, int OUT, bool TRANS>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_w4a8_kernel(QaGemmW4A8Params p) {
    constexpr int STAGES = 2;
    using C = Cfg<TM, TN, WGM, WGN, STAGES>;
    constexpr int BM = C::kBM, BN = C::kBN, WAVES = C::kWaves, THREADS = C::kThreads;
    constexpr int kWPacked = BN * 4 / THREADS;      // 16-byte packed chunks (32 codes) per thread per tile
    static_assert(epilogue_lds_bytes<TM, TN, WAVES>() <= C::kLdsBytes, "epilogue staging does not fit");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int tiles_m = (p.m + BM - 1) / BM;
    const int m0 = (blockIdx.x % tiles_m) * BM;
    const int n0 = (blockIdx.x / tiles_m) * BN;
    const bool grouped = p.group_size > 0;

    const v4i rsrc_a = make_rsrc(p.a, static_cast<int>((static_cast<int64_t>(p.m) - 1) * p.lda + p.k));
    const uint32_t lds_base = lds_offset_of(lds);
    TileLoader<C::kAInstr> load_a;
    load_a.template init<WAVES>(m0, p.m, p.lda, wave, lane);

    // this thread's packed chunks of the weight tile: (row, 32-code quarter)
    const int64_t ldw = p.k / 2;
    const uint8_t* w_src[kWPacked];
    int w_row[kWPacked], w_quarter[kWPacked];
#pragma unroll
    for (int i = 0; i < kWPacked; ++i) {
        const int id = tid + i * THREADS;
        w_row[i] = id >> 2;
        w_quarter[i] = id & 3;
        const int nn = min(n0 + w_row[i], p.n - 1);
        w_src[i] = p.w_packed + nn * ldw + w_quarter[i] * 16;
    }
    const __half* sg = static_cast<const __half*>(p.s_group);

    uint4 wreg[kWPacked];
    __half wscale[kWPacked];
    auto load_w = [&](int tile) {
#pragma unroll
        for (int i = 0; i < kWPacked; ++i) {
            wreg[i] = *reinterpret_cast<const uint4*>(w_src[i] + static_cast<int64_t>(tile) * (kBK / 2));
            if (grouped) wscale[i] = sg[static_cast<int64_t>(tile) * p.n + min(n0 + w_row[i], p.n - 1)];
        }
    };
    auto store_w = [&](int stage) {
        uint8_t* sw = lds + stage * C::kStageBytes + BM * kBK;
#pragma unroll
        for (int i = 0; i < kWPacked; ++i) {
            const uint32_t w[4] = {wreg[i].x, wreg[i].y, wreg[i].z, wreg[i].w};
            uint2 e[4];
            if (grouped) {
                const __half2 s2 = __half2half2(wscale[i]);
#pragma unroll
                for (int t = 0; t < 4; ++t) e[t] = expand_grouped(w[t], s2);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) e[t] = expand_per_channel(w[t]);
            }
            const int row = w_row[i], c0 = w_quarter[i] * 2;
            *reinterpret_cast<uint4*>(sw + row * kBK + swz(row, c0) * 16) = make_uint4(e[0].x, e[0].y, e[1].x, e[1].y);
            *reinterpret_cast<uint4*>(sw + row * kBK + swz(row, c0 + 1) * 16) = make_uint4(e[2].x, e[2].y, e[3].x, e[3].y);
        }
    };

    v16i acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int k_tiles = p.k / kBK;
    load_a.template issue<WAVES>(rsrc_a, 0, p.k, lds_base, wave);
    if (k_tiles > 0) {
        load_w(0);
        store_w(0);
    }
    const int frow = lane & 31, fhalf = lane >> 5;
    for (int kt = 0; kt < k_tiles; ++kt) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();
        const bool more = kt + 1 < k_tiles;
        load_a.template issue<WAVES>(rsrc_a, (kt + 1) * kBK, p.k, lds_base + ((kt + 1) & 1) * C::kStageBytes, wave);
        if (more) load_w(kt + 1);
        const uint8_t* stage = lds + (kt & 1) * C::kStageBytes;
        mma_tile<TM, TN>(stage + (wm * TM * 32) * kBK, stage + BM * kBK + (wn * TN * 32) * kBK, frow, fhalf, acc);
        if (more) store_w((kt + 1) & 1);
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    Epilogue e;
    e.row_scale = p.s_token; e.col_scale = p.s_channel;
    e.row_numel = p.tok_scale_numel; e.col_numel = p.n;
    e.use_alpha = 0; e.alpha = 0.0f; e.round_mode = QA_ROUND_RNE;
    e.ldd = p.ldd; e.d = p.d;
    epilogue<TM, TN, OUT, false, TRANS>(e, acc, lds, p.m, p.n, m0 + wm * TM * 32, n0 + wn * TN * 32, wave, lane);
}

template <int TM, int TN, int WGM, int WGN, int OUT, bool TRANS>
int launch_one(const QaGemmW4A8Params& p, hipStream_t stream) {
    using C = Cfg<TM, TN, WGM, WGN, 2>;
    const int64_t tiles = static_cast<int64_t>((p.m + C::kBM - 1) / C::kBM) * ((p.n + C::kBN - 1) / C::kBN);
    if (tiles > 0x7fffffffLL) return QA_ERR_SHAPE;
    auto kernel = gemm_w4a8_kernel<TM, TN, WGM, WGN, OUT, TRANS>;
    if (C::kLdsBytes > 65536) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                C::kLdsBytes) != hipSuccess) {
            return check_launch();
        }
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(C::kThreads), C::kLdsBytes, stream, p);
    return check_launch();
}

template <int TM, int TN, int WGM, int WGN>
int launch_gemm(const QaGemmW4A8Params& p, hipStream_t stream) {
    if (p.out_type == QA_OUT_I8) {
        return p.output_transpose ? launch_one<TM, TN, WGM, WGN, QA_OUT_I8, true>(p, stream)
                                  : launch_one<TM, TN, WGM, WGN, QA_OUT_I8, false>(p, stream);
    }
    return p.output_transpose ? launch_one<TM, TN, WGM, WGN, QA_OUT_F16, true>(p, stream)
                              : launch_one<TM, TN, WGM, WGN, QA_OUT_F16, false>(p, stream);
}

}  // namespace
}  // namespace qa

extern "C" int qa_gemm_w4a8(const QaGemmW4A8Params* p, void* stream_) {
    using namespace qa;
    if (!p || !p->a || !p->w_packed || !p->s_channel || !p->s_token || !p->d) return QA_ERR_NULL;
    if (p->m < 0 || p->n < 0 || p->k < 0) return QA_ERR_SHAPE;
    if (p->group_size != 128 && p->group_size != -1) return QA_ERR_UNSUPPORTED;
    if (p->group_size == 128 && !p->s_group) return QA_ERR_NULL;
    if (p->out_type != QA_OUT_I8 && p->out_type != QA_OUT_F16) return QA_ERR_UNSUPPORTED;
    if (p->tok_scale_numel != 1 && p->tok_scale_numel != p->m) return QA_ERR_SHAPE;
    if (p->k % 128 != 0) return QA_ERR_SHAPE;                       // whole 128-code groups / k tiles
    if (p->lda % 16 != 0 || p->lda < p->k || !aligned16(p->a) || !aligned16(p->w_packed)) return QA_ERR_STRIDE;
    if (p->ldd < (p->output_transpose ? p->m : p->n)) return QA_ERR_STRIDE;
    if (p->m == 0 || p->n == 0) return QA_OK;
    if (static_cast<int64_t>(p->m) * p->lda >= 0x70000000LL) return QA_ERR_SHAPE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t big_tiles = static_cast<int64_t>((p->m + 255) / 256) * ((p->n + 255) / 256);
    if (big_tiles >= 192) return launch_gemm<4, 2, 2, 4>(*p, stream);
    return launch_gemm<2, 2, 2, 2>(*p, stream);
}
