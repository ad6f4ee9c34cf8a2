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
// subtracting 1032 gives c-8 exactly; one packed FMA with the group scale and the constant 1280
// leaves rne((c-8)*s) as a two's-complement byte in the low byte of each half; v_perm gathers four
// of them.  Everything else is the shared core in gemm_core.hpp.
#include "gemm_core.hpp"

namespace qa {
namespace {

using namespace gemm;

__device__ __forceinline__ uint32_t h2_bits(__half2 v) { return *reinterpret_cast<uint32_t*>(&v); }
__device__ __forceinline__ __half2 bits_h2(uint32_t v) { return *reinterpret_cast<__half2*>(&v); }

// (x & mask) | bits in one instruction; `bits` is held in a vector register because the encoding
// takes a single scalar or literal operand.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(bits));
    return r;
}

// 8 codes (one word) -> 8 int8 in k order (two words), grouped mode.  The rounding constant 1280
// (ulp 1, a multiple of 256) leaves the two's-complement byte of rne((c-8)*s) in the low byte.
__device__ __forceinline__ uint2 expand_grouped(uint32_t p, __half2 s2) {
    const __half2 k1032 = bits_h2(0x64086408u);      // 1032, 1032
    const __half2 k16th = bits_h2(0x2c002c00u);      // 1/16
    const __half2 km72 = bits_h2(0xd480d480u);       // -72
    const __half2 k1280 = bits_h2(0x65006500u);      // 1280
    const uint32_t kOne = 0x64006400u;               // 1024, 1024
    const uint32_t q = p >> 8;
    const __half2 a = __hsub2(bits_h2(and_or(p, 0x000f000fu, kOne)), k1032);            // c0-8, c2-8
    const __half2 b = __hfma2(bits_h2(and_or(p, 0x00f000f0u, kOne)), k16th, km72);      // c4-8, c6-8
    const __half2 c = __hsub2(bits_h2(and_or(q, 0x000f000fu, kOne)), k1032);            // c1-8, c3-8
    const __half2 d = __hfma2(bits_h2(and_or(q, 0x00f000f0u, kOne)), k16th, km72);      // c5-8, c7-8
    const uint32_t ra = h2_bits(__hfma2(a, s2, k1280)), rb = h2_bits(__hfma2(b, s2, k1280));
    const uint32_t rc = h2_bits(__hfma2(c, s2, k1280)), rd = h2_bits(__hfma2(d, s2, k1280));
    uint2 out;
    out.x = __builtin_amdgcn_perm(rc, ra, 0x06020400u);    // k0 k1 k2 k3
    out.y = __builtin_amdgcn_perm(rd, rb, 0x06020400u);    // k4 k5 k6 k7
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
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    int tile_m, tile_n;
    tile_of_workgroup<BM, BN>(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
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
        if (more) load_w(kt + 1);
        const uint8_t* stage = lds + (kt & 1) * C::kStageBytes;
        // the activation requests for the next tile go out one at a time between the multiplications
        const uint32_t nbase = lds_base + ((kt + 1) & 1) * C::kStageBytes;
        static_assert(C::kAInstr <= 4 * TM * TN / 2, "more requests than slots");
        mma_tile_paced<TM, TN>(stage + (wm * TM * 32) * kBK, stage + BM * kBK + (wn * TN * 32) * kBK, frow, fhalf, acc,
                               [&](int slot) {
                                   if (slot < C::kAInstr) load_a.template issue_one<WAVES>(slot, rsrc_a, (kt + 1) * kBK, p.k, nbase, wave);
                               });
        if (more) store_w((kt + 1) & 1);
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    Epilogue e;
    e.row_scale = p.s_token; e.col_scale = p.s_channel;
    e.row_numel = p.tok_scale_numel; e.col_numel = p.n;
    e.use_alpha = 0; e.alpha = 0.0f; e.round_mode = QA_ROUND_RNE; e.col_outer = 0;
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

// ---------------------------------------------------------------------------------------------
// Few activation rows (M <= 64, the decode step): a stream over the packed weights.  A workgroup
// owns 32 output columns and all rows; its WAVES waves split K between them in interleaved pieces
// of 256 codes, i.e. one full 128-byte line of packed weights per row.  A wave fetches a piece with
// eight lanes per row (DEPTH pieces in flight in registers), expands its 32 codes per lane to int8
// and passes them through a staging area in LDS that is private to the wave; the activation tiles
// take the same route, one 128-byte half at a time.  Partial sums meet in LDS at the end.
// ---------------------------------------------------------------------------------------------
template <int TM, int AI, int WAVES, int DEPTH, int OUT, bool TRANS>
__global__ __launch_bounds__(64 * WAVES) void gemm_w4a8_skinny_kernel(QaGemmW4A8Params p) {
    constexpr int kThreads = 64 * WAVES;
    constexpr int kOob = 0x7ffffff0;                       // beyond any buffer: the load returns zeros
    constexpr int kTile = 32 * kBK;
    constexpr int kPiece = 2 * kBK;                        // codes per row and piece
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int* red = reinterpret_cast<int*>(lds + WAVES * (2 + TM) * kTile);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, fhalf = lane >> 5;
    const int n0 = blockIdx.x * 32;
    const bool grouped = p.group_size > 0;
    for (int i = tid; i < TM * 16 * 64; i += kThreads) red[i] = 0;
    uint8_t* stage = lds + wave * ((2 + TM) * kTile);          // two weight halves, TM activation tiles
    if (AI < 4) {
        // only the first 8*AI rows of an activation tile are ever fetched (M <= 8*AI): the rest stays zero
        for (int i = lane; i < TM * kTile / 16; i += 64) reinterpret_cast<v4u*>(stage + 2 * kTile)[i] = v4u{0u, 0u, 0u, 0u};
    }

    const int ldw = p.k / 2;
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.w_packed), 0, static_cast<int>(static_cast<int64_t>(p.n) * ldw), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.a), 0, static_cast<int>((static_cast<int64_t>(p.m) - 1) * p.lda + p.k), kRsrcFlags);
    // fetch mapping: instruction i, lane l -> tile row 8i + l/8, 16-byte chunk l%8.  A packed chunk is
    // 32 codes: chunks 0..3 expand into the first 128-code half of the piece, 4..7 into the second.
    const int lrow = lane >> 3, lchunk = lane & 7;
    const int my_half = lchunk >> 2, my_c0 = (lchunk & 3) * 2;
    int w_off[4], a_off[TM][AI], s_col[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = n0 + 8 * i + lrow;
        w_off[i] = row < p.n ? row * ldw + lchunk * 16 : -1;
        s_col[i] = min(row, p.n - 1);
        if (i < AI) {
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int arow = j * 32 + 8 * i + lrow;
                a_off[j][i] = arow < p.m ? static_cast<int>(arow * p.lda) + lchunk * 16 : -1;
            }
        }
    }
    const __half* sg = static_cast<const __half*>(p.s_group);
    const int n_groups = p.k / kBK;

    const int pieces = (p.k + kPiece - 1) / kPiece;
    const int my_pieces = (pieces - wave + WAVES - 1) / WAVES;
    v4u fw[DEPTH][4], fa[DEPTH][2][TM][AI];
    __half fs[DEPTH][4];
    auto load = [&](int i_piece, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const int k0 = (wave + i_piece * WAVES) * kPiece;
        const bool w_ok = k0 + lchunk * 32 < p.k;
        const int group = min(k0 / kBK + my_half, n_groups - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            fw[buf][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, (w_ok && w_off[i] >= 0) ? w_off[i] + k0 / 2 : kOob, 0, 0);
            if (grouped) fs[buf][i] = sg[static_cast<int64_t>(group) * p.n + s_col[i]];
            if (i < AI) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const bool a_k_ok = k0 + h * kBK + lchunk * 16 < p.k;
#pragma unroll
                    for (int j = 0; j < TM; ++j) {
                        fa[buf][h][j][i] = __builtin_amdgcn_raw_buffer_load_b128(
                            rsrc_a, (a_k_ok && a_off[j][i] >= 0) ? a_off[j][i] + k0 + h * kBK : kOob, 0, 0);
                    }
                }
            }
        }
    };

    v16i acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;

    static_for<0, DEPTH - 1>([&](auto s) {
        if (decltype(s)::value < my_pieces) load(decltype(s)::value, s);
    });
    for (int base = 0; base < my_pieces; base += DEPTH) {
        static_for<0, DEPTH>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            if (base + s + DEPTH - 1 < my_pieces) load(base + s + DEPTH - 1, std::integral_constant<int, (s + DEPTH - 1) % DEPTH>{});
            if (base + s < my_pieces) {
                // expand this lane's 32 codes per fetched row into its half of the staged weights
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t w[4] = {fw[s][i].x, fw[s][i].y, fw[s][i].z, fw[s][i].w};
                    uint2 e[4];
                    if (grouped) {
                        const __half2 s2 = __half2half2(fs[s][i]);
#pragma unroll
                        for (int t = 0; t < 4; ++t) e[t] = expand_grouped(w[t], s2);
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t) e[t] = expand_per_channel(w[t]);
                    }
                    const int row = 8 * i + lrow;
                    uint8_t* dst = stage + my_half * kTile + row * kBK;
                    *reinterpret_cast<v4u*>(dst + swz(row, my_c0) * 16) = v4u{e[0].x, e[0].y, e[1].x, e[1].y};
                    *reinterpret_cast<v4u*>(dst + swz(row, my_c0 + 1) * 16) = v4u{e[2].x, e[2].y, e[3].x, e[3].y};
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int i = 0; i < AI; ++i) {
                        const int row = 8 * i + lrow;
#pragma unroll
                        for (int j = 0; j < TM; ++j)
                            *reinterpret_cast<v4u*>(stage + (2 + j) * kTile + row * kBK + swz(row, lchunk) * 16) = fa[s][h][j][i];
                    }
                    wave_lds_sync();
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        const int off = frow * kBK + swz(frow, kk * 2 + fhalf) * 16;
                        const v4i bw = *reinterpret_cast<const v4i*>(stage + h * kTile + off);
#pragma unroll
                        for (int j = 0; j < TM; ++j) {
                            const v4i ba = *reinterpret_cast<const v4i*>(stage + (2 + j) * kTile + off);
                            acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw, ba, acc[j], 0, 0, 0);
                        }
                    }
                    wave_lds_sync();
                }
            }
        });
    }

    Epilogue e;
    e.row_scale = p.s_token; e.col_scale = p.s_channel;
    e.row_numel = p.tok_scale_numel; e.col_numel = p.n;
    e.use_alpha = 0; e.alpha = 0.0f; e.round_mode = QA_ROUND_RNE; e.col_outer = 0;
    e.ldd = p.ldd; e.d = p.d;
    skinny_reduce_store<TM, OUT, false, TRANS>(e, acc, red, p.m, p.n, n0, tid, kThreads);
}

template <int TM, int AI, int WAVES, int DEPTH, int OUT, bool TRANS>
int launch_skinny_one(const QaGemmW4A8Params& p, hipStream_t stream) {
    constexpr int kLds = skinny_lds_bytes<TM + 1, WAVES>() - 16 * 64 * 4;   // (2 + TM) tiles per wave, TM reduction blocks
    auto kernel = gemm_w4a8_skinny_kernel<TM, AI, WAVES, DEPTH, OUT, TRANS>;
    if (kLds > 65536) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kLds) != hipSuccess) {
            return check_launch();
        }
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>((p.n + 31) / 32)), dim3(64 * WAVES), kLds, stream, p);
    return check_launch();
}

template <int TM, int AI, int WAVES, int DEPTH>
int launch_skinny(const QaGemmW4A8Params& p, hipStream_t stream) {
    if (p.out_type == QA_OUT_I8) {
        return p.output_transpose ? launch_skinny_one<TM, AI, WAVES, DEPTH, QA_OUT_I8, true>(p, stream)
                                  : launch_skinny_one<TM, AI, WAVES, DEPTH, QA_OUT_I8, false>(p, stream);
    }
    return p.output_transpose ? launch_skinny_one<TM, AI, WAVES, DEPTH, QA_OUT_F16, true>(p, stream)
                              : launch_skinny_one<TM, AI, WAVES, DEPTH, QA_OUT_F16, false>(p, stream);
}

int dispatch_skinny(const QaGemmW4A8Params& p, hipStream_t stream) {
    // four waves per workgroup once the columns give a workgroup per CU, else eight when K is long enough
    const bool wide = (p.n + 31) / 32 < 256 && p.k >= 16 * 2 * kBK;
    // activation rows are fetched eight at a time: up to 8 rows need one fetch per tile, up to 32 four
    if (p.m <= 8) return wide ? launch_skinny<1, 1, 8, 3>(p, stream) : launch_skinny<1, 1, 4, 3>(p, stream);
    if (p.m <= 32) return wide ? launch_skinny<1, 4, 8, 2>(p, stream) : launch_skinny<1, 4, 4, 2>(p, stream);
    // two row blocks: a wave's registers allow one workgroup of eight waves or two of four per CU, and
    // eight waves measured faster whenever K has at least two pieces per wave
    return (wide || p.k >= 16 * 2 * kBK) ? launch_skinny<2, 4, 8, 2>(p, stream) : launch_skinny<2, 4, 4, 2>(p, stream);
}

// ---------------------------------------------------------------------------------------------
// The weights expanded to int8 once: w8 (N, K) row-major, the layout the int8 x int8 kernel reads.
// One thread = 32 codes (16 packed bytes in, 32 bytes out), with the same expansion as the fused kernel.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void w4_expand_kernel(QaGemmW4A8Params p, int8_t* w8) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int per_row = p.k / 32;
    if (idx >= static_cast<int64_t>(p.n) * per_row) return;
    const int n = static_cast<int>(idx / per_row), piece = static_cast<int>(idx % per_row);
    const uint4 v = *reinterpret_cast<const uint4*>(p.w_packed + static_cast<int64_t>(n) * (p.k / 2) + piece * 16);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint2 e[4];
    if (p.group_size > 0) {
        const __half sc = static_cast<const __half*>(p.s_group)[static_cast<int64_t>(piece / 4) * p.n + n];
        const __half2 s2 = __half2half2(sc);
#pragma unroll
        for (int t = 0; t < 4; ++t) e[t] = expand_grouped(w[t], s2);
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) e[t] = expand_per_channel(w[t]);
    }
    int8_t* dst = w8 + static_cast<int64_t>(n) * p.k + piece * 32;
    *reinterpret_cast<uint4*>(dst) = make_uint4(e[0].x, e[0].y, e[1].x, e[1].y);
    *reinterpret_cast<uint4*>(dst + 16) = make_uint4(e[2].x, e[2].y, e[3].x, e[3].y);
}

}  // namespace
}  // namespace qa

extern "C" int qa_gemm_w4a8(const QaGemmW4A8Params* p, void* stream_) {
    using namespace qa;
    if (!p) return QA_ERR_NULL;
    if (p->m < 0 || p->n < 0 || p->k < 0) return QA_ERR_SHAPE;
    const bool empty = p->m == 0 || p->n == 0;                      // (an output without elements: tensors may be null)
    if (!empty && (!p->a || !p->w_packed || !p->s_channel || !p->s_token || !p->d)) return QA_ERR_NULL;
    if (p->group_size != 128 && p->group_size != -1) return QA_ERR_UNSUPPORTED;
    if (!empty && p->group_size == 128 && !p->s_group) return QA_ERR_NULL;
    if (p->out_type != QA_OUT_I8 && p->out_type != QA_OUT_F16) return QA_ERR_UNSUPPORTED;
    if (p->tok_scale_numel != 1 && p->tok_scale_numel != p->m) return QA_ERR_SHAPE;
    if (p->k % 128 != 0) return QA_ERR_SHAPE;                       // whole 128-code groups / k tiles
    if (p->lda % 16 != 0 || p->lda < p->k || !aligned16(p->a) || !aligned16(p->w_packed)) return QA_ERR_STRIDE;
    if (p->ldd < (p->output_transpose ? p->m : p->n)) return QA_ERR_STRIDE;
    if (p->m == 0 || p->n == 0) return QA_OK;
    if (static_cast<int64_t>(p->m) * p->lda >= 0x70000000LL) return QA_ERR_SHAPE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (p->m <= 64 && static_cast<int64_t>(p->n) * (p->k / 2) < 0x70000000LL) return dispatch_skinny(*p, stream);
    const int64_t w8_bytes = static_cast<int64_t>(p->n) * p->k;
    if (p->w8_workspace && p->w8_workspace_bytes >= w8_bytes && aligned16(p->w8_workspace) && w8_bytes < 0x70000000LL &&
        (!p->output_transpose || p->n > 64)) {
        int8_t* w8 = static_cast<int8_t*>(p->w8_workspace);
        const int64_t threads = static_cast<int64_t>(p->n) * (p->k / 32);
        hipLaunchKernelGGL(w4_expand_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream, *p, w8);
        // (acc * s_channel[n]) * s_token[m] and s_token[m] * (s_channel[n] * acc) round the same two products
        QaGemmW8A8Params q = {};
        q.k = p->k; q.ldd = p->ldd; q.d = p->d;
        q.out_type = p->out_type;
        q.round_mode = QA_ROUND_RNE;
        if (!p->output_transpose) {
            q.m = p->m; q.n = p->n;
            q.lda = p->lda; q.ldw = p->k;
            q.a = p->a; q.w = w8;
            q.a_scale = p->s_token; q.a_scale_numel = p->tok_scale_numel;
            q.w_scale = p->s_channel; q.w_scale_numel = p->n;
        } else {
            // the (N,M) output is the product with the operands' roles exchanged; the column scale (the
            // token's) is then applied last, which keeps the association s_token * (s_channel * acc)
            q.m = p->n; q.n = p->m;
            q.lda = p->k; q.ldw = p->lda;
            q.a = w8; q.w = p->a;
            q.a_scale = p->s_channel; q.a_scale_numel = p->n;
            q.w_scale = p->s_token; q.w_scale_numel = p->tok_scale_numel;
            q.scale_order = 1;
        }
        return qa_gemm_w8a8(&q, stream_);
    }
    const int64_t big_tiles = static_cast<int64_t>((p->m + 255) / 256) * ((p->n + 255) / 256);
    if (big_tiles >= 192) return launch_gemm<4, 2, 2, 4>(*p, stream);
    return launch_gemm<2, 2, 2, 2>(*p, stream);
}
