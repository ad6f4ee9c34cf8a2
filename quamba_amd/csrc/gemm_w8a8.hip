// W8A8 GEMM on the int8 matrix cores with a fused scale epilogue.
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]            (int32, exact)
//   d[m,n]   = cast( s_a[m|0] * ( s_w[n|0] * float(acc) ) )     cast: fp16 RN, or int8 saturating with
//                                                               round-half-even (or half-away for the GEMV rule)
// Reference arithmetic: csrc/linear/quant_linear_fwd_kernel.cuh:63-130 (epilogue :85-109),
// csrc/linear/quant_linear_fwd_gemv_kernel.cuh:56-60 (roundf variant).
// The tiling, LDS layout and epilogue are in gemm_core.hpp.
#include "gemm_core.hpp"

// Built with -DQA_GEMM_CLK (bench.py --gemm-phase-clocks, never the product library) thread 0 of every workgroup of
// the tiled kernel records the shader clock and the constant 100 MHz clock at four points - start, first fragments
// in registers, end of the main loop, end of the epilogue - and qa_gemm_clk_read copies the table out.
#ifdef QA_GEMM_CLK
__device__ unsigned long long g_gemm_clk[8192][8];
extern "C" int qa_gemm_clk_read(void* dst, int64_t bytes) {     // copies the table out and clears it
    if (bytes != static_cast<int64_t>(sizeof(g_gemm_clk))) return QA_ERR_SHAPE;
    void* table = nullptr;
    if (hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_gemm_clk), sizeof(g_gemm_clk)) != hipSuccess) return QA_ERR_LAUNCH;
    if (hipGetSymbolAddress(&table, HIP_SYMBOL(g_gemm_clk)) != hipSuccess) return QA_ERR_LAUNCH;
    return hipMemset(table, 0, sizeof(g_gemm_clk)) == hipSuccess ? QA_OK : QA_ERR_LAUNCH;
}
#define CLK_MARK(i)                                                 \
    do {                                                            \
        if (threadIdx.x == 0 && blockIdx.x < 8192) {                \
            g_gemm_clk[blockIdx.x][2 * (i)] = clock64();            \
            g_gemm_clk[blockIdx.x][2 * (i) + 1] = wall_clock64();   \
        }                                                           \
    } while (0)
#else
#define CLK_MARK(i)
#endif

namespace qa {
namespace {

using namespace gemm;

template <int TM, int TN, int WGM, int WGN, int STAGES, int OUT, bool FLEX, bool COL_OUTER>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_w8a8_kernel(QaGemmW8A8Params p) {
    using C = Cfg<TM, TN, WGM, WGN, STAGES>;
    constexpr int BM = C::kBM, BN = C::kBN, WAVES = C::kWaves;
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
    const int frow = lane & 31, fhalf = lane >> 5;
    CLK_MARK(0);
    if constexpr (STAGES == 2) {
        // Two stages, the barrier before the last k step of a tile (mma_tile_rotated).  The requests for a tile go
        // out one at a time behind every second multiplication, counted from that barrier: the ones that fit into
        // the last k step of tile t - 2, the rest during the first three steps of tile t - 1.  Past the end of K
        // every lane is out of range and stores zeros.
        constexpr int kReq = C::kAInstr + C::kWInstr, kPerStep = TM * TN;
        constexpr int kEarly = kPerStep / 2 < kReq ? kPerStep / 2 : kReq;      // positions inside the last k step
        static_assert(kReq <= 4 * kPerStep / 2, "more requests than positions");
        auto request = [&](int r, int tile) {
            const uint32_t base = lds_base + (tile & 1) * C::kStageBytes;
            if (r < C::kAInstr) load_a.template issue_one<WAVES>(r, rsrc_a, tile * kBK, p.k, base, wave);
            else if (r < kReq) load_w.template issue_one<WAVES>(r - C::kAInstr, rsrc_w, tile * kBK, p.k, base + BM * kBK, wave);
        };
#pragma unroll
        for (int r = 0; r < kReq; ++r) request(r, 0);
#pragma unroll
        for (int r = 0; r < kEarly; ++r) request(r, 1);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kEarly));
        __syncthreads();
        const uint8_t* my_a = lds + (wm * TM * 32) * kBK;
        const uint8_t* my_w = lds + BM * kBK + (wn * TN * 32) * kBK;
        v4i fa[2][TM], fw[2][TN];
        fetch_fragments<TM, TN>(my_a, my_w, 0, frow, fhalf, fa[0], fw[0]);
        CLK_MARK(1);
        for (int kt = 0; kt < k_tiles; ++kt) {
            const int cur = (kt & 1) * C::kStageBytes, nxt = C::kStageBytes - cur;
            mma_tile_rotated<TM, TN>(my_a + cur, my_w + cur, my_a + nxt, my_w + nxt, frow, fhalf, fa, fw, acc,
                                     [&](int idx) {
                                         if (idx % 2 != 1) return;
                                         const int r = idx / 2;
                                         request(r, r < kEarly ? kt + 2 : kt + 1);
                                     });
        }
    } else {
    auto issue = [&](int tile) {
        const uint32_t base = lds_base + (tile % STAGES) * C::kStageBytes;
        load_a.template issue<WAVES>(rsrc_a, tile * kBK, p.k, base, wave);
        load_w.template issue<WAVES>(rsrc_w, tile * kBK, p.k, base + BM * kBK, wave);
    };
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s);

    for (int kt = 0; kt < k_tiles; ++kt) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * (C::kAInstr + C::kWInstr)));
        __syncthreads();
        const uint8_t* stage = lds + (kt % STAGES) * C::kStageBytes;
        // the requests for the next tile go out one at a time between the multiplications of this one
        // (past the end of K every lane is out of range and stores zeros)
        const int nt = kt + STAGES - 1;
        const uint32_t nbase = lds_base + (nt % STAGES) * C::kStageBytes;
        static_assert(C::kAInstr + C::kWInstr <= 4 * TM * TN / 2, "more requests than slots");
        mma_tile_paced<TM, TN>(stage + (wm * TM * 32) * kBK, stage + BM * kBK + (wn * TN * 32) * kBK, frow, fhalf, acc,
                               [&](int slot) {
                                   if (slot < C::kAInstr) load_a.template issue_one<WAVES>(slot, rsrc_a, nt * kBK, p.k, nbase, wave);
                                   else if (slot < C::kAInstr + C::kWInstr)
                                       load_w.template issue_one<WAVES>(slot - C::kAInstr, rsrc_w, nt * kBK, p.k, nbase + BM * kBK, wave);
                               });
    }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    CLK_MARK(2);

    Epilogue e;
    e.row_scale = p.a_scale; e.col_scale = p.w_scale;
    e.row_numel = p.a_scale_numel; e.col_numel = p.w_scale_numel;
    e.use_alpha = p.use_alpha; e.alpha = p.alpha; e.round_mode = p.round_mode; e.col_outer = p.scale_order;
    e.ldd = p.ldd; e.d = p.d;
    epilogue<TM, TN, OUT, FLEX, false, COL_OUTER>(e, acc, lds, p.m, p.n, m0 + wm * TM * 32, n0 + wn * TN * 32, wave, lane);
    CLK_MARK(3);
}

template <int TM, int TN, int WGM, int WGN, int STAGES, int OUT, bool FLEX, bool COL_OUTER = false>
int launch_one(const QaGemmW8A8Params& p, hipStream_t stream) {
    using C = Cfg<TM, TN, WGM, WGN, STAGES>;
    if constexpr (!FLEX && !COL_OUTER) {
        if (p.scale_order == 1) return launch_one<TM, TN, WGM, WGN, STAGES, OUT, FLEX, true>(p, stream);
    }
    const int64_t tiles = static_cast<int64_t>((p.m + C::kBM - 1) / C::kBM) * ((p.n + C::kBN - 1) / C::kBN);
    if (tiles > 0x7fffffffLL) return QA_ERR_SHAPE;
    auto kernel = gemm_w8a8_kernel<TM, TN, WGM, WGN, STAGES, OUT, FLEX, COL_OUTER>;
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
    if (p.out_type == QA_OUT_I8) return launch_one<TM, TN, WGM, WGN, STAGES, QA_OUT_I8, FLEX>(p, stream);
    if (p.out_type == QA_OUT_BF16) return launch_one<TM, TN, WGM, WGN, STAGES, QA_OUT_BF16, FLEX>(p, stream);
    return launch_one<TM, TN, WGM, WGN, STAGES, QA_OUT_F16, FLEX>(p, stream);
}

// ---------------------------------------------------------------------------------------------
// Few activation rows (M <= 64, the decode step): the product is a stream over the weight matrix
// and HBM-bound, so the shape of the launch is chosen for memory parallelism rather than reuse.
// A workgroup owns 32 output columns and all rows; its WAVES waves split K between them in
// interleaved 128-byte tiles.  A wave fetches its tiles with eight lanes per 128-byte row piece
// (whole cache lines; fetching MFMA fragments directly would touch 64 lines per instruction),
// DEPTH tiles in flight in registers, and turns a tile into fragments through a staging area in
// LDS that is private to the wave, so the main loop has no workgroup barrier.  The small
// activation matrix takes the same route and is served by the caches.  The partial sums of the
// waves are added in LDS (integers: the order does not matter), then every thread scales and
// writes four consecutive columns of one row.
// ---------------------------------------------------------------------------------------------
template <int TM, int WAVES, int DEPTH, int OUT, bool FLEX>
__global__ __launch_bounds__(64 * WAVES) void gemm_w8a8_skinny_kernel(QaGemmW8A8Params p) {
    constexpr int kThreads = 64 * WAVES;
    constexpr int kOob = 0x7ffffff0;                       // beyond any buffer: the load returns zeros
    constexpr int kTile = 32 * kBK;                        // one staged 32-row tile
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int* red = reinterpret_cast<int*>(lds + WAVES * (1 + TM) * kTile);   // [row block][acc register][lane]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, fhalf = lane >> 5;
    const int n0 = blockIdx.x * 32;
    for (int i = tid; i < TM * 16 * 64; i += kThreads) red[i] = 0;

    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.w), 0, static_cast<int>((static_cast<int64_t>(p.n) - 1) * p.ldw + p.k), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.a), 0, static_cast<int>((static_cast<int64_t>(p.m) - 1) * p.lda + p.k), kRsrcFlags);
    // fetch mapping: instruction i, lane l -> tile row 8i + l/8, 16-byte chunk l%8
    const int lrow = lane >> 3, lchunk = lane & 7;
    int w_off[4], a_off[TM][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = n0 + 8 * i + lrow;
        w_off[i] = row < p.n ? static_cast<int>(row * p.ldw) + lchunk * 16 : -1;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int arow = j * 32 + 8 * i + lrow;
            a_off[j][i] = arow < p.m ? static_cast<int>(arow * p.lda) + lchunk * 16 : -1;
        }
    }

    const int k_tiles = (p.k + kBK - 1) / kBK;
    const int my_tiles = (k_tiles - wave + WAVES - 1) / WAVES;      // tiles wave, wave + WAVES, ...
    v4u fw[DEPTH][4], fa[DEPTH][TM][4];
    auto load = [&](int i_tile, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const int k0 = (wave + i_tile * WAVES) * kBK;
        const bool k_ok = k0 + lchunk * 16 < p.k;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            fw[buf][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, (k_ok && w_off[i] >= 0) ? w_off[i] + k0 : kOob, 0, 0);
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                fa[buf][j][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (k_ok && a_off[j][i] >= 0) ? a_off[j][i] + k0 : kOob, 0, 0);
            }
        }
    };

    v16i acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;

    uint8_t* stage = lds + wave * ((1 + TM) * kTile);
    static_for<0, DEPTH - 1>([&](auto s) { load(decltype(s)::value, s); });
    for (int base = 0; base < my_tiles; base += DEPTH) {
        static_for<0, DEPTH>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            // tiles past this wave's share are outside K: their loads touch no memory
            load(base + s + DEPTH - 1, std::integral_constant<int, (s + DEPTH - 1) % DEPTH>{});
            if (base + s < my_tiles) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = 8 * i + lrow;
                    *reinterpret_cast<v4u*>(stage + row * kBK + swz(row, lchunk) * 16) = fw[s][i];
#pragma unroll
                    for (int j = 0; j < TM; ++j)
                        *reinterpret_cast<v4u*>(stage + (1 + j) * kTile + row * kBK + swz(row, lchunk) * 16) = fa[s][j][i];
                }
                wave_lds_sync();
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    const int off = frow * kBK + swz(frow, kk * 2 + fhalf) * 16;
                    const v4i bw = *reinterpret_cast<const v4i*>(stage + off);
#pragma unroll
                    for (int j = 0; j < TM; ++j) {
                        const v4i ba = *reinterpret_cast<const v4i*>(stage + (1 + j) * kTile + off);
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw, ba, acc[j], 0, 0, 0);
                    }
                }
                wave_lds_sync();
            }
        });
    }

    Epilogue e;
    e.row_scale = p.a_scale; e.col_scale = p.w_scale;
    e.row_numel = p.a_scale_numel; e.col_numel = p.w_scale_numel;
    e.use_alpha = p.use_alpha; e.alpha = p.alpha; e.round_mode = p.round_mode; e.col_outer = p.scale_order;
    e.ldd = p.ldd; e.d = p.d;
    skinny_reduce_store<TM, OUT, FLEX, false>(e, acc, red, p.m, p.n, n0, tid, kThreads);
}

template <int TM, int WAVES, int OUT, bool FLEX>
int launch_skinny_one(const QaGemmW8A8Params& p, hipStream_t stream) {
    constexpr int kLds = skinny_lds_bytes<TM, WAVES>();
    auto kernel = gemm_w8a8_skinny_kernel<TM, WAVES, 3, OUT, FLEX>;
    if (kLds > 65536) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kLds) != hipSuccess) {
            return check_launch();
        }
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>((p.n + 31) / 32)), dim3(64 * WAVES), kLds, stream, p);
    return check_launch();
}

template <int TM, int WAVES, bool FLEX>
int launch_skinny(const QaGemmW8A8Params& p, hipStream_t stream) {
    if (p.out_type == QA_OUT_I8) return launch_skinny_one<TM, WAVES, QA_OUT_I8, FLEX>(p, stream);
    if (p.out_type == QA_OUT_BF16) return launch_skinny_one<TM, WAVES, QA_OUT_BF16, FLEX>(p, stream);
    return launch_skinny_one<TM, WAVES, QA_OUT_F16, FLEX>(p, stream);
}

template <bool FLEX>
int dispatch_skinny(const QaGemmW8A8Params& p, hipStream_t stream) {
    // Four waves per workgroup once there is at least one workgroup per CU (measured: more, smaller
    // shares only add per-workgroup overhead); eight when the columns alone give too few workgroups
    // and K is long enough to split further.
    const bool wide = (p.n + 31) / 32 < 256 && p.k >= 16 * kBK;
    if (p.m <= 32) return wide ? launch_skinny<1, 8, FLEX>(p, stream) : launch_skinny<1, 4, FLEX>(p, stream);
    return wide ? launch_skinny<2, 8, FLEX>(p, stream) : launch_skinny<2, 4, FLEX>(p, stream);
}

}  // namespace
}  // namespace qa

extern "C" int qa_gemm_w8a8(const QaGemmW8A8Params* p, void* stream_) {
    using namespace qa;
    if (!p) return QA_ERR_NULL;
    if (p->m < 0 || p->n < 0 || p->k < 0) return QA_ERR_SHAPE;
    const bool empty = p->m == 0 || p->n == 0;                      // (an output without elements: tensors may be null)
    if (!empty && (!p->a || !p->w || !p->d)) return QA_ERR_NULL;
    if (!empty && !p->use_alpha && (!p->a_scale || !p->w_scale)) return QA_ERR_NULL;
    if (p->out_type != QA_OUT_I8 && p->out_type != QA_OUT_F16 && p->out_type != QA_OUT_BF16) return QA_ERR_UNSUPPORTED;
    if (p->scale_order != 0 && p->scale_order != 1) return QA_ERR_UNSUPPORTED;
    if (p->scale_order == 1 && (p->use_alpha || p->round_mode != QA_ROUND_RNE)) return QA_ERR_UNSUPPORTED;
    if (!p->use_alpha && p->a_scale_numel != 1 && p->a_scale_numel != p->m) return QA_ERR_SHAPE;
    if (!p->use_alpha && p->w_scale_numel != 1 && p->w_scale_numel != p->n) return QA_ERR_SHAPE;
    // 16-byte operand chunks: the same alignment the reference's tensor-core path demands
    if (p->k % 16 != 0 || p->lda % 16 != 0 || p->ldw % 16 != 0 || !aligned16(p->a) || !aligned16(p->w)) return QA_ERR_STRIDE;
    if (p->lda < p->k || p->ldw < p->k || p->ldd < p->n) return QA_ERR_STRIDE;
    if (p->m == 0 || p->n == 0) return QA_OK;
    // operands are addressed with 32-bit byte offsets inside a buffer descriptor
    if (static_cast<int64_t>(p->m) * p->lda >= 0x70000000LL || static_cast<int64_t>(p->n) * p->ldw >= 0x70000000LL) return QA_ERR_SHAPE;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const bool flex = p->use_alpha || p->round_mode != QA_ROUND_RNE;
    if (p->m <= 64) return flex ? dispatch_skinny<true>(*p, stream) : dispatch_skinny<false>(*p, stream);
    // the single-row rules (host alpha, round-half-away) only ever come with tiny M
    if (flex) return launch_gemm<2, 2, 2, 2, 2, true>(*p, stream);
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
        const int64_t c_sq = cost(256, 256), c_wide = cost(256, 320), c_tall = cost(320, 256);
        if (c_wide < c_sq && c_wide <= c_tall) return launch_gemm<2, 5, 4, 2, 2, false>(*p, stream);
        // at equal arithmetic the larger tile has fewer rounds, each with its own start and epilogue
        if (c_tall <= c_sq) return launch_gemm<5, 2, 2, 4, 2, false>(*p, stream);
        return launch_gemm<4, 2, 2, 4, 2, false>(*p, stream);                        // 256x256 tile, 8 waves
    }
    // 128x128 tile, 4 waves.  Two stages (64 KB) let two workgroups share a CU; when there is at most one
    // workgroup per CU anyway and K is long (x_proj: 16384 x 5120 -> 192), four stages keep three k-tiles
    // in flight instead of one (36 -> 28 us for that shape).
    const int64_t small_tiles = static_cast<int64_t>((p->m + 127) / 128) * ((p->n + 127) / 128);
    if (small_tiles <= 256 && p->k >= 8 * gemm::kBK) return launch_gemm<2, 2, 2, 2, 4, false>(*p, stream);
    return launch_gemm<2, 2, 2, 2, 2, false>(*p, stream);
}
