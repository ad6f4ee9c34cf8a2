// Shared int8-MFMA GEMM core for the W8A8 and W4A8 linears (gfx950).
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]   (int32)      a: (M,K) int8, K-contiguous
//   d[m,n]   = cast(s_row[m|0] * (s_col[n|0] * float(acc)))          w: (N,K) int8, K-contiguous (W8A8)
//                                                                       or 4-bit codes + group scales (W4A8)
// Structure: WGM x WGN waves per workgroup, each wave TM x TN tiles of v_mfma_i32_32x32x32_i8; block
// tile (WGM*TM*32) x (WGN*TN*32) x 128 k-bytes.  The k extent of 128 bytes is one full cache line
// per operand row: measured on MI355X, 64-byte row pieces halve the L1 load rate.  Operand tiles live
// in LDS as rows of eight 16-byte chunks, the chunk index XOR-swizzled with bits 1..3 of the row
// (measured conflict-free for the 32-row x 16-byte fragment reads).  int8 operands go global -> LDS
// directly (buffer_load ... lds, 16 bytes per lane, out-of-range lanes deliver zeros), so no
// registers are spent on staging and the next tile is in flight while the current one is multiplied.
// The 4-bit operand passes through registers, is expanded to int8 there and stored to the same
// layout.  The weight fragment is the MFMA "A" operand, so a lane ends up with four consecutive
// output columns of one row; the epilogue scales, converts, stages through LDS (privately per wave)
// and writes 16-byte pieces of output rows (or of output columns for the transposed layout).
#pragma once
#include "qa_common.hpp"

namespace qa {
namespace gemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr int kBK = 128;                 // k-bytes per tile row
constexpr int kChunks = kBK / 16;        // 16-byte chunks per tile row
constexpr int kRsrcFlags = 0x00020000;   // raw buffer, 32-bit data format

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// s_waitcnt immediate for "at most n vector-memory operations outstanding" (gfx9 encoding),
// leaving the LDS/scalar and export counters unconstrained.
__host__ __device__ constexpr int vmcnt_imm(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8); }

// round (half-even or half-away) and saturate to int8, returned in the low byte of an int
__device__ __forceinline__ int quant8(float v, int round_mode) {
    const float r = round_mode == QA_ROUND_RNE ? __builtin_rintf(v) : __builtin_roundf(v);
    // med3 returns -128 for NaN inputs as min(max(r,-128),127) would
    return static_cast<int>(__builtin_amdgcn_fmed3f(r, -128.0f, 127.0f));
}

// Four values -> four int8 bytes (round half to even, saturating) in one word.  Clamping to the
// integers -128 and 127 first does not change the rounded result; adding 1.5 * 2^23 then rounds to
// nearest-even in the addition itself and leaves the two's-complement byte in the low 8 bits.  The additions of the
// second to fourth value write that low byte straight into its place in the word (sub-dword destination select,
// the other bytes preserved), so no byte permutes are needed.
__device__ __forceinline__ uint32_t pack4_rne_sat8(float v0, float v1, float v2, float v3) {
    const float magic = 12582912.0f;
    const float c1 = __builtin_amdgcn_fmed3f(v1, -128.0f, 127.0f), c2 = __builtin_amdgcn_fmed3f(v2, -128.0f, 127.0f);
    const float c3 = __builtin_amdgcn_fmed3f(v3, -128.0f, 127.0f);
    uint32_t word = __float_as_uint(__builtin_amdgcn_fmed3f(v0, -128.0f, 127.0f) + magic);   // byte 0; bytes 1..3 replaced below
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(c1), "v"(magic));
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(c2), "v"(magic));
    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(c3), "v"(magic));
    return word;
}

// Two fp32 values -> two 16-bit floats of the output type (round to nearest even) in one word; bf16 rounds on the
// bit pattern: add 0x7fff plus the lowest kept bit, keep the high half (NaN payloads are not preserved).
__device__ __forceinline__ uint32_t bf16_bits(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
template <int OUT>
__device__ __forceinline__ uint32_t pack2_f16_or_bf16(float v0, float v1) {
    if (OUT == QA_OUT_BF16) return bf16_bits(v0) | (bf16_bits(v1) << 16);
    const __half2 h = __floats2half2_rn(v0, v1);
    return *reinterpret_cast<const uint32_t*>(&h);
}
template <int OUT>
__device__ __forceinline__ uint16_t one_f16_or_bf16(float v) {
    if (OUT == QA_OUT_BF16) return static_cast<uint16_t>(bf16_bits(v));
    const __half h = __float2half(v);
    return *reinterpret_cast<const uint16_t*>(&h);
}

struct Epilogue {
    const float* row_scale;   // s_row, numel 1 or M (unused with use_alpha)
    const float* col_scale;   // s_col, numel 1 or N
    int row_numel, col_numel;
    int use_alpha;            // d = cast(alpha * acc)
    float alpha;
    int round_mode;           // QaRound
    int col_outer;            // d = cast(s_col * (s_row * acc)) instead of s_row * (s_col * acc)
    int64_t ldd;
    void* d;
};

template <int TM, int TN, int WGM, int WGN, int STAGES>
struct Cfg {
    static constexpr int kWaves = WGM * WGN;
    static constexpr int kThreads = 64 * kWaves;
    static constexpr int kBM = WGM * TM * 32;
    static constexpr int kBN = WGN * TN * 32;
    static constexpr int kAInstr = kBM * kChunks / kThreads;   // direct-to-LDS loads per thread per tile
    static constexpr int kWInstr = kBN * kChunks / kThreads;
    static constexpr int kStageBytes = (kBM + kBN) * kBK;
    static constexpr int kLdsBytes = STAGES * kStageBytes;
};

// Output tile of workgroup `linear`.  Workgroups go to the eight XCDs (each with an L2 of its own) in turn by linear
// index, and with one workgroup per CU a launch runs in rounds of 256.  The tiles an XCD works on at the same time
// should share operand panels, so that its L2 fetches each panel once per round: the 32 workgroups an XCD gets in a
// round take 32 consecutive positions of an order that walks the tile grid in bands of BAND m-tiles, n-tile by
// n-tile - a block of BAND x 32/BAND tiles, whatever the tile counts are (the natural m-first order does that only
// when the number of m-tiles is a multiple of eight).  BAND is 4 or 8, whichever makes the block's operand rows
// (BAND BM + 32/BAND BN) fewer.  The workgroups past the last full round keep the band order as it is.
template <int BM, int BN>
__device__ __forceinline__ void tile_of_workgroup(int linear, int tiles_m, int tiles_n, int& tm, int& tn) {
    constexpr int kXcds = 8, kPerXcd = 32, kRound = kXcds * kPerXcd, kBand = BN > BM ? 8 : 4;
    const int tiles = tiles_m * tiles_n;
    int g = linear;
    if (linear < tiles / kRound * kRound) {
        const int xcd = linear % kXcds, pos = linear / kXcds;
        g = ((pos / kPerXcd) * kXcds + xcd) * kPerXcd + pos % kPerXcd;
    }
    const int per_band = kBand * tiles_n;
    const int band = g / per_band, in_band = g % per_band;
    const int rows = min(kBand, tiles_m - band * kBand);          // the last band may be narrower
    tm = band * kBand + in_band % rows;
    tn = in_band / rows;
}

// Raw buffer descriptor (base, stride 0, num_records bytes) held in four scalar registers.
__device__ __forceinline__ v4i make_rsrc(const void* base, int num_bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(base);
    v4i r;
    r.x = __builtin_amdgcn_readfirstlane(static_cast<int>(addr & 0xffffffffu));
    r.y = __builtin_amdgcn_readfirstlane(static_cast<int>((addr >> 32) & 0xffffu));
    r.z = __builtin_amdgcn_readfirstlane(num_bytes);
    r.w = __builtin_amdgcn_readfirstlane(kRsrcFlags);
    return r;
}

// 16 bytes per lane from buffer offset `voff` straight into LDS at lds_addr + lane*16 (lds_addr is
// wave-uniform); lanes whose offset is outside the buffer deliver zeros.  Written as assembly so
// that the vector-memory counter stays under this kernel's control: a tile's loads stay in flight
// during the arithmetic and are waited for with an explicit s_waitcnt just before the barrier.
__device__ __forceinline__ void buffer_load_lds_b128(v4i rsrc, uint32_t lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory");
}

__device__ __forceinline__ uint4 buffer_load_b128(v4i rsrc, int voff) {
    uint4 v;
    asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(v) : "v"(voff), "s"(rsrc) : "memory");
    return v;
}

__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)p));
}

// Per-lane addressing of one int8 operand tile (ROWS x 128 bytes) for the direct-to-LDS loads:
// instruction g = j*waves + wave fills LDS bytes [g*1024, +1024) of the tile, lane l the slot
// g*64 + l = (row, physical chunk); the lane fetches the logical chunk that the swizzle maps there.
template <int INSTR>
struct TileLoader {
    int voff[INSTR];     // byte offset at k0 = 0 (0x70000000 for rows outside the matrix)
    int kc[INSTR];       // k offset of the chunk inside the tile
    template <int WAVES>
    __device__ __forceinline__ void init(int row0, int rows_total, int64_t ld, int wave, int lane) {
#pragma unroll
        for (int j = 0; j < INSTR; ++j) {
            const int slot = (j * WAVES + wave) * 64 + lane, row = slot / kChunks, c = swz(row, slot % kChunks);
            kc[j] = c * 16;
            voff[j] = row0 + row < rows_total ? static_cast<int>((row0 + row) * ld) + c * 16 : 0x70000000;
        }
    }
    template <int WAVES>
    __device__ __forceinline__ void issue_one(int j, v4i rsrc, int k0, int k_end, uint32_t dst, int wave) const {
        const int off = (k0 + kc[j] < k_end) ? voff[j] + k0 : 0x7ffffff0;
        buffer_load_lds_b128(rsrc, dst + (j * WAVES + wave) * 1024, off);
    }
    template <int WAVES>
    __device__ __forceinline__ void issue(v4i rsrc, int k0, int k_end, uint32_t dst, int wave) const {
#pragma unroll
        for (int j = 0; j < INSTR; ++j) {
            const int off = (k0 + kc[j] < k_end) ? voff[j] + k0 : 0x7ffffff0;
            buffer_load_lds_b128(rsrc, dst + (j * WAVES + wave) * 1024, off);
        }
    }
};

// Accumulates one 128-byte k tile with the instruction order pinned: sa / sw point at this wave's rows of the
// staged operands.  The fragments of step kk+1 are requested
// before the multiplications of step kk are issued, and `hook(slot)` runs after every second
// multiplication (slot = 0 .. 4*TM*TN/2 - 1): the caller places its global -> LDS requests for the
// next tile there, one at a time, so that the wave never waits on a full memory queue with
// multiplications behind it in program order.  sched_barrier keeps the compiler from regrouping.
template <int TM, int TN, class Hook>
__device__ __forceinline__ void mma_tile_paced(const uint8_t* sa, const uint8_t* sw, int frow, int fhalf,
                                               v16i (&acc)[TN][TM], Hook&& hook) {
    v4i fa[2][TM], fw[2][TN];
    auto fetch = [&](int kk, int buf) {
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            const int row = i * 32 + frow;
            fw[buf][i] = *reinterpret_cast<const v4i*>(sw + row * kBK + swz(row, kk * 2 + fhalf) * 16);
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int row = j * 32 + frow;
            fa[buf][j] = *reinterpret_cast<const v4i*>(sa + row * kBK + swz(row, kk * 2 + fhalf) * 16);
        }
    };
    fetch(0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < kBK / 32; ++kk) {
        if (kk + 1 < kBK / 32) fetch(kk + 1, (kk + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[kk & 1][i], fa[kk & 1][j], acc[i][j], 0, 0, 0);
                if ((i * TM + j) % 2 == 1) {
                    __builtin_amdgcn_sched_barrier(0);
                    hook(kk * (TM * TN / 2) + (i * TM + j) / 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
    }
}

// The fragments of k step kk of this wave's rows (sa: TM row blocks of the a operand, sw: TN of the w operand).
template <int TM, int TN>
__device__ __forceinline__ void fetch_fragments(const uint8_t* sa, const uint8_t* sw, int kk, int frow, int fhalf,
                                                v4i (&fa)[TM], v4i (&fw)[TN]) {
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        const int row = i * 32 + frow;
        fw[i] = *reinterpret_cast<const v4i*>(sw + row * kBK + swz(row, kk * 2 + fhalf) * 16);
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int row = j * 32 + frow;
        fa[j] = *reinterpret_cast<const v4i*>(sa + row * kBK + swz(row, kk * 2 + fhalf) * 16);
    }
}

// One k tile of a main loop whose workgroup barrier sits before the last k step instead of between tiles.  On entry
// the fragments of k step 0 of the tile at `sa`/`sw` are in fa[0]/fw[0].  Steps 0..2 fetch the fragments of the step
// after them; before the multiplications of step 3 the wave waits for its own global -> LDS requests, meets the
// others at the barrier - every wave then holds all fragments of this tile, so this stage may be overwritten, and
// the next tile's stage is complete - and fetches step 0 of the next tile from `na`/`nw`.  The matrix pipe has the
// multiplications of step 3 queued behind the barrier, so it does not drain while the first fragments of the next
// tile travel.  `hook(idx)` runs after every multiplication, idx counted from the barrier: 0 .. TM*TN-1 during
// step 3 of this tile, the following 3*TM*TN during steps 0..2 of the next one; the caller places its global ->
// LDS requests behind the multiplications it chooses (a hook that does nothing costs nothing).
template <int TM, int TN, class Hook>
__device__ __forceinline__ void mma_tile_rotated(const uint8_t* sa, const uint8_t* sw, const uint8_t* na, const uint8_t* nw,
                                                 int frow, int fhalf, v4i (&fa)[2][TM], v4i (&fw)[2][TN],
                                                 v16i (&acc)[TN][TM], Hook&& hook) {
#pragma unroll
    for (int kk = 0; kk < kBK / 32; ++kk) {
        if (kk + 1 < kBK / 32) {
            fetch_fragments<TM, TN>(sa, sw, kk + 1, frow, fhalf, fa[(kk + 1) & 1], fw[(kk + 1) & 1]);
        } else {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            __syncthreads();
            fetch_fragments<TM, TN>(na, nw, 0, frow, fhalf, fa[0], fw[0]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[kk & 1][i], fa[kk & 1][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                hook(((kk + 1) % (kBK / 32)) * (TM * TN) + i * TM + j);
                __builtin_amdgcn_sched_barrier(0);
            }
    }
}

// Orders this wave's LDS writes before its later LDS reads (the staging area is private to the
// wave, and one wave's LDS operations execute in order, so no workgroup barrier is needed).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// In acc[i][j] lane l holds output row m = j*32 + (l & 31) and, in register r, column
// n = i*32 + 8*(r/4) + 4*(l/32) + (r%4).
// FLEX = false compiles the common rule only (d = cast_rne(s_row * (s_col * acc))); FLEX = true also
// honours use_alpha and the round-half-away GEMV rule at run time.  TRANS selects the (N,M) output.
// COL_OUTER (the column scale applied last) is a compile-time choice: selecting the association per
// element costs two extra instructions on each of the 128 outputs of a lane.
template <int TM, int TN, int OUT, bool FLEX, bool TRANS, bool COL_OUTER = false>
__device__ __forceinline__ void epilogue(const Epilogue& e, v16i (&acc)[TN][TM], uint8_t* lds, int m, int n,
                                         int wave_m0, int wave_n0, int wave, int lane) {
    constexpr int kElt = OUT == QA_OUT_I8 ? 1 : 2;
    const int frow = lane & 31, fhalf = lane >> 5;
    const bool vec_ok = (e.ldd * kElt) % 16 == 0 && aligned16(e.d);
    const bool use_alpha = FLEX && e.use_alpha;
    const bool away = FLEX && e.round_mode == QA_ROUND_HALF_AWAY;
    const int round_mode = FLEX ? e.round_mode : QA_ROUND_RNE;

    // this lane's column scales: 4 consecutive columns per (i, q), loaded once
    float s_col[TN][4][4];
    if (use_alpha || e.col_numel == 1) {
        // one scale for every column: a single (scalar) fetch instead of one per column and lane
        const float one = use_alpha ? 1.0f : e.col_scale[0];
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int t = 0; t < 4; ++t) s_col[i][q][t] = one;
    } else {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int nn = wave_n0 + i * 32 + 8 * q + 4 * fhalf + t;
                    s_col[i][q][t] = e.col_scale[min(nn, n - 1)];
                }
    }
    float s_row[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int mm = wave_m0 + j * 32 + frow;
        s_row[j] = use_alpha ? e.alpha : e.row_scale[e.row_numel == 1 ? 0 : min(mm, m - 1)];
    }
    auto scaled = [&](int i, int j, int q, int t) -> float {
        const float accf = static_cast<float>(acc[i][j][q * 4 + t]);
        float v;
        if (use_alpha) v = s_row[j] * accf;
        // GEMV rule (round-half-away mode): the two scales are multiplied first
        else if (COL_OUTER) v = s_col[i][q][t] * (s_row[j] * accf);
        else v = away ? (s_col[i][q][t] * s_row[j]) * accf : s_row[j] * (s_col[i][q][t] * accf);
        // keep the fp32 product a value of its own: folding the multiply into a mixed-precision
        // convert would round once instead of twice and change the fp16 result in rare cases
        asm volatile("" : "+v"(v));
        return v;
    };

    if (!TRANS) {
        constexpr int kPitch = TN * 32 * kElt + 16;
        uint8_t* stg = lds + wave * (32 * kPitch);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
#pragma unroll
            for (int i = 0; i < TN; ++i) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = i * 32 + 8 * q + 4 * fhalf;
                    const float v0 = scaled(i, j, q, 0), v1 = scaled(i, j, q, 1);
                    const float v2 = scaled(i, j, q, 2), v3 = scaled(i, j, q, 3);
                    if (OUT == QA_OUT_I8) {
                        uint32_t word;
                        if (!away) {
                            word = pack4_rne_sat8(v0, v1, v2, v3);
                        } else {
                            const uint32_t b0 = quant8(v0, round_mode) & 0xff, b1 = quant8(v1, round_mode) & 0xff;
                            const uint32_t b2 = quant8(v2, round_mode) & 0xff, b3 = quant8(v3, round_mode);
                            word = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
                        }
                        *reinterpret_cast<uint32_t*>(stg + frow * kPitch + nl) = word;
                    } else {
                        uint2 pk;
                        pk.x = pack2_f16_or_bf16<OUT>(v0, v1);
                        pk.y = pack2_f16_or_bf16<OUT>(v2, v3);
                        *reinterpret_cast<uint2*>(stg + frow * kPitch + nl * 2) = pk;
                    }
                }
            }
            wave_lds_sync();
            constexpr int kPiecesPerRow = TN * 32 * kElt / 16;
#pragma unroll
            for (int piece = lane; piece < 32 * kPiecesPerRow; piece += 64) {
                const int r = piece / kPiecesPerRow, cb = (piece % kPiecesPerRow) * 16;
                const int mm2 = wave_m0 + j * 32 + r;
                const int nn = wave_n0 + cb / kElt;
                if (mm2 >= m || nn >= n) continue;
                uint8_t* dst = static_cast<uint8_t*>(e.d) + (static_cast<int64_t>(mm2) * e.ldd + nn) * kElt;
                const uint4 val = *reinterpret_cast<const uint4*>(stg + r * kPitch + cb);
                if (vec_ok && nn + 16 / kElt <= n) {
                    *reinterpret_cast<uint4*>(dst) = val;
                } else {
                    const uint8_t* src = reinterpret_cast<const uint8_t*>(&val);
                    const int nbytes = min(16, (n - nn) * kElt);
                    for (int t = 0; t < nbytes; ++t) dst[t] = src[t];
                }
            }
            wave_lds_sync();
        }
    } else {
        // transposed output d[n][m]: stage 32 columns n x (TM*32) rows m per pass
        constexpr int kPitch = TM * 32 * kElt + 16;
        uint8_t* stg = lds + wave * (32 * kPitch);
#pragma unroll
        for (int i = 0; i < TN; ++i) {
#pragma unroll
            for (int j = 0; j < TM; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int nl = 8 * q + 4 * fhalf + t;          // column inside this 32-column tile
                        const float v = scaled(i, j, q, t);
                        if (OUT == QA_OUT_I8) {
                            *reinterpret_cast<int8_t*>(stg + nl * kPitch + j * 32 + frow) =
                                static_cast<int8_t>(quant8(v, round_mode));
                        } else {
                            *reinterpret_cast<uint16_t*>(stg + nl * kPitch + (j * 32 + frow) * 2) = one_f16_or_bf16<OUT>(v);
                        }
                    }
                }
            }
            wave_lds_sync();
            constexpr int kPiecesPerRow = TM * 32 * kElt / 16;
#pragma unroll
            for (int piece = lane; piece < 32 * kPiecesPerRow; piece += 64) {
                const int r = piece / kPiecesPerRow, cb = (piece % kPiecesPerRow) * 16;
                const int nn = wave_n0 + i * 32 + r;
                const int mm2 = wave_m0 + cb / kElt;
                if (nn >= n || mm2 >= m) continue;
                uint8_t* dst = static_cast<uint8_t*>(e.d) + (static_cast<int64_t>(nn) * e.ldd + mm2) * kElt;
                const uint4 val = *reinterpret_cast<const uint4*>(stg + r * kPitch + cb);
                if (vec_ok && mm2 + 16 / kElt <= m) {
                    *reinterpret_cast<uint4*>(dst) = val;
                } else {
                    const uint8_t* src = reinterpret_cast<const uint8_t*>(&val);
                    const int nbytes = min(16, (m - mm2) * kElt);
                    for (int t = 0; t < nbytes; ++t) dst[t] = src[t];
                }
            }
            wave_lds_sync();
        }
    }
}

// Largest epilogue staging footprint (fp16, either orientation) must fit in the operand stages.
template <int TM, int TN, int WAVES>
constexpr int epilogue_lds_bytes() {
    return WAVES * 32 * ((TM > TN ? TM : TN) * 32 * 2 + 16);
}

// ---------------------------------------------------------------------------------------------
// Pieces shared by the kernels for few activation rows (one 32-column block per workgroup, K split
// over the waves, a wave-private staging area of one weight tile and TM activation tiles).
// ---------------------------------------------------------------------------------------------
template <int TM, int WAVES>
constexpr int skinny_lds_bytes() { return WAVES * (1 + TM) * 32 * kBK + TM * 16 * 64 * 4; }

// Adds the waves' partial accumulators in `red` (TM*16*64 ints, zeroed by the caller before any
// barrier it has passed), then every thread scales and writes four consecutive columns of one row.
// Lane l of the accumulator layout holds row (l & 31) and, in registers 4q..4q+3, the columns
// 8q + 4*(l >> 5) + (0..3): one unit = (row block, q, lane).
template <int TM, int OUT, bool FLEX, bool TRANS>
__device__ __forceinline__ void skinny_reduce_store(const Epilogue& e, v16i (&acc)[TM], int* red, int m, int n,
                                                    int n0, int tid, int threads) {
    const int lane = tid & 63;
    __syncthreads();                                       // red is zero
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            __hip_atomic_fetch_add(&red[(j * 16 + r) * 64 + lane], acc[j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();

    constexpr int kElt = OUT == QA_OUT_I8 ? 1 : 2;
    const bool use_alpha = FLEX && e.use_alpha;
    const bool away = FLEX && e.round_mode == QA_ROUND_HALF_AWAY;
    const int round_mode = FLEX ? e.round_mode : QA_ROUND_RNE;
    const bool vec_ok = !TRANS && e.ldd % 4 == 0 && (reinterpret_cast<uintptr_t>(e.d) & (4 * kElt - 1)) == 0;
    for (int u = tid; u < TM * 4 * 64; u += threads) {
        const int ul = u & 63, j = u >> 8, q = (u >> 6) & 3;
        const int mm = j * 32 + (ul & 31);
        const int nn = n0 + 8 * q + 4 * (ul >> 5);
        if (mm >= m || nn >= n) continue;
        const float s_row = use_alpha ? e.alpha : e.row_scale[e.row_numel == 1 ? 0 : mm];
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float accf = static_cast<float>(red[(j * 16 + q * 4 + t) * 64 + ul]);
            const float s_col = use_alpha ? 1.0f : e.col_scale[e.col_numel == 1 ? 0 : min(nn + t, n - 1)];
            if (use_alpha) v[t] = s_row * accf;
            else if (e.col_outer) v[t] = s_col * (s_row * accf);
            else v[t] = away ? (s_col * s_row) * accf : s_row * (s_col * accf);
            asm volatile("" : "+v"(v[t]));                 // the fp32 product is rounded on its own
        }
        const int cols = min(4, n - nn);
        const int64_t step = TRANS ? e.ldd : 1;            // distance between consecutive columns
        const int64_t at = TRANS ? static_cast<int64_t>(nn) * e.ldd + mm : static_cast<int64_t>(mm) * e.ldd + nn;
        if (OUT == QA_OUT_I8) {
            int8_t* dst = static_cast<int8_t*>(e.d) + at;
            if (vec_ok && cols == 4) {
                const uint32_t b0 = quant8(v[0], round_mode) & 0xff, b1 = quant8(v[1], round_mode) & 0xff;
                const uint32_t b2 = quant8(v[2], round_mode) & 0xff, b3 = quant8(v[3], round_mode);
                *reinterpret_cast<uint32_t*>(dst) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
            } else {
                for (int t = 0; t < cols; ++t) dst[t * step] = static_cast<int8_t>(quant8(v[t], round_mode));
            }
        } else {
            uint16_t* dst = static_cast<uint16_t*>(e.d) + at;
            if (vec_ok && cols == 4) {
                uint2 pk;
                pk.x = pack2_f16_or_bf16<OUT>(v[0], v[1]);
                pk.y = pack2_f16_or_bf16<OUT>(v[2], v[3]);
                *reinterpret_cast<uint2*>(dst) = pk;
            } else {
                for (int t = 0; t < cols; ++t) dst[t * step] = one_f16_or_bf16<OUT>(v[t]);
            }
        }
    }
}

}  // namespace gemm
}  // namespace qa
