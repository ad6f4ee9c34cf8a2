// Micro-benchmark probes used by bench.py only (built into libqa_bench_probes.so, never linked into
// libquamba_amd.so and not part of its C ABI): the rate the matrix cores and the vector ALUs sustain on this part,
// against which the kernels' own figures are read.
#include "../quamba_amd/csrc/qa_common.hpp"

namespace qa {
void set_last_hip_error(int) {}
}  // namespace qa

// ---------------------------------------------------------------------------------------------
// Diagnostic: a register-only loop of v_mfma_i32_32x32x32_i8 (eight independent accumulators, two
// waves per SIMD, every CU busy), with operands that are either one repeated byte or pseudo-random
// bytes.  What the matrix cores sustain depends on the operand values: the switching activity of
// random bytes makes the part lower its clock, so the rate measured here with random operands, not
// the data-sheet figure, is the ceiling a GEMM on real data can approach.  The counters written to
// `ticks` (shader clock and the constant 100 MHz clock, both over the loop of workgroup 0) give the
// clock the loop ran at.
// ---------------------------------------------------------------------------------------------
namespace qa {
namespace {
typedef int v4i_d __attribute__((ext_vector_type(4)));
typedef int v16i_d __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned mix32(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(256) void diag_mfma_i8_kernel(int* sink, long long* ticks, int iters, int random_operands) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    v4i_d a[4], b[2];
    for (int i = 0; i < 4; ++i)
        for (int e = 0; e < 4; ++e) a[i][e] = random_operands ? static_cast<int>(mix32(t * 64 + i * 4 + e)) : 0x01010101;
    for (int i = 0; i < 2; ++i)
        for (int e = 0; e < 4; ++e) b[i][e] = random_operands ? static_cast<int>(mix32(t * 64 + 32 + i * 4 + e)) : 0x01010101;
    v16i_d acc[8];
    for (int i = 0; i < 8; ++i)
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[i / 4], a[i % 4], acc[i], 0, 0, 0);
    }
    int s = 0;
    for (int i = 0; i < 8; ++i)
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    sink[t] = s;
    if (t == 0 && ticks) {
        ticks[0] = clock64() - c0;
        ticks[1] = wall_clock64() - w0;
    }
}
// op 0: v_mul_f32, 1: v_exp_f32, 2: v_rcp_f32, 3: v_log_f32, 4: v_fmac_f32, 5: v_mul_f32 with a quad broadcast (DPP);
// eight chains per lane (op 6, 7: diag_scan_mix_kernel below)
template <int OP>
__global__ __launch_bounds__(256) void diag_valu_kernel(float* sink, long long* ticks, int iters) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = 0.001f * static_cast<float>((t & 255u) + i + 1);
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (OP == 0) asm volatile("v_mul_f32 %0, 0.5, %0" : "+v"(v[i]));
            else if (OP == 1) asm volatile("v_exp_f32 %0, %0" : "+v"(v[i]));
            else if (OP == 2) asm volatile("v_rcp_f32 %0, %0" : "+v"(v[i]));
            else if (OP == 3) asm volatile("v_log_f32 %0, %0" : "+v"(v[i]));
            else if (OP == 4) asm volatile("v_fmac_f32 %0, %1, %1" : "+v"(v[i]) : "v"(v[(i + 1) & 7]));
            else asm volatile("v_mul_f32_dpp %0, %0, %1 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(v[i]) : "v"(v[(i + 1) & 7]));
        }
    }
    float s = 0.0f;
    for (int i = 0; i < 8; ++i) s += v[i];
    sink[t] = s;
    if (t == 0 && ticks) {
        ticks[0] = clock64() - c0;
        ticks[1] = wall_clock64() - w0;
    }
}
// The selective scan's recurrence on live values, registers only: per chain and iteration
//   x = -|h| A;  a = exp2(x);  t = B u;  h = a h + t;  acc = h C + acc      (four plain instructions, one exp2)
// and, with EXTRA, four more plain instructions on changing values.  The values keep moving (h is bounded: the larger
// it gets the faster it decays), so the vector ALUs switch as they do in the real kernel and the part settles at the
// clock it would run the real kernel at; constant operands, as in diag_valu_kernel, leave it at its highest clock.
template <bool EXTRA>
__global__ __launch_bounds__(256) void diag_scan_mix_kernel(float* sink, long long* ticks, int iters) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    float h[8], acc[8], u[8], e1[8];
    const float A = 0.05f + 1e-4f * static_cast<float>(mix32(t) & 1023u);
    const float Bv = 1e-3f * (static_cast<float>(mix32(t + 7u) & 2047u) - 1024.0f);
    const float Cv = 1e-3f * (static_cast<float>(mix32(t + 13u) & 2047u) - 1024.0f);
    for (int i = 0; i < 8; ++i) {
        h[i] = 0.0f; acc[i] = 0.0f; e1[i] = 1.0f;
        u[i] = 1e-2f * (static_cast<float>(mix32(t * 8 + i) & 255u) - 128.0f);
    }
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float x, a, tt;
            asm volatile("v_mul_f32 %0, -|%1|, %2" : "=v"(x) : "v"(h[i]), "v"(A));
            asm volatile("v_exp_f32 %0, %1" : "=v"(a) : "v"(x));
            asm volatile("v_mul_f32 %0, %1, %2" : "=v"(tt) : "v"(Bv), "v"(u[i]));
            asm volatile("v_fma_f32 %0, %1, %0, %2" : "+v"(h[i]) : "v"(a), "v"(tt));
            asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[i]) : "v"(h[i]), "v"(Cv));
            if (EXTRA) {
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(e1[i]) : "v"(a), "v"(Cv));
                asm volatile("v_mul_f32 %0, %1, %0" : "+v"(e1[i]) : "v"(a));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(e1[i]) : "v"(tt), "v"(A));
                asm volatile("v_mul_f32 %0, %1, %0" : "+v"(e1[i]) : "v"(a));
            }
        }
    }
    float s = 0.0f;
    for (int i = 0; i < 8; ++i) s += acc[i] + e1[i];
    sink[t] = s;
    if (t == 0 && ticks) {
        ticks[0] = clock64() - c0;
        ticks[1] = wall_clock64() - w0;
    }
}
}  // namespace
}  // namespace qa

extern "C" int qa_probe_valu(float* sink, int64_t sink_elems, long long* ticks, int workgroups, int iters, int op,
                            void* stream) {
    if (!sink) return QA_ERR_NULL;
    if (workgroups < 1 || iters < 0 || sink_elems < static_cast<int64_t>(workgroups) * 256) return QA_ERR_SHAPE;
    if (op < 0 || op > 7) return QA_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(workgroups)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (op == 0) hipLaunchKernelGGL(qa::diag_valu_kernel<0>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 1) hipLaunchKernelGGL(qa::diag_valu_kernel<1>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 2) hipLaunchKernelGGL(qa::diag_valu_kernel<2>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 3) hipLaunchKernelGGL(qa::diag_valu_kernel<3>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 4) hipLaunchKernelGGL(qa::diag_valu_kernel<4>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 5) hipLaunchKernelGGL(qa::diag_valu_kernel<5>, grid, block, 0, st, sink, ticks, iters);
    else if (op == 6) hipLaunchKernelGGL(qa::diag_scan_mix_kernel<false>, grid, block, 0, st, sink, ticks, iters);
    else hipLaunchKernelGGL(qa::diag_scan_mix_kernel<true>, grid, block, 0, st, sink, ticks, iters);
    return qa::check_launch();
}

extern "C" int qa_probe_mfma_i8(int* sink, int64_t sink_elems, long long* ticks, int workgroups, int iters,
                               int random_operands, void* stream) {
    if (!sink) return QA_ERR_NULL;
    if (workgroups < 1 || iters < 0 || sink_elems < static_cast<int64_t>(workgroups) * 256) return QA_ERR_SHAPE;
    hipLaunchKernelGGL(qa::diag_mfma_i8_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), sink, ticks, iters, random_operands);
    return qa::check_launch();
}
