/*
 * quamba_amd.h - C ABI of libquamba_amd.so: quantized Mamba mixer kernels for AMD MI355X (gfx950).
 *
 * Every entry point takes a parameter block of plain pointers, sizes, element strides and scales,
 * plus the HIP stream (hipStream_t passed as void*) on which the kernels are enqueued.  The
 * library never allocates, never synchronises and keeps no mutable global state, so calls are
 * re-entrant and can be captured into HIP graphs.  All pointers are device pointers unless said
 * otherwise.  Strides count elements, not bytes.  Return value: QA_OK (0) or a negative QaStatus.
 * A call whose sizes leave nothing to compute (no batch entries, rows or steps) returns QA_OK without a
 * launch, and its tensors may then be null; a scan over no steps writes the zero state it starts from.
 *
 * Each entry point names the interface of the reference (enyac-group/Quamba, paths relative to
 * its root) that it replaces.
 */
#ifndef QUAMBA_AMD_H
#define QUAMBA_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum QaStatus {
    QA_OK = 0,
    QA_ERR_NULL = -1,        /* a required pointer is null */
    QA_ERR_SHAPE = -2,       /* a size is out of the supported range */
    QA_ERR_STRIDE = -3,      /* a stride / alignment requirement is violated */
    QA_ERR_UNSUPPORTED = -4, /* valid request the library has no kernel for */
    QA_ERR_LAUNCH = -5,      /* the HIP runtime refused the launch */
    QA_ERR_SCRATCH = -6      /* the problem needs more scratch than the library's fixed buffer holds */
} QaStatus;

/* Human-readable text for a status code (static storage). */
const char* qa_status_string(int status);
/* ABI version, bumped on any incompatible change of the structs below. */
int qa_abi_version(void);
/* Last HIP error code seen by a failed launch on this thread (0 if none). */
int qa_last_hip_error(void);

/* ------------------------------------------------------------------------------------------
 * Mamba1 int8 depthwise causal conv1d (+ optional SiLU) with int8 requantisation.
 * Replaces quant_causal_conv1d_cuda.fwd / .update
 *   (csrc/causal_conv1d/quant_causal_conv1d.cpp:76-164, :167-226; parameter block
 *    csrc/causal_conv1d/causal_conv1d.h:9-55).
 * ---------------------------------------------------------------------------------------- */
typedef struct QaConvParams {
    int32_t batch, dim, seqlen, width;   /* width in [2,4] */
    int32_t silu_activation;             /* 0 / 1 */
    int32_t reserved0;
    /* x, out: int8 (batch, dim, seqlen).  Either seqlen-contiguous (x_l_stride == 1) or
     * channel-contiguous (x_c_stride == 1); out uses its own strides. */
    int64_t x_batch_stride, x_c_stride, x_l_stride;
    int64_t out_batch_stride, out_c_stride, out_l_stride;
    int64_t weight_c_stride, weight_width_stride;   /* weight int8 (dim, width) */
    /* update only: conv_state int8 (batch, dim, state_len), state_len == width or width-1 */
    int64_t conv_state_batch_stride, conv_state_c_stride, conv_state_l_stride;
    int32_t conv_state_len;
    int32_t reserved1;
    const int8_t* x;
    const int8_t* weight;
    const int8_t* bias;        /* int8 (dim) or null */
    int8_t* out;
    int8_t* conv_state;        /* update only, modified in place */
    float scale_x, scale_w, scale_b, scale_out;
    /* fwd only, optional: a second copy of the output with channels contiguous, int8 (batch, seqlen, dim),
     * element (b, t, c) at out_t + b*out_t_batch_stride + t*out_t_l_stride + c.  It replaces the separate
     * transposition the reference's caller runs before x_proj (quamba/qMambaLayer.py:923).  Needs the
     * seqlen-contiguous input layout; null to skip. */
    int8_t* out_t;
    int64_t out_t_batch_stride, out_t_l_stride;
} QaConvParams;

int qa_causal_conv1d_fwd(const QaConvParams* p, void* stream);
int qa_causal_conv1d_update(const QaConvParams* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * Mamba2 xBC conv: one depthwise causal conv1d (+ SiLU) over the concatenated channels
 * [x (x_dim) | B (n_groups*d_state) | C (n_groups*d_state)], each part with its own input, weight
 * and bias scales, requantised into three int8 tensors: x with one output scale or one per
 * (ssd group, head group, dim group) found through cumulative end-index tables, B and C with one
 * output scale or one per ssd group.
 * Replaces quamba2_conv1d_cuda.fwd / .update
 *   (csrc/causal_conv1d/quamba2_conv1d.cpp:109-251, :254-379; kernels
 *    quamba2_conv1d_fwd_kernel.cuh:57-347, quamba2_conv1d_update_kernel.cuh:28-147).
 * Forward takes the channel-contiguous layout only, as the reference does: element (b, c, l) of
 * xBC at b*xBC_batch_stride + l*xBC_l_stride + c; the outputs likewise (x_l_stride etc.).
 * Update: xBC (batch, dim) with xBC_c_stride; outputs (batch, part) with *_c_stride; conv_state
 * int8 (batch, dim, conv_state_len), conv_state_len == width or width-1, shifted in place.
 * ---------------------------------------------------------------------------------------- */
typedef struct QaConv2Params {
    int32_t batch, dim, seqlen, width;   /* dim == x_dim + 2*n_groups*d_state, width in [2,4] */
    int32_t silu_activation;
    int32_t x_dim, x_headdim, d_state, n_groups;
    int32_t nhead_groups, ndim_groups;   /* 0, 0: one output scale per part */
    int32_t conv_state_len;
    int64_t xBC_batch_stride, xBC_l_stride, xBC_c_stride;   /* fwd: c stride 1; update: l stride unused */
    int64_t x_batch_stride, x_l_stride, x_c_stride;
    int64_t B_batch_stride, B_l_stride, B_c_stride;
    int64_t C_batch_stride, C_l_stride, C_c_stride;
    int64_t weight_c_stride, weight_width_stride;           /* weight int8 (dim, width) */
    int64_t conv_state_batch_stride, conv_state_c_stride, conv_state_l_stride;
    const int8_t* xBC;
    const int8_t* weight;
    const int8_t* bias;                  /* int8 (dim) or null */
    int8_t* x;
    int8_t* B;
    int8_t* C;
    int8_t* conv_state;                  /* update only */
    const float* x_out_scales;           /* [1] or [n_groups, nhead_groups, ndim_groups] */
    const float* B_out_scales;           /* [1] or [n_groups] */
    const float* C_out_scales;
    const int32_t* x_head_group_range;   /* [n_groups, nhead_groups] cumulative end indices, or null */
    const int32_t* x_dim_group_range;    /* [n_groups, nhead_groups, ndim_groups], or null */
    float scale_x, scale_B, scale_C;     /* input scales of the three parts */
    float scale_wx, scale_wB, scale_wC;  /* weight scales */
    float scale_bx, scale_bB, scale_bC;  /* bias scales */
    float reserved0;
} QaConv2Params;

int qa_quamba2_conv1d_fwd(const QaConv2Params* p, void* stream);
int qa_quamba2_conv1d_update(const QaConv2Params* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * Gated RMS norm of fp16 rows with int8 gate input and int8 or fp16 output (Mamba2, between the SSD
 * scan and out_proj).  Per (row, group of group_size columns):
 *   x' = x * silu(z_scale*qz)            (gate first: norm_before_gate == 0)
 *   y  = x' / sqrt(mean(x'^2) + eps) * w
 *   y *= silu(z_scale*qz)                (norm_before_gate == 1)
 *   out = fp16(y) | sat8(rint(y / out_scale)) | sat8(rint(y / (max(y)/127))) with that scale stored at
 *         dyn_scale[group*rows + row]    (out_mode 0 | 1 | 2; max(y), not max|y|, as the reference)
 * Replaces _qlayer_normgated_fwd (quamba/triton/quant_normgated.py:11-134) as used by QRMSNormGated
 * (quamba/qNorm.py:93-177).  RMS norm without bias only.
 * ---------------------------------------------------------------------------------------- */
enum { QA_NORM_OUT_F16 = 0, QA_NORM_OUT_I8_STATIC = 1, QA_NORM_OUT_I8_DYNAMIC = 2 };

typedef struct QaNormGatedParams {
    int32_t rows, dim, group_size;   /* dim % group_size == 0, group_size % 8 == 0, group_size <= 8192 */
    int32_t norm_before_gate;
    int32_t out_mode;
    float eps, z_scale, out_scale;
    int64_t x_row_stride, z_row_stride, out_row_stride;   /* elements */
    const void* x;        /* fp16 (rows, dim) */
    const void* weight;   /* fp16 (dim) */
    const int8_t* qz;     /* int8 (rows, dim) or null (no gate) */
    void* out;            /* fp16 or int8 (rows, dim) */
    float* dyn_scale;     /* [dim/group_size * rows], out_mode 2 only */
} QaNormGatedParams;

int qa_rmsnorm_gated(const QaNormGatedParams* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * Hadamard transform of every row of a (rows, dim) matrix + int8 quantisation:
 *   out[r, :] = sat8(round_half_away(H x[r, :] * scale)),  dim = S * 2^k with S in {1, 12, 40},
 *   H = H_S (x) W_{2^k} (natural-order Walsh-Hadamard on the low index, the fixed 12- or 40-point
 *   matrix on the high index); the caller folds 1/sqrt(dim) and 1/output scale into `scale`.
 * Replaces quant_hadamard.fast_hadamard_transform / _12N / _40N
 *   (csrc/hadamard/quant_hadamard.cpp, kernel csrc/hadamard/quant_hadamard_fwd.cu:153-229).
 * Values beyond the int8 range saturate (the reference's cast is undefined there).
 * ---------------------------------------------------------------------------------------- */
enum { QA_IN_F16 = 0, QA_IN_F32 = 1 };

typedef struct QaHadamardParams {
    int32_t rows, dim;       /* dim <= 32768 */
    int32_t in_type;         /* QA_IN_F16 / QA_IN_F32 */
    float scale;
    int64_t x_row_stride, out_row_stride;   /* elements; columns are contiguous */
    const void* x;
    int8_t* out;
} QaHadamardParams;

int qa_hadamard_quant(const QaHadamardParams* p, void* stream);

/* The gated RMS norm and the Hadamard transform + quantisation of its fp16 output in one pass over the
 * rows: out = qa_hadamard_quant(qa_rmsnorm_gated(...)) bit for bit, without the fp16 matrix between them.
 * Replaces the pair QRMSNormGated.forward (quamba/qNorm.py:93-177, fp16 output) -> HadLinear's
 * transform (quamba/qHadamard.py, quant_hadamard.fast_hadamard_transform) in the Mamba2 mixer
 * (quamba/qMamba2.py, `y = self.norm(y, z)` then `self.out_proj(y)`).
 * `norm`: rows, dim, group_size, norm_before_gate, eps, z_scale, x, weight, qz and their strides as for
 * qa_rmsnorm_gated; out_mode must be QA_NORM_OUT_F16; out, out_row_stride, out_scale, dyn_scale unused.
 * `had`: rows, dim (equal to the norm's), scale, out, out_row_stride; x, x_row_stride, in_type unused.
 * Supported: dim 2048, 4096 or 8192 with group_size 512, 1024 or 2048, 16-byte aligned rows;
 * anything else returns QA_ERR_UNSUPPORTED (callers then make the two calls). */
int qa_rmsnorm_gated_hadamard_quant(const QaNormGatedParams* norm, const QaHadamardParams* had, void* stream);

/* ------------------------------------------------------------------------------------------
 * Mamba1 int8 selective scan, forward over a sequence.
 * Replaces quant_sscan_cuda.fwd (csrc/selective_scan/quant_sscan.cpp:122-265; parameter block
 * csrc/selective_scan/quant_sscan.h:26-86).  Differences kept deliberate: the output is written
 * directly in (batch, seqlen, dim) order (the reference transposes afterwards, quant_sscan.cpp:262),
 * and the last state can be returned as fp32 and/or int8.
 * Scales are device pointers to one fp32 each, exactly as the reference passes them.
 * ---------------------------------------------------------------------------------------- */
typedef struct QaSScanParams {
    int32_t batch, dim, seqlen, dstate;  /* dstate <= 256 */
    int32_t n_groups;                    /* B/C groups, dim % n_groups == 0 */
    int32_t delta_softplus;
    /* u, delta, z: int8 (batch, dim, seqlen), seqlen-contiguous */
    int64_t u_batch_stride, u_d_stride;
    int64_t delta_batch_stride, delta_d_stride;
    int64_t z_batch_stride, z_d_stride;
    /* B, C: int8 (batch, n_groups, dstate, seqlen), seqlen-contiguous */
    int64_t B_batch_stride, B_group_stride, B_dstate_stride;
    int64_t C_batch_stride, C_group_stride, C_dstate_stride;
    int64_t A_d_stride, A_dstate_stride;             /* A_log int8 (dim, dstate) */
    /* out: fp16, element (b, l, d) at b*out_batch_stride + l*out_l_stride + d*out_d_stride */
    int64_t out_batch_stride, out_l_stride, out_d_stride;
    const int8_t* u;
    const int8_t* delta;
    const int8_t* A_log;
    const int8_t* B;
    const int8_t* C;
    const int8_t* D;           /* int8 (dim) or null */
    const int8_t* delta_bias;  /* int8 (dim) or null */
    const int8_t* z;           /* or null */
    const float* scale_u;
    const float* scale_delta;
    const float* scale_A;
    const float* scale_B;
    const float* scale_C;
    const float* scale_D;          /* required iff D */
    const float* scale_delta_bias; /* required iff delta_bias */
    const float* scale_z;          /* required iff z */
    const float* scale_ssm_state;  /* required iff last_state_i8 */
    void* out;                     /* fp16 */
    int8_t* last_state_i8;         /* int8 (batch, dim, dstate) contiguous, or null */
    float* last_state_f32;         /* fp32 (batch, dim, dstate) contiguous, or null */
    /* Optional (all null / 0 otherwise): one long sequence scanned as several segments side by side - no
     * counterpart in the reference, whose kernel splits the sequence inside a thread block instead
     * (csrc/selective_scan/quant_sscan_fwd_kernel.cuh, BlockScan over (a, b) pairs).
     * dt_sum_out: fp32 (batch, dim), receives the sum over the steps of each channel's step size after bias
     *   and softplus; the decay of the whole run of steps is exp(A * that).
     * carry_dt_sum fp32 (n, dim), carry_state fp32 (n, dim, dstate), carry_first: the batch entries are
     *   segments carry_first, carry_first + 1, ... of one sequence; carry_* hold, for the segments before
     *   them, the step-size sums and the end states of a scan from a zero state.  Entry b starts from
     *   the state obtained by chaining segments 0 .. carry_first + b - 1:
     *   h <- exp(A * carry_dt_sum[s]) * h + carry_state[s]. */
    float* dt_sum_out;
    const float* carry_dt_sum;
    const float* carry_state;
    int32_t carry_first;
    /* 0: the library picks how lanes are laid over channels and states.  Tests name a mapping to cover every
     * kernel variant on one shape: QA_SSCAN_MAPPING(lanes per channel, waves per workgroup) for d_state <= 16
     * (lanes 1, 2, 4, 8); lanes == 0 is the launch with two kinds of workgroup, the second argument then being
     * the number of 64-channel workgroups per batch entry that take four lanes per channel.  A mapping the
     * shape does not admit returns QA_ERR_SHAPE or QA_ERR_UNSUPPORTED.  Results agree to fp32 rounding. */
    int32_t mapping;
} QaSScanParams;

/* marker bit 30, lanes in bits 20..27, the second argument in bits 0..19; a value without the marker is refused */
#define QA_SSCAN_MAPPING(lanes, arg) (0x40000000 | ((lanes) << 20) | (arg))

int qa_sscan_fwd(const QaSScanParams* p, void* stream);
/* The mapping qa_sscan_fwd takes for these sizes on the current device, as a QA_SSCAN_MAPPING code (0 for d_state
 * above 16, which has one mapping per size; p->mapping itself when the caller named one), or a negative QaStatus.
 * Only batch, dim, dstate, n_groups and mapping are read; nothing is launched.  No counterpart in the reference
 * (csrc/selective_scan/quant_sscan_fwd_kernel.cuh:296-349 has one launch shape per d_state); bench.py prices the
 * launch's instruction mix with it. */
int qa_sscan_chosen_mapping(const QaSScanParams* p);

/* ------------------------------------------------------------------------------------------
 * Single-token recurrent state update (decode step), Mamba1 (nheads == 1, headdim == d_inner)
 * and Mamba2 (nheads x headdim).
 * Replaces quant_sscan_update_triton / quamba2_sscan_update_triton
 *   (quamba/triton/selective_state_update.py:129-227, :365-478).
 * The state is either int8 with a scale (reference behaviour: dequantise, update, requantise in
 * place) or fp32 (updated in place, no requantisation).
 * ---------------------------------------------------------------------------------------- */
typedef struct QaSsmUpdateParams {
    int32_t batch, nheads, dim, dstate;  /* dim = channels per head */
    int32_t ngroups;                     /* B/C groups, nheads % ngroups == 0 */
    int32_t dt_softplus;
    int32_t state_is_fp32;               /* 0: int8 state + state_scale, 1: fp32 state */
    int32_t dt_bias_is_fp16;             /* 0: int8 dt_bias + scale (Mamba1), 1: fp16 dt_bias (Mamba2) */
    /* grouped state scales (Mamba2 head/dim groups); 0 groups = one scalar state scale */
    int32_t nhead_groups, ndim_groups;
    int64_t state_batch_stride, state_head_stride, state_dim_stride, state_dstate_stride;
    int64_t x_batch_stride, x_head_stride, x_dim_stride;
    int64_t dt_batch_stride, dt_head_stride, dt_dim_stride;      /* stride 0 = broadcast */
    int64_t dt_bias_head_stride, dt_bias_dim_stride;
    int64_t A_head_stride, A_dim_stride, A_dstate_stride;
    int64_t B_batch_stride, B_group_stride, B_dstate_stride;
    int64_t C_batch_stride, C_group_stride, C_dstate_stride;
    int64_t D_head_stride, D_dim_stride;
    int64_t z_batch_stride, z_head_stride, z_dim_stride;
    int64_t out_batch_stride, out_head_stride, out_dim_stride;
    void* state;               /* int8 or fp32, in place */
    const int8_t* x;
    const int8_t* dt;
    const void* dt_bias;       /* int8 or fp16 or null */
    const int8_t* A_log;
    const int8_t* B;
    const int8_t* C;
    const int8_t* D;           /* or null */
    const int8_t* z;           /* or null */
    const float* x_scale;      /* one fp32, or [ngroups, nhead_groups, ndim_groups] when grouped */
    const float* dt_scale;
    const float* dt_bias_scale; /* int8 dt_bias only */
    const float* A_log_scale;
    const float* state_scale;  /* one fp32, or [ngroups, nhead_groups, ndim_groups, dstate] when grouped */
    const float* B_scale;      /* one fp32, or [ngroups] when grouped */
    const float* C_scale;
    const float* D_scale;
    const float* z_scale;
    const int32_t* x_head_group_range; /* [ngroups, nhead_groups] cumulative end indices, grouped only */
    const int32_t* x_dim_group_range;  /* [ngroups, nhead_groups, ndim_groups] */
    void* out;                 /* fp16 (batch, nheads, dim) */
} QaSsmUpdateParams;

int qa_ssm_state_update(const QaSsmUpdateParams* p, void* stream);

/* One Mamba1 decode step in one launch: the conv's single-step update (qa_causal_conv1d_update on `conv`) and the
 * state update (qa_ssm_state_update on `p`), the state update taking the conv's int8 output as its x (p->x is not
 * read).  Replaces the pair quant_causal_conv1d_cuda.update (csrc/causal_conv1d/quant_causal_conv1d.cpp, kernel
 * quant_causal_conv1d_update_kernel.cuh:34-75) + quant_sscan_cuda.update / selective_state_update
 * (quamba/triton/selective_state_update.py:83-126) for callers whose dt, B and C do not depend on the conv output of
 * the same step (a benchmark loop with given inputs; in the full Mamba1 layer x_proj sits between the two, so the
 * layer calls them separately).  Same bits as the two calls: conv_state and state are updated in place, conv->out
 * (may be null) receives the conv output.  One head (p->nheads == 1), d_state <= 16, per-tensor scales.
 * The reference layer's own layout - sixteen states, contiguous (batch, dim, 16) state and (dim, 16) A_log,
 * (batch, dim, 4) or contiguous (batch, dim, 3) conv state, four taps, int8 or no dt bias, dim a multiple of 64 for an
 * fp32 state - takes a kernel compiled for that shape (the state moves in 1 KB runs per wave); any other layout the
 * generic one.  The same holds for qa_ssm_state_update alone. */
int qa_mamba1_decode_step(const QaConvParams* conv, const QaSsmUpdateParams* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * W8A8 GEMM with scale epilogue:  D[m,n] = cast( s_a[m|0] * ( s_b[n|0] * float(sum_k a[m,k] w[n,k]) ) )
 * Replaces quant_linear_cuda.cutlass_scaled_mm_dq / cutlass_scaled_mv_dq / w8a8o8_gemv
 *   (csrc/linear/quant_linear_fwd_kernel.cuh:356-401, quant_linear_fwd_gemv_kernel.cuh:96-134).
 * Both operands are K-contiguous: a is (M,K) with row stride lda; w is (N,K) with row stride ldw
 * (the reference's column-major (K,N) "b" operand is the same memory).
 * ---------------------------------------------------------------------------------------- */
/* BF16 (round to nearest even, csrc/linear/quant_linear_fwd_kernel.cuh:312-316) is an output of the W8A8 GEMM only. */
typedef enum QaOutType { QA_OUT_I8 = 0, QA_OUT_F16 = 1, QA_OUT_BF16 = 2 } QaOutType;
/* QA_ROUND_HALF_AWAY selects the rule of w8a8o8_gemv: d = sat8(roundf((s_w[n] * s_a[m|0]) * float(acc))) */
typedef enum QaRound { QA_ROUND_RNE = 0, QA_ROUND_HALF_AWAY = 1 } QaRound;

typedef struct QaGemmW8A8Params {
    int32_t m, n, k;
    int32_t out_type;      /* QaOutType */
    int32_t round_mode;    /* QaRound, int8 output only */
    int32_t a_scale_numel; /* 1 or m */
    int32_t w_scale_numel; /* 1 or n */
    int32_t use_alpha;     /* 1: d = cast(alpha * float(acc)) with the host scalar below (the GEMV
                              rule of cutlass_scaled_mv_dq); the scale pointers are then ignored */
    float alpha;
    int32_t scale_order;   /* 0: D = s_a[m] * (s_b[n] * acc) as above; 1: D = s_b[n] * (s_a[m] * acc), the
                              association a caller needs when it exchanges the roles of the two operands
                              to obtain the (N,M) output of a product defined the first way */
    int64_t lda, ldw, ldd; /* element strides between rows of a, w, d (d is (M,N) row-major) */
    const int8_t* a;
    const int8_t* w;
    const float* a_scale;  /* device */
    const float* w_scale;  /* device */
    void* d;               /* int8 or fp16 */
} QaGemmW8A8Params;

int qa_gemm_w8a8(const QaGemmW8A8Params* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * W4A8 GEMM (int4 weights, group-wise fp16 scales, int8 activations).
 * Replaces quant_linear_cuda.w4a8o8_gemm / w4a8o16_gemm
 *   (csrc/linear/marlin_qqq_gemm_kernel.cuh:1187-1314, marlin_qqq_gemm_kernel_o8.cuh).
 * Weights are held in this library's own packing (below); k must be a multiple of 128; arithmetic is the
 * reference's: w8 = rne((q4-8) * s_group) as int8, int32 accumulation, out = (acc*s_ch[n])*s_tok[m|0].
 * ---------------------------------------------------------------------------------------- */
typedef struct QaGemmW4A8Params {
    int32_t m, n, k;
    int32_t group_size;      /* 128, or -1 for per-channel (w8 = 16 * (q4 - 8)) */
    int32_t out_type;        /* QaOutType */
    int32_t tok_scale_numel; /* 1 or m */
    int32_t output_transpose;/* 0: d is (M,N); 1: d is (N,M) */
    int32_t reserved0;
    int64_t lda, ldd;
    const int8_t* a;         /* (M,K) */
    const uint8_t* w_packed; /* (N, K/2): per row, each aligned group of 8 codes is 4 bytes; byte i holds
                                code[8w+i] in the low nibble and code[8w+4+i] in the high nibble.
                                Grouped: code in [0,15] meaning code-8; per-channel: signed nibble. */
    const void* s_group;     /* fp16 (K/group_size, N) or null when per-channel */
    const float* s_channel;  /* fp32 (N) */
    const float* s_token;    /* fp32 (1) or (M) */
    void* d;
    /* Optional scratch of n*k bytes (16-byte aligned), or null.  With many activation rows every 256-row
     * band of the output expands the same 4-bit weights again; given this buffer (and more than 64 rows)
     * the weights are expanded once (same arithmetic, same int8 values) and the int8 x int8 kernel runs on
     * the result, for the (N,M) output with the roles of the operands exchanged.  It pays from about 1000
     * activation rows on; whether to pass it is the caller's choice.  Results are bit-identical either way. */
    void* w8_workspace;
    int64_t w8_workspace_bytes;
} QaGemmW4A8Params;

int qa_gemm_w4a8(const QaGemmW4A8Params* p, void* stream);

/* ------------------------------------------------------------------------------------------
 * Mamba2 quantized SSD chunk scan (prefill).
 * Replaces _quant_mamba_chunk_scan_combined_fwd / _quamba2_mamba_chunk_scan_combined_fwd
 *   (quamba/triton/quant_ssd_combined.py:11-81, :84-166).
 * Workspace is supplied by the caller (size from qa_ssd_workspace_bytes).
 * ---------------------------------------------------------------------------------------- */
typedef struct QaSsdParams {
    int32_t batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size;
    int32_t dt_softplus;
    int32_t dt_is_fp32;          /* 0: int8 dt + dt_scale + fp16 dt_bias; 1: fp32 dt already processed */
    int32_t D_has_hdim;          /* D is (nheads, headdim) instead of (nheads) */
    int32_t nhead_groups, ndim_groups;  /* 0 = per-tensor x scale */
    int32_t final_state_is_fp32; /* 1: fp32 final states, 0: int8 with state scale */
    int32_t reserved0;
    float dt_min, dt_max;        /* clamp after softplus */
    const int8_t* x;             /* (batch, seqlen, nheads, headdim) contiguous */
    const void* dt;              /* int8 or fp32 (batch, seqlen, nheads) contiguous */
    const int8_t* A_log;         /* (nheads) */
    const int8_t* B;             /* (batch, seqlen, ngroups, dstate) contiguous */
    const int8_t* C;
    const int8_t* D;             /* or null */
    const int8_t* z;             /* (batch, seqlen, nheads, headdim) or null */
    const void* dt_bias;         /* fp16 (nheads) or null */
    const float* x_scale;        /* (1) or [ngroups, nhead_groups, ndim_groups] */
    const float* dt_scale;
    const float* A_log_scale;
    const float* B_scale;        /* (1) or [ngroups] */
    const float* C_scale;
    const float* D_scale;
    const float* z_scale;
    const float* state_scale;    /* (1) or [ngroups, nhead_groups, ndim_groups, dstate] */
    const int32_t* x_head_group_range;
    const int32_t* x_dim_group_range;
    void* out;                   /* fp16 (batch, seqlen, nheads, headdim) */
    void* final_states;          /* fp32 or int8 (batch, nheads, headdim, dstate), or null */
    void* workspace;
    int64_t workspace_bytes;
} QaSsdParams;

/* Any headdim up to 256, dstate up to 1024 and chunk_size up to 1024, like the reference's launchers
 * (quamba/triton/quant_chunk_scan.py:286-414); beyond that QA_ERR_UNSUPPORTED (qa_ssd_workspace_bytes: 0).
 * Two sets of kernels with the same arithmetic and rounding points: matrix-core kernels for headdim 64, 128, 192 or
 * 256 with dstate 64 or 128, chunk_size 64, 128 or 256 and 16-byte aligned x, B, C, z, out (and D when it has
 * one weight per channel) - the shapes of the released models; general kernels for everything else, three to four
 * times slower.  The workspace has the same size either way.  The launches are one-dimensional grids: batch *
 * chunks * nheads * headdim / 64 (general kernels: * ceil(chunk_size / 64) as well) must fit 2^31 - 1, else
 * QA_ERR_SHAPE. */
int64_t qa_ssd_workspace_bytes(const QaSsdParams* p);
int qa_ssd_chunk_scan_fwd(const QaSsdParams* p, void* stream);

/* qa_ssd_chunk_scan_fwd for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its launcher allocates its
 * intermediates with torch.empty on every call, quamba/triton/quant_ssd_combined.py:61-77).  The caller passes
 * inputs and outputs as usual; `workspace` and `workspace_bytes` are ignored: the intermediates live in a fixed
 * buffer of QA_SSD_STATIC_SCRATCH_BYTES (64 MiB) that is part of the library's device image - every GPU the
 * library runs on holds it until the process ends.  A problem whose qa_ssd_workspace_bytes() exceeds that size
 * returns QA_ERR_SCRATCH.  The call allocates nothing and frees nothing; same kernels, same results as
 * qa_ssd_chunk_scan_fwd.  All calls on one GPU share the buffer: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream, or ordered by events, do not.  Nothing in the buffer has to start at zero.
 * The first call on a device looks the buffer's address up and raises the kernels' LDS limit (two runtime calls
 * that do not belong under stream capture): make one ordinary call on a device before capturing this entry point
 * into a HIP graph.  The size check comes before any runtime call. */
#define QA_SSD_STATIC_SCRATCH_BYTES (64ll << 20)
int qa_ssd_chunk_scan_fwd_noalloc(const QaSsdParams* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QUAMBA_AMD_H */
