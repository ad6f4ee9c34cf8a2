/*
 * qoracle.c - CPU restatement of the reference's quantized Mamba mixer arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (quamba_amd/) may link, load or call this
 * file; it is the checker the GPU kernels are compared with, and the CPU baseline bench.py times.
 *
 * Every function follows the reference kernel named above it (paths relative to the root of
 * enyac-group/Quamba), operation for operation in fp32, on dense row-major arrays.
 * Where the CUDA compiler contracts a*b+c into one FMA (its default), the FMA is written out.
 * Compile with -ffp-contract=off so no other contraction happens.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------------------------------
 * exp used by the int8-output ops.  The reference calls expf under --use_fast_math, whose low
 * bits are not reproducible off its GPU; this build defines exp as the following fixed fp32
 * sequence (Cody-Waite reduction by ln2 in two FMAs, degree-7 Taylor polynomial in Horner form,
 * exact scaling by 2^n), so that results are reproducible bit for bit.  tests pin it to libm's
 * expf within 2 ulp.
 * ------------------------------------------------------------------------------------------- */
float qo_expf(float x) {
    if (x > 88.0f) return INFINITY;
    if (x < -87.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);
    r = fmaf(n, -1.42860682030941723e-6f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    int e = (int)n;
    uint32_t bits = (uint32_t)(e + 127) << 23;
    float s;
    memcpy(&s, &bits, 4);
    return p * s;
}

/* roundf = half away from zero, then clamp to int8 (quant_causal_conv1d_fwd_kernel.cuh:149-150) */
static int8_t sat8_half_away(float v) {
    float r = roundf(v);
    r = fmaxf(r, -128.0f);
    r = fminf(r, 127.0f);
    return (int8_t)(int)r;
}

/* rint = half to even, then clamp (quamba/triton/quant_ssm_states.py:43) */
static int8_t sat8_rne(float v) {
    float r = rintf(v);
    r = fmaxf(r, -128.0f);
    r = fminf(r, 127.0f);
    return (int8_t)(int)r;
}

int qo_sat8_half_away(float v) { return sat8_half_away(v); }
int qo_sat8_rne(float v) { return sat8_rne(v); }

static float conv_finish(float v, float s_out, int silu) {
    if (silu) v = v / (1.0f + qo_expf(-v));      /* quant_causal_conv1d_fwd_kernel.cuh:139-144 */
    return v / s_out;                            /* :149 */
}

/*
 * Causal depthwise conv forward on x int8 (batch, dim, seqlen), weight int8 (dim, width).
 * tapwise == 0: seqlen-contiguous kernel, quant_causal_conv1d_fwd_kernel.cuh:57-157
 *     out_tmp = sum_w W[w] * x[t-(width-1-w)]  (fp32, exact integers), v = s_wx*out_tmp + bias (:130-136)
 * tapwise == 1: channel-contiguous kernel, quant_causal_conv1d_fwd_kernel.cuh:340-375
 *     v = s_b*bias; v += s_wx * W[w] * x[..] per tap (:356-362)
 */
void qo_conv1d_fwd(const int8_t* x, const int8_t* weight, const int8_t* bias, int8_t* out,
                   int batch, int dim, int seqlen, int width,
                   float s_x, float s_w, float s_b, float s_out, int silu, int tapwise) {
    const float s_wx = s_w * s_x;                                           /* :62 */
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            const int8_t* xr = x + ((int64_t)b * dim + d) * seqlen;
            int8_t* orow = out + ((int64_t)b * dim + d) * seqlen;
            const int8_t* w = weight + (int64_t)d * width;
            const float bias_f = bias ? (float)bias[d] * s_b : 0.0f;        /* :80-81 */
            for (int t = 0; t < seqlen; ++t) {
                float v;
                if (!tapwise) {
                    float acc = 0.0f;
                    for (int k = 0; k < width; ++k) {
                        const int ti = t - (width - 1 - k);
                        const float xv = ti >= 0 ? (float)xr[ti] : 0.0f;
                        acc += (float)w[k] * xv;                            /* exact in fp32 */
                    }
                    v = fmaf(s_wx, acc, bias_f);
                } else {
                    v = bias_f;
                    for (int k = 0; k < width; ++k) {
                        const int ti = t - (width - 1 - k);
                        const float xv = ti >= 0 ? (float)xr[ti] : 0.0f;
                        v = fmaf(s_wx * (float)w[k], xv, v);
                    }
                }
                orow[t] = sat8_half_away(conv_finish(v, s_out, silu));
            }
        }
    }
}

/*
 * Single-step conv update, quant_causal_conv1d_update_kernel.cuh:34-75.
 * x int8 (batch, dim); state int8 (batch, dim, state_len) shifted in place; state_len is width
 * (the reference's layout: slot 0 is dropped) or width-1 (only the live history).
 */
void qo_conv1d_update(const int8_t* x, int8_t* state, const int8_t* weight, const int8_t* bias, int8_t* out,
                      int batch, int dim, int width, int state_len,
                      float s_x, float s_w, float s_b, float s_out, int silu) {
    const int drop = state_len - (width - 1);
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            int8_t* st = state + ((int64_t)b * dim + d) * state_len;
            const int8_t* w = weight + (int64_t)d * width;
            int8_t xs[8];
            for (int i = 0; i < width - 1; ++i) xs[i] = st[i + drop];       /* :59-62 */
            xs[width - 1] = x[(int64_t)b * dim + d];
            for (int i = 0; i < state_len; ++i) st[i] = xs[i + (width - state_len)];   /* :63-66 */
            float v = bias ? (float)bias[d] * s_b : 0.0f;
            for (int i = 0; i < width; ++i) {
                v = fmaf(s_w * s_x * (float)w[i], (float)xs[i], v);         /* :68-70 */
            }
            out[(int64_t)b * dim + d] = sat8_half_away(conv_finish(v, s_out, silu));
        }
    }
}

/*
 * Mamba2 xBC conv with per-channel scales, quamba2_conv1d_fwd_kernel.cuh:215-262 (forward) and
 * quamba2_conv1d_update_kernel.cuh:134-143 (update).  The caller resolves, per channel of the
 * concatenated [x | B | C] input, s_in = weight scale * input scale of its part, s_bias, and the output
 * scale of its group (the range walk of fwd kernel :151-212 is restated in oracle/__init__.py).
 * x int8 (batch, dim, seqlen) seqlen-major here (the layout is not part of the arithmetic).
 *   forward: tmp = sum_w W[w]*x[t-(width-1-w)]; v = s_in*tmp + s_bias*bias (:233-237, contracted to one fma)
 *   update:  v = s_bias*bias; v += s_in*W[i]*x[i] per tap (:134-136)
 */
void qo_conv1d_fwd_perchannel(const int8_t* x, const int8_t* weight, const int8_t* bias, int8_t* out,
                              int batch, int dim, int seqlen, int width,
                              const float* s_in, const float* s_bias, const float* s_out, int silu) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            const int8_t* xr = x + ((int64_t)b * dim + d) * seqlen;
            int8_t* orow = out + ((int64_t)b * dim + d) * seqlen;
            const int8_t* w = weight + (int64_t)d * width;
            const float bias_f = bias ? s_bias[d] * (float)bias[d] : 0.0f;
            for (int t = 0; t < seqlen; ++t) {
                float acc = 0.0f;
                for (int k = 0; k < width; ++k) {
                    const int ti = t - (width - 1 - k);
                    const float xv = ti >= 0 ? (float)xr[ti] : 0.0f;
                    acc += (float)w[k] * xv;                                /* exact in fp32 */
                }
                const float v = fmaf(s_in[d], acc, bias_f);
                orow[t] = sat8_half_away(conv_finish(v, s_out[d], silu));   /* :238, :250-252 */
            }
        }
    }
}

void qo_conv1d_update_perchannel(const int8_t* x, int8_t* state, const int8_t* weight, const int8_t* bias,
                                 int8_t* out, int batch, int dim, int width, int state_len,
                                 const float* s_in, const float* s_bias, const float* s_out, int silu) {
    const int drop = state_len - (width - 1);
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            int8_t* st = state + ((int64_t)b * dim + d) * state_len;
            const int8_t* w = weight + (int64_t)d * width;
            int8_t xs[8];
            for (int i = 0; i < width - 1; ++i) xs[i] = st[i + drop];       /* update kernel :50-55 */
            xs[width - 1] = x[(int64_t)b * dim + d];
            for (int i = 0; i < state_len; ++i) st[i] = xs[i + (width - state_len)];
            float v = bias ? s_bias[d] * (float)bias[d] : 0.0f;             /* :134 */
            for (int i = 0; i < width; ++i) {
                v = fmaf(s_in[d] * (float)w[i], (float)xs[i], v);           /* :136 */
            }
            out[(int64_t)b * dim + d] = sat8_half_away(conv_finish(v, s_out[d], silu));   /* :137-141 */
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Mamba1 selective scan forward, quant_sscan_fwd_kernel.cuh:110-293.
 * u, delta, z int8 (batch, dim, seqlen); A_log int8 (dim, dstate); B, C int8 (batch, groups,
 * dstate, seqlen); D, delta_bias int8 (dim) or NULL.  y fp32 (batch, seqlen, dim) holds the value
 * the kernel converts to fp16 (:272 / :285; the transposition is quant_sscan.cpp:262).
 * The recurrence is evaluated sequentially (the kernel's block scan differs only in association).
 * state_i8 / state_f32 (batch, dim, dstate) receive the state after the last step (:240-241).
 * ------------------------------------------------------------------------------------------- */
static float softplus20(float v) { return v <= 20.0f ? log1pf(expf(v)) : v; }   /* :160 */

void qo_sscan_fwd(const int8_t* u, const int8_t* delta, const int8_t* A_log, const int8_t* B, const int8_t* C,
                  const int8_t* D, const int8_t* delta_bias, const int8_t* z,
                  float s_u, float s_delta, float s_A, float s_B, float s_C, float s_D, float s_db, float s_z,
                  float s_state, int batch, int dim, int seqlen, int dstate, int groups, int softplus,
                  float* y, int8_t* state_i8, float* state_f32) {
    const int per_group = dim / groups;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            const int g = d / per_group;
            const int8_t* ur = u + ((int64_t)b * dim + d) * seqlen;
            const int8_t* dr = delta + ((int64_t)b * dim + d) * seqlen;
            const int8_t* zr = z ? z + ((int64_t)b * dim + d) * seqlen : 0;
            const float D_f = D ? s_D * (float)D[d] : 0.0f;                          /* :115-118 */
            const float db = delta_bias ? s_db * (float)delta_bias[d] : 0.0f;        /* :121-128 */
            float h[256];
            float A[256];
            for (int n = 0; n < dstate; ++n) {
                h[n] = 0.0f;
                A[n] = -expf(s_A * (float)A_log[(int64_t)d * dstate + n]);           /* :173 */
            }
            for (int t = 0; t < seqlen; ++t) {
                const float u_val = s_u * (float)ur[t];                              /* :157 */
                float dt = fmaf(s_delta, (float)dr[t], db);                          /* :158 */
                if (softplus) dt = softplus20(dt);
                const float du = dt * u_val;                                         /* :162 */
                float acc = D_f * u_val;                                             /* :163 */
                for (int n = 0; n < dstate; ++n) {
                    const int64_t bc = (((int64_t)b * groups + g) * dstate + n) * seqlen + t;
                    const float a = expf(dt * A[n]);                                 /* :219 */
                    const float bb = s_B * (float)B[bc] * du;                        /* :221 */
                    h[n] = fmaf(a, h[n], bb);                    /* quant_sscan_common.h:124-127 */
                    acc = fmaf(h[n], s_C * (float)C[bc], acc);                       /* :246-249 */
                }
                if (zr) {
                    const float zv = s_z * (float)zr[t];
                    acc = acc * zv / (1.0f + expf(-zv));                             /* :271-272 */
                }
                y[((int64_t)b * seqlen + t) * dim + d] = acc;
            }
            for (int n = 0; n < dstate; ++n) {
                const int64_t si = ((int64_t)b * dim + d) * dstate + n;
                if (state_f32) state_f32[si] = h[n];
                if (state_i8) state_i8[si] = sat8_half_away(h[n] / s_state);         /* :240-241 */
            }
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Single-step state update, quamba/triton/selective_state_update.py:83-126 (Mamba1 layout:
 * one head, per-tensor scales).  state int8 (batch, dim, dstate) is dequantised, updated and
 * requantised in place with rint((h*1e2)/(s*1e2)) (:119); with state_f32 != NULL the fp32 state
 * is used instead and kept un-quantised.  y fp32 (batch, dim) is the value stored as fp16 and is
 * computed from the un-requantised state (:121).
 * ------------------------------------------------------------------------------------------- */
void qo_sscan_update(int8_t* state_i8, float* state_f32, const int8_t* x, const int8_t* dt, const int8_t* A_log,
                     const int8_t* B, const int8_t* C, const int8_t* D, const int8_t* dt_bias, const int8_t* z,
                     float s_x, float s_dt, float s_A, float s_B, float s_C, float s_D, float s_db, float s_z,
                     float s_state, int batch, int dim, int dstate, int softplus, float* y) {
    for (int b = 0; b < batch; ++b) {
        for (int d = 0; d < dim; ++d) {
            const int64_t i = (int64_t)b * dim + d;
            const float xv = s_x * (float)x[i];                                       /* :83 */
            float dtv = s_dt * (float)dt[i];                                          /* :87 */
            if (dt_bias) dtv += s_db * (float)dt_bias[d];                             /* :90 */
            if (softplus) dtv = softplus20(dtv);                                      /* :94 */
            float acc = 0.0f;
            for (int n = 0; n < dstate; ++n) {
                const int64_t si = i * dstate + n;
                float h = state_f32 ? state_f32[si] : s_state * (float)state_i8[si];  /* :85 */
                const float A = -expf(s_A * (float)A_log[(int64_t)d * dstate + n]);   /* :96 */
                const float dA = expf(A * dtv);                                       /* :97 */
                const float Bv = s_B * (float)B[(int64_t)b * dstate + n];             /* :106 */
                const float Cv = s_C * (float)C[(int64_t)b * dstate + n];             /* :107 */
                const float dB = Bv * dtv;                                            /* :114 */
                h = h * dA + dB * xv;                                                 /* :118 */
                if (state_f32) state_f32[si] = h;
                else state_i8[si] = sat8_rne((h * 1e2f) / (s_state * 1e2f));          /* :119 */
                acc += h * Cv;                                                        /* :121 */
            }
            if (D) acc += xv * (s_D * (float)D[d]);                                   /* :122-123 */
            if (z) {
                const float zv = s_z * (float)z[i];
                acc *= zv * (1.0f / (1.0f + expf(-zv)));                              /* :124-125 */
            }
            y[i] = acc;
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Single-step state update with heads, quamba/triton/selective_state_update.py:23-126 (per-tensor
 * scales, requantisation factor 1e2, :119) and :236-362 (Mamba2: x scale per (ssd group, head group,
 * dim group), state scale per (ssd group, head group, dim group, state), B / C scale per ssd group,
 * factor 1e6, :355).  Dense arrays: state (batch, nheads, dim, dstate) int8 or fp32, x / dt / z int8
 * (batch, nheads, dim), A_log int8 (nheads, dim, dstate), B / C int8 (batch, ngroups, dstate), D int8
 * (nheads, dim), dt_bias fp32 (nheads, dim) holding the value the kernel adds (:90-92 / :327).  The
 * kernel's TIE_HDIM branch (:98-105 / :333-340: dt, dt_bias and A_log are one value per head, passed
 * as stride-0 views) evaluates the same expressions on those values, so the caller expands the views.
 * Group lookup (:303-315): hg = #{j : h mod (H/G) >= head_range[g,j]}, dg = #{j : p >= dim_range[g,hg,j]}.
 * y fp32 (batch, nheads, dim) is the value stored as fp16, from the un-requantised state (:357).
 * ------------------------------------------------------------------------------------------- */
void qo_ssm_update_heads(int8_t* state_i8, float* state_f32, const int8_t* x, const int8_t* dt, const int8_t* A_log,
                         const int8_t* B, const int8_t* C, const int8_t* D, const float* dt_bias, const int8_t* z,
                         const float* x_scale, const float* state_scale, const float* s_B, const float* s_C,
                         const int32_t* head_range, const int32_t* dim_range,
                         float s_dt, float s_A, float s_D, float s_z,
                         int batch, int nheads, int dim, int dstate, int ngroups, int nhead_groups, int ndim_groups,
                         int softplus, float* y) {
    const int hpg = nheads / ngroups;
    const int grouped = nhead_groups > 0;
    const float K = grouped ? 1e6f : 1e2f;
    for (int b = 0; b < batch; ++b) {
        for (int h = 0; h < nheads; ++h) {
            const int g = h / hpg;
            int hg = 0;
            if (grouped) {
                for (int j = 0; j < nhead_groups; ++j) hg += (h % hpg) >= head_range[g * nhead_groups + j];   /* :306 */
            }
            const float sB = s_B[grouped ? g : 0], sC = s_C[grouped ? g : 0];                    /* :277-279 */
            for (int p = 0; p < dim; ++p) {
                int sidx = 0;
                if (grouped) {
                    int dg = 0;
                    const int32_t* dr = dim_range + (g * nhead_groups + hg) * ndim_groups;
                    for (int j = 0; j < ndim_groups; ++j) dg += p >= dr[j];                       /* :312 */
                    sidx = (g * nhead_groups + hg) * ndim_groups + dg;
                }
                const int64_t i = ((int64_t)b * nheads + h) * dim + p;
                const int64_t hp = (int64_t)h * dim + p;
                const float xv = x_scale[sidx] * (float)x[i];                                     /* :83 / :316 */
                float dtv = s_dt * (float)dt[i];                                                  /* :87 / :325 */
                if (dt_bias) dtv += dt_bias[hp];                                                  /* :90-92 / :327 */
                if (softplus) dtv = softplus20(dtv);
                float acc = 0.0f;
                for (int n = 0; n < dstate; ++n) {
                    const int64_t si = i * dstate + n;
                    const float sc = grouped ? state_scale[(int64_t)sidx * dstate + n] : state_scale[0];
                    float hv = state_f32 ? state_f32[si] : sc * (float)state_i8[si];              /* :85 / :323 */
                    const float A = -expf(s_A * (float)A_log[hp * dstate + n]);                   /* :96 / :331 */
                    const float dA = expf(A * dtv);                                               /* :97 / :332 */
                    const float Bv = sB * (float)B[((int64_t)b * ngroups + g) * dstate + n];      /* :107 / :342 */
                    const float Cv = sC * (float)C[((int64_t)b * ngroups + g) * dstate + n];
                    hv = hv * dA + (Bv * dtv) * xv;                                               /* :118 / :353 */
                    if (state_f32) state_f32[si] = hv;
                    else state_i8[si] = sat8_rne((hv * K) / (sc * K));                            /* :119 / :355 */
                    acc += hv * Cv;                                                               /* :121 / :357 */
                }
                if (D) acc += xv * (s_D * (float)D[hp]);                                          /* :123 / :359 */
                if (z) {
                    const float zv = s_z * (float)z[i];
                    acc *= zv * (1.0f / (1.0f + expf(-zv)));                                      /* :125 / :361 */
                }
                y[i] = acc;
            }
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * W8A8 GEMM, csrc/linear/quant_linear_fwd_kernel.cuh:63-130:
 *   acc = int32 sum_k a[m,k]*w[n,k];  d = s_a[m|0] * (s_b[n|0] * float(acc))  (:85-97)
 * out_f32 receives the fp32 value before the final cast; out_i8 its int8 cast (round to nearest
 * even, saturating, :98-100).  round_half_away selects the GEMV epilogue's roundf
 * (quant_linear_fwd_gemv_kernel.cuh:56-60).
 * ------------------------------------------------------------------------------------------- */
void qo_gemm_w8a8(const int8_t* a, const int8_t* w, const float* s_a, int s_a_numel, const float* s_b,
                  int s_b_numel, int m, int n, int k, int round_half_away, int32_t* acc_out, float* out_f32,
                  int8_t* out_i8) {
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            int32_t acc = 0;
            const int8_t* ar = a + (int64_t)i * k;
            const int8_t* wr = w + (int64_t)j * k;
            for (int kk = 0; kk < k; ++kk) acc += (int32_t)ar[kk] * (int32_t)wr[kk];
            const float sa = s_a[s_a_numel == 1 ? 0 : i];
            const float sb = s_b[s_b_numel == 1 ? 0 : j];
            /* GEMM epilogue :85-97; GEMV: scale = s_a*s_b first (quant_linear_fwd_gemv_kernel.cuh:56-58) */
            const float v = round_half_away ? (sb * sa) * (float)acc : sa * (sb * (float)acc);
            const int64_t o = (int64_t)i * n + j;
            if (acc_out) acc_out[o] = acc;
            if (out_f32) out_f32[o] = v;
            if (out_i8) out_i8[o] = round_half_away ? sat8_half_away(v) : sat8_rne(v);
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * W4A8 GEMM, csrc/linear/marlin_qqq_gemm_kernel.cuh:
 *   grouped (group 128):  w8 = low byte of ( rne_fp16( (code-8) * s_group + 1152 ) ) ^ 0x80  (:136-178)
 *       = int8( rint( (code-8) * s_group ) ): the fp16 FMA rounds the exact product once, to an
 *       integer because fp16 spacing is 1 in [1024,2048); values outside [-128,127] wrap.
 *   per channel (group_size < 0): w8 = code << 4 as int8, i.e. 16 * signed nibble (:127-132).
 *   acc = int32 sum_k a[m,k] * w8[k,n];  out = (float(acc) * s_channel[n]) * s_token[m|0]  (:744-749)
 *   int8 output: round to nearest even, saturating (marlin_qqq_gemm_kernel_o8.cuh:107-116).
 * codes: uint8 (N,K) one 4-bit code per byte; s_group: fp32 holding fp16 values, (K/128, N).
 * ------------------------------------------------------------------------------------------- */
void qo_gemm_w4a8(const int8_t* a, const uint8_t* codes, const float* s_group, const float* s_channel,
                  const float* s_token, int s_token_numel, int m, int n, int k, int group_size,
                  int8_t* w8_out, int32_t* acc_out, float* out_f32, int8_t* out_i8) {
    for (int j = 0; j < n; ++j) {
        for (int kk = 0; kk < k; ++kk) {
            const int code = codes[(int64_t)j * k + kk] & 0xf;
            int w;
            if (group_size > 0) {
                const float prod = (float)(code - 8) * s_group[(int64_t)(kk / group_size) * n + j];
                w = (int)rintf(prod) & 0xff;
            } else {
                w = (code << 4) & 0xff;
            }
            w8_out[(int64_t)j * k + kk] = (int8_t)(uint8_t)w;
        }
    }
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            int32_t acc = 0;
            const int8_t* ar = a + (int64_t)i * k;
            const int8_t* wr = w8_out + (int64_t)j * k;
            for (int kk = 0; kk < k; ++kk) acc += (int32_t)ar[kk] * (int32_t)wr[kk];
            const float v = ((float)acc * s_channel[j]) * s_token[s_token_numel == 1 ? 0 : i];
            const int64_t o = (int64_t)i * n + j;
            if (acc_out) acc_out[o] = acc;
            if (out_f32) out_f32[o] = v;
            if (out_i8) out_i8[o] = sat8_rne(v);
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Mamba2 quantized SSD chunk scan, quamba/triton/quant_ssd_combined.py:61-77 (per-tensor scales)
 * and :146-162 (head/dim-grouped scales).  Stages, each as its Triton kernel computes it:
 *   1 quant_chunk_cumsum.py:56-70      dt = clamp(softplus(s_dt q_dt + dt_bias)), 0 past seqlen;
 *                                      dA_cs = cumsum within the chunk of dt * A, A = -exp(s_A q_A)
 *   2 quant_chunk_state.py:76-89       S_c[p,n] = sum_k f16(x^[k,p]) * f16(B^[k,n] * exp(dA_last-dA_k) * dt_k)
 *   3 quant_state_passing.py:60-83     P_0 = 0; P_{c+1} = exp(dA_last,c) P_c + S_c; P_c kept as fp16
 *   4 quant_bmm_chunk.py:60-66         CB[m,k] = sum_n C^[m,n] B^[k,n]   (fp32)
 *   5 quant_chunk_scan.py:96-171       y[m,p] = exp(dA_m) sum_n f16(C^[m,n]) f16(P_c[p,n])
 *                                               + sum_{k<=m} f16(CB[m,k] exp(dA_m-dA_k) dt_k) f16(x^[k,p])
 *                                               + x^[m,p] D;   y *= z sigmoid(z) when z is given
 *   6 quant_ssm_states.py:43,119       final int8 = sat8(rint(f16(P_final)*K / (scale*K))), K = 1e2 (1e6 grouped)
 * Products of fp16 operands are accumulated in fp32 (the order of accumulation is the kernels' own).
 * x^ = s_x[g,hg,dg] q_x with the group looked up from cumulative end indices
 * (quant_chunk_state.py:202-214): hg = #{j : h mod (H/G) >= head_range[g,j]}, dg = #{j : p >= dim_range[g,hg,j]}.
 * ------------------------------------------------------------------------------------------- */
static float f16_round(float v) {
    /* round to nearest even fp16 and back (normal, subnormal, overflow to inf) */
    uint32_t x;
    memcpy(&x, &v, 4);
    const uint32_t sign = x & 0x80000000u;
    x &= 0x7fffffffu;
    float a;
    memcpy(&a, &x, 4);
    if (x >= 0x7f800000u) return v;                       /* inf / nan */
    if (a >= 65520.0f) { uint32_t inf = sign | 0x7f800000u; float r; memcpy(&r, &inf, 4); return r; }
    float r;
    if (a < 6.103515625e-05f) {                           /* subnormal half: multiples of 2^-24 */
        r = rintf(a * 16777216.0f) / 16777216.0f;
    } else {
        const uint32_t lsb = (x >> 13) & 1u;
        uint32_t y = x + 0xfffu + lsb;
        y &= 0xffffe000u;
        memcpy(&r, &y, 4);
    }
    uint32_t rb;
    memcpy(&rb, &r, 4);
    rb |= sign;
    memcpy(&r, &rb, 4);
    return r;
}

float qo_f16_round(float v) { return f16_round(v); }

typedef struct {
    int batch, seqlen, nheads, headdim, dstate, ngroups, chunk;
    int softplus, dt_is_f32, D_has_hdim, nhead_groups, ndim_groups;
    float dt_min, dt_max;
} QoSsdDims;

void qo_ssd_fwd(const QoSsdDims* d, const int8_t* x, const void* dt_in, const int8_t* A_log, const int8_t* Bm,
                const int8_t* Cm, const int8_t* D, const int8_t* z, const float* dt_bias,
                const float* x_scale, const int32_t* head_range, const int32_t* dim_range,
                float s_dt, float s_A, const float* s_B, const float* s_C, float s_D, float s_z,
                const float* state_scale,
                float* y, float* final_f32, int8_t* final_i8,
                float* dt_out, float* dA_out, float* cb_out, float* chunk_states_out, float* prev_states_out) {
    const int Bsz = d->batch, L = d->seqlen, H = d->nheads, P = d->headdim, N = d->dstate, G = d->ngroups, Q = d->chunk;
    const int nc = (L + Q - 1) / Q;
    const int hpg = H / G;
    const int grouped = d->nhead_groups > 0;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < Bsz; ++b) {
        for (int h = 0; h < H; ++h) {
            const int g = h / hpg;
            int hg = 0;
            if (grouped) {
                for (int j = 0; j < d->nhead_groups; ++j) hg += (h % hpg) >= head_range[g * d->nhead_groups + j];
            }
            float xs_p[256];          /* x scale per p */
            int dg_p[256];
            for (int p = 0; p < P; ++p) {
                int dg = 0;
                if (grouped) {
                    const int32_t* dr = dim_range + (g * d->nhead_groups + hg) * d->ndim_groups;
                    for (int j = 0; j < d->ndim_groups; ++j) dg += p >= dr[j];
                    xs_p[p] = x_scale[(g * d->nhead_groups + hg) * d->ndim_groups + dg];
                } else {
                    xs_p[p] = x_scale[0];
                }
                dg_p[p] = dg;
            }
            const float sB = grouped ? s_B[g] : s_B[0];
            const float sC = grouped ? s_C[g] : s_C[0];
            const float A = -expf(s_A * (float)A_log[h]);
            float* Pst = (float*)calloc((size_t)P * N, sizeof(float));      /* running state, fp32 */
            float* P16 = (float*)malloc((size_t)P * N * sizeof(float));     /* state entering the chunk, fp16 values */
            float* S = (float*)malloc((size_t)P * N * sizeof(float));
            float* dtc = (float*)malloc((size_t)Q * sizeof(float));
            float* dAc = (float*)malloc((size_t)Q * sizeof(float));
            float* cb = (float*)malloc((size_t)Q * Q * sizeof(float));
            for (int c = 0; c < nc; ++c) {
                const int t0 = c * Q;
                const int lim = L - t0 < Q ? L - t0 : Q;
                /* stage 1 */
                float run = 0.0f;
                for (int k = 0; k < Q; ++k) {
                    float dtv = 0.0f;
                    if (k < lim) {
                        const int64_t di = ((int64_t)b * L + t0 + k) * H + h;
                        if (d->dt_is_f32) {
                            dtv = ((const float*)dt_in)[di];
                        } else {
                            dtv = s_dt * (float)((const int8_t*)dt_in)[di];
                            if (dt_bias) dtv += dt_bias[h];
                            if (d->softplus) dtv = softplus20(dtv);
                            dtv = fminf(fmaxf(dtv, d->dt_min), d->dt_max);
                        }
                    }
                    dtc[k] = dtv;
                    run += dtv * A;
                    dAc[k] = run;
                    if (dt_out) dt_out[(((int64_t)b * H + h) * nc + c) * Q + k] = dtv;
                    if (dA_out) dA_out[(((int64_t)b * H + h) * nc + c) * Q + k] = run;
                }
                const float dA_last = dAc[Q - 1];
                /* stage 4: CB for this (b, c, g) (recomputed per head; identical for heads of a group) */
                for (int m = 0; m < Q; ++m) {
                    for (int k = 0; k < Q; ++k) {
                        float acc = 0.0f;
                        if (m < lim && k < lim) {
                            const int8_t* cr = Cm + (((int64_t)b * L + t0 + m) * G + g) * N;
                            const int8_t* br = Bm + (((int64_t)b * L + t0 + k) * G + g) * N;
                            int32_t iacc = 0;
                            for (int n = 0; n < N; ++n) iacc += (int32_t)cr[n] * (int32_t)br[n];
                            /* sum_n (sC c)(sB b): every product is exact up to the two scale roundings;
                               the integer sum times the scale product is the same value to fp32 accuracy */
                            acc = (sC * sB) * (float)iacc;
                        }
                        cb[(int64_t)m * Q + k] = acc;
                        if (cb_out && h % hpg == 0) cb_out[((((int64_t)b * nc + c) * G + g) * Q + m) * Q + k] = acc;
                    }
                }
                /* stage 3 (entering state) */
                for (int i = 0; i < P * N; ++i) P16[i] = f16_round(Pst[i]);
                if (prev_states_out) memcpy(prev_states_out + ((((int64_t)b * nc + c) * H + h) * P) * N, P16, (size_t)P * N * 4);
                /* stage 5 */
                for (int m = 0; m < lim; ++m) {
                    const int8_t* cr = Cm + (((int64_t)b * L + t0 + m) * G + g) * N;
                    const float scale_m = expf(dAc[m]);
                    for (int p = 0; p < P; ++p) {
                        float acc = 0.0f;
                        for (int n = 0; n < N; ++n) acc += f16_round(sC * (float)cr[n]) * P16[p * N + n];
                        acc *= scale_m;
                        for (int k = 0; k <= m; ++k) {
                            const float w = f16_round(cb[(int64_t)m * Q + k] * expf(dAc[m] - dAc[k]) * dtc[k]);
                            const float xv = f16_round(xs_p[p] * (float)x[(((int64_t)b * L + t0 + k) * H + h) * P + p]);
                            acc += w * xv;
                        }
                        const int64_t oi = (((int64_t)b * L + t0 + m) * H + h) * P + p;
                        if (D) {
                            const float Dv = s_D * (float)D[d->D_has_hdim ? h * P + p : h];
                            acc += (xs_p[p] * (float)x[oi]) * Dv;
                        }
                        if (z) {
                            const float zv = s_z * (float)z[oi];
                            acc *= zv * (1.0f / (1.0f + expf(-zv)));
                        }
                        y[oi] = acc;
                    }
                }
                /* stage 2 */
                for (int p = 0; p < P; ++p) {
                    for (int n = 0; n < N; ++n) {
                        float acc = 0.0f;
                        for (int k = 0; k < lim; ++k) {
                            const float xv = f16_round(xs_p[p] * (float)x[(((int64_t)b * L + t0 + k) * H + h) * P + p]);
                            const float bv = sB * (float)Bm[(((int64_t)b * L + t0 + k) * G + g) * N + n];
                            acc += xv * f16_round(bv * (expf(dA_last - dAc[k]) * dtc[k]));
                        }
                        S[p * N + n] = acc;
                    }
                }
                if (chunk_states_out) memcpy(chunk_states_out + ((((int64_t)b * nc + c) * H + h) * P) * N, S, (size_t)P * N * 4);
                /* stage 3 (update) */
                const float decay = expf(dA_last);
                for (int i = 0; i < P * N; ++i) Pst[i] = decay * Pst[i] + S[i];
            }
            for (int p = 0; p < P; ++p) {
                for (int n = 0; n < N; ++n) {
                    const int64_t si = (((int64_t)b * H + h) * P + p) * N + n;
                    const float v = Pst[p * N + n];
                    if (final_f32) final_f32[si] = v;
                    if (final_i8) {
                        const float K = grouped ? 1e6f : 1e2f;
                        const float sc = grouped ? state_scale[((g * d->nhead_groups + hg) * d->ndim_groups + dg_p[p]) * N + n]
                                                 : state_scale[0];
                        final_i8[si] = sat8_rne((f16_round(v) * K) / (sc * K));
                    }
                }
            }
            free(Pst); free(P16); free(S); free(dtc); free(dAc); free(cb);
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Hadamard transform + int8 quantisation of each row, csrc/hadamard/quant_hadamard_fwd.cu:153-229.
 * x fp32 (rows, dim) holds the input values already widened (the kernel widens on load,
 * fast_hadamard_transform_common.h:128-143); dim = S * M, M a power of two.  The kernel applies
 * butterflies (a+b, a-b) to the index bits of m from the lowest (registers, :84-104) through the lane
 * bits (:107-123: sign*x + other) to the warp bits, then the S-point matrix to the chunk index c
 * (element c*M + m, quant_hadamard_fwd.cu:203-224) as one left-to-right signed sum per output
 * (fast_hadamard_transform_special.h).  signs is that S x S matrix as +1/-1 (S == 1: unused).
 * Output: roundf(y * scale) (:147-154), saturated to int8 here.
 * ------------------------------------------------------------------------------------------- */
void qo_hadamard_quant(const float* x, int8_t* out, int rows, int dim, int S, const int8_t* signs, float scale) {
    const int M = dim / S;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        float* v = (float*)malloc(sizeof(float) * (size_t)dim);
        float tmp[64];
        for (int e = 0; e < dim; ++e) v[e] = x[(int64_t)r * dim + e];
        for (int stride = 1; stride < M; stride <<= 1) {
            for (int e = 0; e < dim; ++e) {
                if ((e & stride) == 0) {
                    const float a = v[e], b = v[e + stride];
                    v[e] = a + b;
                    v[e + stride] = a - b;
                }
            }
        }
        if (S > 1) {
            for (int m = 0; m < M; ++m) {
                for (int i = 0; i < S; ++i) {
                    float acc = signs[i * S] > 0 ? v[m] : -v[m];
                    for (int j = 1; j < S; ++j) {
                        acc = signs[i * S + j] > 0 ? acc + v[j * M + m] : acc - v[j * M + m];
                    }
                    tmp[i] = acc;
                }
                for (int i = 0; i < S; ++i) v[i * M + m] = tmp[i];
            }
        }
        for (int e = 0; e < dim; ++e) out[(int64_t)r * dim + e] = sat8_half_away(v[e] * scale);
        free(v);
    }
}
