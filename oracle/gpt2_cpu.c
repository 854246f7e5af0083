/*
 * CPU oracle for the GPT-2 fp32 forward pass.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP kernels are compared against.  It is never
 * linked into, imported by or called from the product library; only tests,
 * the smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * It restates, in plain C + OpenMP, the CPU forward pass of llm.c
 * (train_gpt2.c), which is the fp32 path the reference's kernels replace
 * (reference README.md:19).  llm.c itself is not available offline, so each
 * function follows llm.c's published per-element arithmetic:
 *
 *   encoder   out = wte[ix] + wpe[t]
 *   layernorm two-pass: m = sum(x)/C ; v = sum((x-m)^2)/C ; s = 1/sqrtf(v+1e-5f)
 *             out = (s*(x-m))*w + b                (the reference's GPU kernels
 *             use the single-pass E[x^2]-m^2 form, 3_layernorm_warp.cuh:49-50;
 *             the oracle keeps llm.c's two-pass CPU form)
 *   matmul    val = bias ? bias[o] : 0 ; for i<C: val += inp[bt,i]*W[o,i]
 *             (weight is (OC,C) row-major: 2_matmul_cublas.cuh:44-54)
 *   attention causal softmax((q.k)*1/sqrtf(hs)) . v from packed qkv (B,T,3C)
 *             (layout: 3_flash_attention_permute.cuh:46-58, permute.cuh:22-24)
 *   gelu      0.5x(1+tanhf(sqrtf(2/pi)(x+0.044715x^3)))
 *             (9_matmul_async_cg_tf32_gelu.cuh:5-11)
 *   residual  out = a + b                         (1_residual_naive.cuh:5-13)
 *
 * All arithmetic is IEEE fp32 with separate multiply and add (the file must be
 * compiled with -ffp-contract=off); sums run in the index order written here.
 *
 * Pinning status.  The reference ships no golden vectors, fixtures or tests
 * for this path, so nothing here can be pinned against reference-held data.
 * Every function is instead pinned by tests/test_oracle.py against what the
 * mathematics fixes: float64 brute force on small shapes, closed forms
 * (identity weights, constant rows, T=1 attention, q=0 attention = running
 * mean of v), invariants (causality, row-stochastic weights, odd-part identity
 * of gelu) and library routines (torch CPU layer_norm / linear / gelu /
 * scaled_dot_product_attention).  What stays unpinned: bit-for-bit agreement
 * with an upstream llm.c binary's summation order ("parity unpinned" for
 * last-ulp behaviour only; tolerances in the tests are far above that).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* out[b,t,:] = wte[inp[b,t],:] + wpe[t,:] */
ORACLE_API void oracle_encoder_forward(float* out, const int* inp, const float* wte,
                                       const float* wpe, int B, int T, int C) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < B; b++) {
    for (int t = 0; t < T; t++) {
      float* o = out + ((size_t)b * T + t) * C;
      const float* we = wte + (size_t)inp[b * T + t] * C;
      const float* pe = wpe + (size_t)t * C;
      for (int i = 0; i < C; i++) o[i] = we[i] + pe[i];
    }
  }
}

/* Two-pass layernorm over the last dimension; also stores mean and rstd. */
ORACLE_API void oracle_layernorm_forward(float* out, float* mean, float* rstd, const float* inp,
                                         const float* weight, const float* bias, int B, int T,
                                         int C) {
  const float eps = 1e-5f;
  const size_t N = (size_t)B * T;
#pragma omp parallel for
  for (size_t r = 0; r < N; r++) {
    const float* x = inp + r * C;
    float m = 0.0f;
    for (int i = 0; i < C; i++) m += x[i];
    m = m / C;
    float v = 0.0f;
    for (int i = 0; i < C; i++) {
      float xs = x[i] - m;
      v += xs * xs;
    }
    v = v / C;
    float s = 1.0f / sqrtf(v + eps);
    float* o = out + r * C;
    for (int i = 0; i < C; i++) {
      float n = s * (x[i] - m);
      o[i] = n * weight[i] + bias[i];
    }
    if (mean) mean[r] = m;
    if (rstd) rstd[r] = s;
  }
}

ORACLE_API void oracle_residual_forward(float* out, const float* inp1, const float* inp2,
                                        size_t N) {
#pragma omp parallel for
  for (size_t i = 0; i < N; i++) out[i] = inp1[i] + inp2[i];
}

/* res = inp1 + inp2 ; ln = layernorm(res).  The composition of the two
 * functions above, which is what the reference's fused kernel is meant to
 * compute (fused_residual_layernorm.cuh:26-85). */
ORACLE_API void oracle_fused_residual_layernorm_forward(float* res_out, float* ln_out, float* mean,
                                                        float* rstd, const float* inp1,
                                                        const float* inp2, const float* weight,
                                                        const float* bias, int B, int T, int C) {
  oracle_residual_forward(res_out, inp1, inp2, (size_t)B * T * C);
  oracle_layernorm_forward(ln_out, mean, rstd, res_out, weight, bias, B, T, C);
}

ORACLE_API void oracle_gelu_forward(float* out, const float* inp, size_t N) {
  const float k = sqrtf(2.0f / (float)M_PI);
#pragma omp parallel for
  for (size_t i = 0; i < N; i++) {
    float x = inp[i];
    float cube = 0.044715f * x * x * x;
    out[i] = 0.5f * x * (1.0f + tanhf(k * (x + cube)));
  }
}

/* The textbook triple loop, kept as the definition the blocked version below
 * must reproduce bit for bit. */
ORACLE_API void oracle_matmul_forward_naive(float* out, const float* inp, const float* weight,
                                            const float* bias, int B, int T, int C, int OC) {
  const size_t N = (size_t)B * T;
#pragma omp parallel for
  for (size_t bt = 0; bt < N; bt++) {
    const float* x = inp + bt * C;
    for (int o = 0; o < OC; o++) {
      float val = bias ? bias[o] : 0.0f;
      const float* w = weight + (size_t)o * C;
      for (int i = 0; i < C; i++) val += x[i] * w[i];
      out[bt * OC + o] = val;
    }
  }
}

/* Same per-output arithmetic as the naive loop (start from the bias, then add
 * x[i]*w[o,i] for i = 0..C-1, one rounding per multiply and per add), but
 * blocked so that it vectorises ACROSS outputs: a panel of PANEL weight rows
 * is transposed to (C, PANEL) and ROWS input rows are carried together.  No
 * sum is reassociated, so the result is bit-identical to the naive loop. */
#define PANEL 32
#define ROWS 8
ORACLE_API void oracle_matmul_forward(float* out, const float* inp, const float* weight,
                                      const float* bias, int B, int T, int C, int OC) {
  const size_t N = (size_t)B * T;
  const int npanel = (OC + PANEL - 1) / PANEL;
  const size_t chunk = 512; /* input rows per work item */
  const int nchunk = (int)((N + chunk - 1) / chunk);
#pragma omp parallel
  {
    float* wt = (float*)aligned_alloc(64, (size_t)C * PANEL * sizeof(float));
#pragma omp for collapse(2) schedule(dynamic, 1)
    for (int p = 0; p < npanel; p++) {
      for (int ch = 0; ch < nchunk; ch++) {
        const int o0 = p * PANEL;
        const int on = (OC - o0 < PANEL) ? (OC - o0) : PANEL;
        for (int i = 0; i < C; i++) {
          for (int j = 0; j < PANEL; j++)
            wt[(size_t)i * PANEL + j] = (j < on) ? weight[(size_t)(o0 + j) * C + i] : 0.0f;
        }
        float b0[PANEL];
        for (int j = 0; j < PANEL; j++) b0[j] = (bias && j < on) ? bias[o0 + j] : 0.0f;
        const size_t r0 = (size_t)ch * chunk;
        const size_t r1 = (r0 + chunk < N) ? (r0 + chunk) : N;
        size_t r = r0;
        for (; r + ROWS <= r1; r += ROWS) {
          float acc[ROWS][PANEL];
          for (int q = 0; q < ROWS; q++)
            for (int j = 0; j < PANEL; j++) acc[q][j] = b0[j];
          for (int i = 0; i < C; i++) {
            const float* w = wt + (size_t)i * PANEL;
            for (int q = 0; q < ROWS; q++) {
              const float x = inp[(r + q) * C + i];
#pragma omp simd
              for (int j = 0; j < PANEL; j++) acc[q][j] += x * w[j];
            }
          }
          for (int q = 0; q < ROWS; q++)
            for (int j = 0; j < on; j++) out[(r + q) * OC + o0 + j] = acc[q][j];
        }
        for (; r < r1; r++) {
          float acc[PANEL];
          for (int j = 0; j < PANEL; j++) acc[j] = b0[j];
          for (int i = 0; i < C; i++) {
            const float* w = wt + (size_t)i * PANEL;
            const float x = inp[r * C + i];
#pragma omp simd
            for (int j = 0; j < PANEL; j++) acc[j] += x * w[j];
          }
          for (int j = 0; j < on; j++) out[r * OC + o0 + j] = acc[j];
        }
      }
    }
    free(wt);
  }
}

/* Causal multi-head self-attention on packed qkv (B,T,3C): q at column 0, k at
 * +C, v at +2C, head h at h*hs inside each.  out is (B,T,C).  Follows llm.c's
 * four passes per (b,t,h): scaled scores with running max (start -10000),
 * exp and sum, normalise, weighted sum of v in key order.  The score row lives
 * in a per-thread scratch of T floats instead of llm.c's (B,NH,T,T) buffers. */
ORACLE_API void oracle_attention_forward(float* out, const float* inp, int B, int T, int C,
                                         int NH) {
  const int C3 = 3 * C;
  const int hs = C / NH;
  const float scale = 1.0f / sqrtf((float)hs);
#pragma omp parallel
  {
    float* att = (float*)malloc((size_t)T * sizeof(float));
#pragma omp for collapse(3) schedule(dynamic, 16)
    for (int b = 0; b < B; b++) {
      for (int t = 0; t < T; t++) {
        for (int h = 0; h < NH; h++) {
          const float* q = inp + ((size_t)b * T + t) * C3 + h * hs;
          float maxval = -10000.0f;
          for (int t2 = 0; t2 <= t; t2++) {
            const float* k = inp + ((size_t)b * T + t2) * C3 + h * hs + C;
            float val = 0.0f;
            for (int i = 0; i < hs; i++) val += q[i] * k[i];
            val *= scale;
            if (val > maxval) maxval = val;
            att[t2] = val;
          }
          float expsum = 0.0f;
          for (int t2 = 0; t2 <= t; t2++) {
            float e = expf(att[t2] - maxval);
            expsum += e;
            att[t2] = e;
          }
          const float inv = (expsum == 0.0f) ? 0.0f : 1.0f / expsum;
          for (int t2 = 0; t2 <= t; t2++) att[t2] *= inv;
          float* o = out + ((size_t)b * T + t) * C + h * hs;
          for (int i = 0; i < hs; i++) o[i] = 0.0f;
          for (int t2 = 0; t2 <= t; t2++) {
            const float* v = inp + ((size_t)b * T + t2) * C3 + h * hs + 2 * C;
            const float a = att[t2];
            for (int i = 0; i < hs; i++) o[i] += a * v[i];
          }
        }
      }
    }
    free(att);
  }
}

/* ids[r] = argmax_v logits[r,v]; the lowest index wins ties. */
ORACLE_API void oracle_argmax_forward(int* ids, const float* logits, int N, int V) {
#pragma omp parallel for
  for (int r = 0; r < N; r++) {
    const float* x = logits + (size_t)r * V;
    int best = 0;
    float bv = x[0];
    for (int v = 1; v < V; v++) {
      if (x[v] > bv) {
        bv = x[v];
        best = v;
      }
    }
    ids[r] = best;
  }
}

/* ---- whole model ------------------------------------------------------- */

/* Parameter tensors in llm.c checkpoint order. */
enum { P_WTE, P_WPE, P_LN1W, P_LN1B, P_QKVW, P_QKVB, P_ATTPROJW, P_ATTPROJB, P_LN2W, P_LN2B,
       P_FCW, P_FCB, P_FCPROJW, P_FCPROJB, P_LNFW, P_LNFB, P_COUNT };

ORACLE_API void oracle_param_sizes(size_t* sizes, int maxT, int V, int L, int C) {
  const size_t l = (size_t)L, c = (size_t)C;
  sizes[P_WTE] = (size_t)V * c;
  sizes[P_WPE] = (size_t)maxT * c;
  sizes[P_LN1W] = l * c;
  sizes[P_LN1B] = l * c;
  sizes[P_QKVW] = l * 3 * c * c;
  sizes[P_QKVB] = l * 3 * c;
  sizes[P_ATTPROJW] = l * c * c;
  sizes[P_ATTPROJB] = l * c;
  sizes[P_LN2W] = l * c;
  sizes[P_LN2B] = l * c;
  sizes[P_FCW] = l * 4 * c * c;
  sizes[P_FCB] = l * 4 * c;
  sizes[P_FCPROJW] = l * c * 4 * c;
  sizes[P_FCPROJB] = l * c;
  sizes[P_LNFW] = c;
  sizes[P_LNFB] = c;
}

ORACLE_API size_t oracle_num_parameters(int maxT, int V, int L, int C) {
  size_t s[P_COUNT], n = 0;
  oracle_param_sizes(s, maxT, V, L, C);
  for (int i = 0; i < P_COUNT; i++) n += s[i];
  return n;
}

/* Forward pass over a flat parameter buffer.  logits is (B,T,V) (no vocabulary
 * padding, no softmax); ids, if not NULL, receives the per-position argmax;
 * lnf_out, if not NULL, receives the final layernorm output (B,T,C).
 * Activations are reused from layer to layer.  Returns 0, or -1 if out of
 * memory or the shape is invalid. */
ORACLE_API int oracle_gpt2_forward(float* logits, int* ids, float* lnf_out, const float* params,
                                   const int* inputs, int B, int T, int maxT, int V, int L, int NH,
                                   int C) {
  if (T > maxT || C % NH != 0) return -1;
  size_t sz[P_COUNT];
  const float* p[P_COUNT];
  oracle_param_sizes(sz, maxT, V, L, C);
  const float* cur = params;
  for (int i = 0; i < P_COUNT; i++) {
    p[i] = cur;
    cur += sz[i];
  }
  const size_t N = (size_t)B * T, c = (size_t)C;
  float* residual = (float*)malloc(N * c * sizeof(float));
  float* residual2 = (float*)malloc(N * c * sizeof(float));
  float* ln = (float*)malloc(N * c * sizeof(float));
  float* qkv = (float*)malloc(N * 3 * c * sizeof(float));
  float* atty = (float*)malloc(N * c * sizeof(float));
  float* proj = (float*)malloc(N * c * sizeof(float));
  float* fch = (float*)malloc(N * 4 * c * sizeof(float));
  float* fch_gelu = (float*)malloc(N * 4 * c * sizeof(float));
  int rc = -1;
  if (residual && residual2 && ln && qkv && atty && proj && fch && fch_gelu) {
    oracle_encoder_forward(residual, inputs, p[P_WTE], p[P_WPE], B, T, C);
    for (int l = 0; l < L; l++) {
      oracle_layernorm_forward(ln, NULL, NULL, residual, p[P_LN1W] + l * c, p[P_LN1B] + l * c, B,
                               T, C);
      oracle_matmul_forward(qkv, ln, p[P_QKVW] + l * 3 * c * c, p[P_QKVB] + l * 3 * c, B, T, C,
                            3 * C);
      oracle_attention_forward(atty, qkv, B, T, C, NH);
      oracle_matmul_forward(proj, atty, p[P_ATTPROJW] + l * c * c, p[P_ATTPROJB] + l * c, B, T, C,
                            C);
      oracle_residual_forward(residual2, residual, proj, N * c);
      oracle_layernorm_forward(ln, NULL, NULL, residual2, p[P_LN2W] + l * c, p[P_LN2B] + l * c, B,
                               T, C);
      oracle_matmul_forward(fch, ln, p[P_FCW] + l * 4 * c * c, p[P_FCB] + l * 4 * c, B, T, C,
                            4 * C);
      oracle_gelu_forward(fch_gelu, fch, N * 4 * c);
      oracle_matmul_forward(proj, fch_gelu, p[P_FCPROJW] + l * 4 * c * c, p[P_FCPROJB] + l * c, B,
                            T, 4 * C, C);
      oracle_residual_forward(residual, residual2, proj, N * c);
    }
    oracle_layernorm_forward(ln, NULL, NULL, residual, p[P_LNFW], p[P_LNFB], B, T, C);
    if (lnf_out) memcpy(lnf_out, ln, N * c * sizeof(float));
    oracle_matmul_forward(logits, ln, p[P_WTE], NULL, B, T, C, V);
    if (ids) oracle_argmax_forward(ids, logits, (int)N, V);
    rc = 0;
  }
  free(residual); free(residual2); free(ln); free(qkv); free(atty); free(proj); free(fch);
  free(fch_gelu);
  return rc;
}
