/*
 * moe_oracle.c -- CPU restatement of the quantized MoE block (test infrastructure
 * only; see moe_oracle.h for what each function follows and how it is pinned).
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off: no fused contraction, so the
 * float results are the same on every x86-64 host).
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static _Thread_local char g_err[256];
const char *orc_last_error(void) { return g_err; }
static int fail(const char *msg) {
  snprintf(g_err, sizeof g_err, "%s", msg);
  return 1;
}

/* ------------------------------------------------------------------ bf16 */

uint16_t orc_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* quiet NaN */
  u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest, ties to even */
  return (uint16_t)(u >> 16);
}
float orc_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
void orc_f32_to_bf16_n(const float *s, uint16_t *d, int64_t n) {
  for (int64_t i = 0; i < n; ++i) d[i] = orc_f32_to_bf16(s[i]);
}
void orc_bf16_to_f32_n(const uint16_t *s, float *d, int64_t n) {
  for (int64_t i = 0; i < n; ++i) d[i] = orc_bf16_to_f32(s[i]);
}

/* ------------------------------------------------------------------ exp
 * exp(x) = 2^n * e^r, n = rint(x*log2(e)), r = x - n*ln2 (two-step Cody-Waite),
 * e^r by a degree-7 minimax polynomial in Horner form.  Only fmaf, rintf and one
 * multiply are used, each correctly rounded in IEEE-754, so the same formula gives
 * the same bits on a CPU and on a GPU. Arguments below -80 give 0 (no denormals). */
float orc_expf(float x) {
  if (!(x >= -80.0f)) return 0.0f;
  if (x > 80.0f) x = 80.0f;
  float n = rintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693145751953125f, x);
  r = fmaf(n, -1.42860682030941723e-6f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  float e = fmaf(p, r2, r);
  e = e + 1.0f;
  int32_t ni = (int32_t)n;
  uint32_t sb = (uint32_t)(ni + 127) << 23; /* 2^n, n in [-116, 116] */
  float s;
  memcpy(&s, &sb, 4);
  return e * s;
}

/* ------------------------------------------------------------------ W: quantize
 * mlx.core.quantize, mode "affine" (docs cited at ops/quantization.rs:31-47):
 * every `group` consecutive elements of a row share (scale, bias);
 * w_hat = scale*q + bias; the `bits`-wide codes are packed into uint32 words, element
 * i of a row in word i/(32/bits) at bit (i mod (32/bits))*bits (low bits first).
 * Shapes pinned by ops/quantization.rs:306-309.  Quantiser restated from the
 * published MLX algorithm: scale from the group's range, the edge of larger magnitude
 * made exactly representable. */
int orc_quantize_f32(const float *w, int64_t rows, int64_t cols, int bits, int group,
                     uint32_t *q, float *scales, float *biases) {
  if (!(bits == 2 || bits == 4 || bits == 8)) return fail("quantize: bits must be 2, 4 or 8");
  if (!(group == 32 || group == 64 || group == 128)) return fail("quantize: group_size must be 32, 64 or 128");
  if (cols % group != 0) return fail("quantize: columns must be divisible by group_size");
  const int per_word = 32 / bits;
  const float n_bins = (float)((1 << bits) - 1);
  const int64_t gpr = cols / group, wpr = cols / per_word;
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t g = 0; g < gpr; ++g) {
      const float *wg = w + r * cols + g * group;
      float w_min = INFINITY, w_max = -INFINITY;
      for (int i = 0; i < group; ++i) {
        w_min = fminf(w_min, wg[i]);
        w_max = fmaxf(w_max, wg[i]);
      }
      int mask = fabsf(w_min) > fabsf(w_max);
      float scale = fmaxf((w_max - w_min) / n_bins, 1e-7f);
      scale = mask ? scale : -scale;
      float edge = mask ? w_min : w_max;
      float q0 = rintf(edge / scale);
      float bias = 0.0f;
      if (q0 != 0.0f) {
        scale = edge / q0;
        bias = edge;
      }
      scales[r * gpr + g] = scale;
      biases[r * gpr + g] = bias;
      uint32_t *qw = q + r * wpr + g * (group / per_word);
      for (int i = 0; i < group; i += per_word) {
        uint32_t word = 0;
        for (int j = 0; j < per_word; ++j) {
          float c = rintf((wg[i + j] - bias) / scale);
          c = fminf(fmaxf(c, 0.0f), n_bins);
          word |= (uint32_t)c << (j * bits);
        }
        qw[i / per_word] = word;
      }
    }
  }
  return 0;
}

int orc_quantize(const float *w, int64_t rows, int64_t cols, int bits, int group,
                 uint32_t *q, uint16_t *scales, uint16_t *biases) {
  if (group <= 0 || cols % group != 0) return fail("quantize: columns must be divisible by group_size");
  int64_t ng = rows * (cols / group);
  float *s = (float *)malloc(sizeof(float) * (size_t)ng * 2);
  if (!s) return fail("quantize: out of memory");
  int rc = orc_quantize_f32(w, rows, cols, bits, group, q, s, s + ng);
  if (rc == 0) {
    orc_f32_to_bf16_n(s, scales, ng);
    orc_f32_to_bf16_n(s + ng, biases, ng);
  }
  free(s);
  return rc;
}

static inline uint32_t code_at(const uint32_t *row, int64_t c, int bits) {
  const int per_word = 32 / bits;
  return (row[c / per_word] >> ((c % per_word) * bits)) & ((1u << bits) - 1u);
}

int orc_dequantize_f32(const uint32_t *q, const float *scales, const float *biases,
                       int64_t rows, int64_t cols, int bits, int group, float *out) {
  if (!(bits == 2 || bits == 4 || bits == 8)) return fail("dequantize: bits must be 2, 4 or 8");
  if (group <= 0 || cols % group != 0) return fail("dequantize: columns must be divisible by group_size");
  const int64_t gpr = cols / group, wpr = cols * bits / 32;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      float s = scales[r * gpr + c / group], b = biases[r * gpr + c / group];
      out[r * cols + c] = s * (float)code_at(q + r * wpr, c, bits) + b;
    }
  return 0;
}

int orc_dequantize(const uint32_t *q, const uint16_t *scales, const uint16_t *biases,
                   int64_t rows, int64_t cols, int bits, int group, float *out) {
  if (!(bits == 2 || bits == 4 || bits == 8)) return fail("dequantize: bits must be 2, 4 or 8");
  if (group <= 0 || cols % group != 0) return fail("dequantize: columns must be divisible by group_size");
  const int64_t gpr = cols / group, wpr = cols * bits / 32;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      float s = orc_bf16_to_f32(scales[r * gpr + c / group]);
      float b = orc_bf16_to_f32(biases[r * gpr + c / group]);
      out[r * cols + c] = s * (float)code_at(q + r * wpr, c, bits) + b;
    }
  return 0;
}

/* one dequantised row in fp32: w_hat[c] = float(scale)*q + float(bias) */
static void dequant_row(const uint32_t *qrow, const uint16_t *srow, const uint16_t *brow,
                        int K, int bits, int group, float *out) {
  const uint32_t maskv = (1u << bits) - 1u;
  const int per_word = 32 / bits;
  for (int g = 0; g < K / group; ++g) {
    float s = orc_bf16_to_f32(srow[g]), b = orc_bf16_to_f32(brow[g]);
    const uint32_t *qw = qrow + (int64_t)g * group / per_word;
    float *o = out + (int64_t)g * group;
    for (int wi = 0; wi < group / per_word; ++wi) {
      uint32_t word = qw[wi];
      for (int j = 0; j < per_word; ++j) {
        o[wi * per_word + j] = s * (float)(word & maskv) + b;
        word >>= bits;
      }
    }
  }
}

/* fp32 dot product in 8 interleaved partial sums (element c goes to sum c mod 8),
 * combined in a fixed tree: the accumulation MLX's CPU quantized matmul does with a
 * float SIMD accumulator, width fixed here so the result does not depend on the host. */
static inline float dot8(const float *a, const float *b, int K) {
  float l[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int c = 0;
  for (; c + 8 <= K; c += 8)
    for (int j = 0; j < 8; ++j) l[j] += a[c + j] * b[c + j];
  for (int j = 0; c < K; ++c, ++j) l[j] += a[c] * b[c];
  return ((l[0] + l[4]) + (l[2] + l[6])) + ((l[1] + l[5]) + (l[3] + l[7]));
}

/* ------------------------------------------------------------------ R1 logits
 * bias-free Linear: y = x . W^T (nn/linear.rs:84-96 -> ops::matmul).  The dot product
 * is accumulated in fp64 (every bf16*bf16 product is exact in fp32, and an fp64 sum of
 * 2^12 of them is within 2^-40 of the exact value), then rounded once to fp32 and
 * once to bf16.  The result is therefore the same for every summation order up to
 * events of probability ~2^-34 per logit: a GPU kernel that sums in another order
 * still selects the same experts.  MLX's own fp32 summation order is not known here;
 * orc_router_logits_f32seq measures how far an fp32 order moves the bf16 logits. */
void orc_router_logits(const uint16_t *x, const uint16_t *wg, const float *bias,
                       int64_t T, int H, int E, uint16_t *g) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t)
    for (int e = 0; e < E; ++e) {
      double acc = 0.0;
      const uint16_t *xr = x + t * H, *wr = wg + (int64_t)e * H;
      /* the product of two bf16 values is exact in double over the whole range (in float it would
       * underflow below 2^-149: two factors of 1e-25 each) */
      for (int h = 0; h < H; ++h) acc += (double)orc_bf16_to_f32(xr[h]) * (double)orc_bf16_to_f32(wr[h]);
      if (bias) acc += (double)bias[e];
      g[t * E + e] = orc_f32_to_bf16((float)acc);
    }
}

void orc_router_logits_f32seq(const uint16_t *x, const uint16_t *wg, const float *bias,
                              int64_t T, int H, int E, uint16_t *g) {
  for (int64_t t = 0; t < T; ++t)
    for (int e = 0; e < E; ++e) {
      float acc = 0.0f;
      const uint16_t *xr = x + t * H, *wr = wg + (int64_t)e * H;
      for (int h = 0; h < H; ++h) acc += orc_bf16_to_f32(xr[h]) * orc_bf16_to_f32(wr[h]);
      if (bias) acc += bias[e];
      g[t * E + e] = orc_f32_to_bf16(acc);
    }
}

/* ------------------------------------------------------------------ R2 softmax
 * softmax(precise = true): computed in fp32, result cast to the input dtype
 * (ops/arithmetic.rs:1291-1327).  Terms by orc_expf; their sum in fp64 (exact up to
 * 2^-46 whatever the order), rounded to fp32; one fp32 division per element. */
void orc_softmax(const uint16_t *g, int64_t T, int E, uint16_t *p) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t) {
    const uint16_t *gr = g + t * E;
    float m = -INFINITY;
    for (int e = 0; e < E; ++e) m = fmaxf(m, orc_bf16_to_f32(gr[e]));
    double sum = 0.0;
    for (int e = 0; e < E; ++e) sum += (double)orc_expf(orc_bf16_to_f32(gr[e]) - m);
    float sf = (float)sum;
    for (int e = 0; e < E; ++e)
      p[t * E + e] = orc_f32_to_bf16(orc_expf(orc_bf16_to_f32(gr[e]) - m) / sf);
  }
}

/* ------------------------------------------------------------------ R3 top-k
 * argpartition(...)[..., -k:] returns the k largest in unspecified order
 * (ops/sort.rs:186-260).  Here: the first k of the total order (value descending,
 * expert id ascending), slot 0 = best.  Values are compared as floats (so -0 == +0);
 * NaN-free input is a precondition. */
void orc_topk(const uint16_t *v, int64_t T, int E, int k, uint32_t *inds) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t) {
    const uint16_t *row = v + t * E;
    uint32_t *out = inds + t * k;
    for (int s = 0; s < k; ++s) {
      int best = -1;
      float bv = 0.0f;
      for (int e = 0; e < E; ++e) {
        int taken = 0;
        for (int j = 0; j < s; ++j) taken |= (out[j] == (uint32_t)e);
        if (taken) continue;
        float f = orc_bf16_to_f32(row[e]);
        if (best < 0 || f > bv) { /* strict >: a later equal value never displaces */
          best = e;
          bv = f;
        }
      }
      out[s] = (uint32_t)best;
    }
  }
}

/* ------------------------------------------------------------------ R4 scores
 * Qwen3-MoE: scores = take_along_axis(p, inds); with norm_topk_prob
 * scores /= scores.sum(-1, keepdims=True) (sum and divide are separate bf16 ops:
 * the sum is rounded to bf16 before the division).  Mixtral: softmax(precise) over
 * the k selected logits. */
void orc_scores(const uint16_t *g, const uint16_t *p, const uint32_t *inds, int64_t T,
                int E, int k, int score_mode, uint16_t *scores) {
  for (int64_t t = 0; t < T; ++t) {
    const uint32_t *id = inds + t * k;
    uint16_t *sc = scores + t * k;
    if (score_mode == ORC_SCORE_TOPK_SOFTMAX) {
      float m = -INFINITY;
      for (int s = 0; s < k; ++s) m = fmaxf(m, orc_bf16_to_f32(g[t * E + id[s]]));
      double sum = 0.0;
      for (int s = 0; s < k; ++s) sum += (double)orc_expf(orc_bf16_to_f32(g[t * E + id[s]]) - m);
      float sf = (float)sum;
      for (int s = 0; s < k; ++s)
        sc[s] = orc_f32_to_bf16(orc_expf(orc_bf16_to_f32(g[t * E + id[s]]) - m) / sf);
    } else {
      for (int s = 0; s < k; ++s) sc[s] = p[t * E + id[s]];
      if (score_mode == ORC_SCORE_SOFTMAX_TOPK_RENORM) {
        float sum = 0.0f; /* <= 2^15 bf16 terms of like sign: exact in fp32 for k <= 256 */
        for (int s = 0; s < k; ++s) sum += orc_bf16_to_f32(sc[s]);
        float denom = orc_bf16_to_f32(orc_f32_to_bf16(sum));
        for (int s = 0; s < k; ++s) sc[s] = orc_f32_to_bf16(orc_bf16_to_f32(sc[s]) / denom);
      }
    }
  }
}

void orc_route(const orc_config *cfg, const uint16_t *router_w, const float *router_bias,
               const uint16_t *x, int64_t T, uint32_t *inds, uint16_t *scores) {
  const int E = cfg->n_experts, k = cfg->top_k, H = cfg->hidden;
  uint16_t *g = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)T * E * 2);
  uint16_t *p = g + (size_t)T * E;
  orc_router_logits(x, router_w, router_bias, T, H, E, g);
  if (cfg->score_mode == ORC_SCORE_TOPK_SOFTMAX) {
    orc_topk(g, T, E, k, inds);
  } else {
    orc_softmax(g, T, E, p);
    orc_topk(p, T, E, k, inds);
  }
  orc_scores(g, p, inds, T, E, k, cfg->score_mode, scores);
  free(g);
}

/* ------------------------------------------------------------------ R5 dispatch
 * mlx-lm sorts the flattened (token, slot) pairs by expert with argsort (stable),
 * inverts the order with a second argsort, and takes token = order / k
 * (ops/sort.rs:75-109, ops/arithmetic.rs:1006-1014).  A stable counting sort gives
 * the same permutation. */
int orc_dispatch(const uint32_t *flat, int64_t P, int E, uint32_t *counts,
                 uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm) {
  for (int e = 0; e < E; ++e) counts[e] = 0;
  for (int64_t j = 0; j < P; ++j) {
    if (flat[j] >= (uint32_t)E) return fail("dispatch: expert index out of range");
    counts[flat[j]]++;
  }
  offsets[0] = 0;
  for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
  uint32_t *cur = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)E);
  if (!cur) return fail("dispatch: out of memory");
  memcpy(cur, offsets, sizeof(uint32_t) * (size_t)E);
  for (int64_t j = 0; j < P; ++j) {
    uint32_t r = cur[flat[j]]++;
    perm[r] = (uint32_t)j;
    if (inv_perm) inv_perm[j] = r;
  }
  free(cur);
  return 0;
}

/* ------------------------------------------------------------------ R6 gather_qmm
 * ops/quantization.rs:160-230 with transpose = true: for every index j,
 * out[j] (M x N) = x[lhs[j]] (M x K) . W_hat[rhs[j]]^T, W_hat = dequantize(w).
 * fp32 accumulation (dot8).  This is by definition what the reference's own test
 * checks: gather_qmm == gather_mm(x, dequantize(w)^T) (ops/quantization.rs:345-423). */
int orc_gather_qmm(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                   const uint16_t *biases, const uint32_t *lhs, const uint32_t *rhs,
                   int64_t n_idx, int64_t x_batch, int M, int N, int K, int E, int bits,
                   int group, float *y_f32, uint16_t *y_bf16, int n_threads) {
  if (!(bits == 4 || bits == 8 || bits == 2)) return fail("gather_qmm: bits must be 2, 4 or 8");
  if (group <= 0 || K % group != 0) return fail("gather_qmm: K must be divisible by group_size");
  for (int64_t j = 0; j < n_idx; ++j) {
    if (rhs[j] >= (uint32_t)E) return fail("gather_qmm: rhs index out of range");
    if ((lhs ? (int64_t)lhs[j] : j) >= x_batch) return fail("gather_qmm: lhs index out of range");
  }
  const int64_t wpr = (int64_t)K * bits / 32, gpr = K / group;
  (void)n_threads;
#pragma omp parallel num_threads(n_threads > 0 ? n_threads : 1)
  {
    float *wrow = (float *)malloc(sizeof(float) * (size_t)K);
    float *xf = (float *)malloc(sizeof(float) * (size_t)M * K);
#pragma omp for schedule(dynamic, 1)
    for (int64_t j = 0; j < n_idx; ++j) {
      const int64_t xb = lhs ? lhs[j] : j;
      const int64_t e = rhs[j];
      orc_bf16_to_f32_n(x + xb * M * K, xf, (int64_t)M * K);
      for (int n = 0; n < N; ++n) {
        dequant_row(w + (e * N + n) * wpr, scales + (e * N + n) * gpr, biases + (e * N + n) * gpr,
                    K, bits, group, wrow);
        for (int m = 0; m < M; ++m) {
          float acc = dot8(xf + (int64_t)m * K, wrow, K);
          int64_t o = (j * M + m) * N + n;
          if (y_f32) y_f32[o] = acc;
          if (y_bf16) y_bf16[o] = orc_f32_to_bf16(acc);
        }
      }
    }
    free(wrow);
    free(xf);
  }
  return 0;
}

/* transpose = false (the default of ops::quantized_matmul, ops/quantization.rs:91-122; the layout of
 * the reference's test_quantized_matmul, :318-342): w holds a K x N matrix quantised along N,
 * w: [E, K, N*bits/32], scales/biases: [E, K, N/group]; out[j] (M x N) = x[lhs[j]] (M x K) . W_hat[rhs[j]].
 * fp32 accumulation in k order. */
int orc_gather_qmm_nt(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                      const uint16_t *biases, const uint32_t *lhs, const uint32_t *rhs,
                      int64_t n_idx, int64_t x_batch, int M, int N, int K, int E, int bits,
                      int group, float *y_f32, uint16_t *y_bf16) {
  if (!(bits == 4 || bits == 8 || bits == 2)) return fail("gather_qmm: bits must be 2, 4 or 8");
  if (group <= 0 || N % group != 0) return fail("gather_qmm: N must be divisible by group_size");
  for (int64_t j = 0; j < n_idx; ++j) {
    if (rhs[j] >= (uint32_t)E) return fail("gather_qmm: rhs index out of range");
    if ((lhs ? (int64_t)lhs[j] : j) >= x_batch) return fail("gather_qmm: lhs index out of range");
  }
  const int64_t wpr = (int64_t)N * bits / 32, gpr = N / group;
  float *wrow = (float *)malloc(sizeof(float) * (size_t)N);
  float *acc = (float *)malloc(sizeof(float) * (size_t)M * N);
  if (!wrow || !acc) return fail("gather_qmm: out of memory");
  for (int64_t j = 0; j < n_idx; ++j) {
    const int64_t xb = lhs ? lhs[j] : j, e = rhs[j];
    for (int64_t i = 0; i < (int64_t)M * N; ++i) acc[i] = 0.0f;
    for (int k = 0; k < K; ++k) {
      dequant_row(w + (e * K + k) * wpr, scales + (e * K + k) * gpr, biases + (e * K + k) * gpr, N,
                  bits, group, wrow);
      for (int m = 0; m < M; ++m) {
        const float xv = orc_bf16_to_f32(x[(xb * M + m) * K + k]);
        for (int n = 0; n < N; ++n) acc[(int64_t)m * N + n] += xv * wrow[n];
      }
    }
    for (int64_t i = 0; i < (int64_t)M * N; ++i) {
      if (y_f32) y_f32[j * M * N + i] = acc[i];
      if (y_bf16) y_bf16[j * M * N + i] = orc_f32_to_bf16(acc[i]);
    }
  }
  free(wrow);
  free(acc);
  return 0;
}

/* ------------------------------------------------------------------ R7 SwiGLU
 * nn::silu = compile(x * sigmoid(x)) (nn/activation.rs:142-144,876-880), then
 * multiply by `up`.  Op by op on bf16 arrays every result is a bf16 value. */
static inline float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

void orc_swiglu_bf16(const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out) {
  for (int64_t i = 0; i < n; ++i) {
    float g = orc_bf16_to_f32(gate[i]), u = orc_bf16_to_f32(up[i]);
    float sg = orc_bf16_to_f32(orc_f32_to_bf16(sigmoidf_(g)));
    float t = orc_bf16_to_f32(orc_f32_to_bf16(g * sg));
    out[i] = orc_f32_to_bf16(t * u);
  }
}
void orc_swiglu_f32(const float *gate, const float *up, int64_t n, uint16_t *out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(gate[i] * sigmoidf_(gate[i]) * up[i]);
}

/* ------------------------------------------------------------------ R8 combine
 * (y * scores[..., None]).sum(-2): slots added in order s = 0..k-1 in fp32
 * (ops/arithmetic.rs:138-160, ops/reduction.rs:260-276). */
static void combine_impl(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                         int64_t T, int k, int H, int strict, const uint16_t *residual,
                         uint16_t *out) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t)
    for (int h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int s = 0; s < k; ++s) {
        int64_t r = inv_perm ? (int64_t)inv_perm[t * k + s] : t * k + s;
        float v = orc_bf16_to_f32(scores[t * k + s]) * orc_bf16_to_f32(y[r * H + h]);
        if (strict) v = orc_bf16_to_f32(orc_f32_to_bf16(v));
        acc += v;
      }
      if (residual) {  /* h + mlp(...): one more bf16 op in the op-by-op sequence */
        if (strict) acc = orc_bf16_to_f32(orc_f32_to_bf16(acc));
        acc = orc_bf16_to_f32(residual[t * H + h]) + acc;
      }
      out[t * H + h] = orc_f32_to_bf16(acc);
    }
}

void orc_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                 int64_t T, int k, int H, int strict, uint16_t *out) {
  combine_impl(y, scores, inv_perm, T, k, H, strict, NULL, out);
}

/* ------------------------------------------------------------------ M: the block
 * mlx-lm's sparse MoE block (SwitchGLU over gather_qmm): route, sort pairs by expert,
 * gate/up products, SwiGLU, down product, unsort, weighted sum over slots.  The block
 * sits where the dense Mlp sits in mlx-lm/src/models/qwen3.rs:204-255,321-324. */
static int moe_forward_impl(const orc_config *cfg, const orc_weights *w, const uint16_t *x,
                            int64_t T, uint16_t *out, const orc_debug_out *dbg, int strict,
                            int n_threads, const uint16_t *residual) {
  const int H = cfg->hidden, E = cfg->n_experts, k = cfg->top_k, I = cfg->intermediate;
  const int bits = cfg->bits, group = cfg->group_size;
  if (!(bits == 2 || bits == 4 || bits == 8)) return fail("forward: bits must be 2, 4 or 8");
  if (group != 64 && group != 32 && group != 128) return fail("forward: unsupported group_size");
  if (H % group || I % group) return fail("forward: hidden and intermediate must be divisible by group_size");
  if (k < 1 || k > E) return fail("forward: top_k must be in [1, n_experts]");
  if (T < 0) return fail("forward: negative token count");
  if (n_threads < 1) n_threads = 1;
#ifdef _OPENMP
  omp_set_num_threads(n_threads);
#endif
  const int64_t P = T * k;
  uint32_t *inds = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)(P * 3 + 2 * E + 2));
  uint32_t *perm = inds + P, *inv = perm + P, *counts = inv + P, *offsets = counts + E;
  uint16_t *scores = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(P + 1));
  uint16_t *hh = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(P * I + 1));
  uint16_t *y = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(P * H + 1));
  if (!inds || !scores || !hh || !y) return fail("forward: out of memory");

  orc_route(cfg, w->router_w, w->router_bias, x, T, inds, scores);
  int rc = orc_dispatch(inds, P, E, counts, offsets, perm, inv);
  if (rc) goto done;

  const int64_t wpr_gu = (int64_t)H * bits / 32, gpr_gu = H / group;
  const int64_t wpr_d = (int64_t)I * bits / 32, gpr_d = I / group;
#pragma omp parallel num_threads(n_threads)
  {
    float *rg = (float *)malloc(sizeof(float) * (size_t)(H > I ? H : I) * 2);
    float *ru = rg + (H > I ? H : I);
    float *xf = NULL;
    int64_t xf_cap = 0;
#pragma omp for schedule(dynamic, 1)
    for (int e = 0; e < E; ++e) {
      const int64_t r0 = offsets[e], cnt = counts[e];
      if (cnt == 0) continue;
      const int64_t need = cnt * (H > I ? H : I);
      if (need > xf_cap) {
        free(xf);
        xf = (float *)malloc(sizeof(float) * (size_t)need);
        xf_cap = need;
      }
      for (int64_t r = 0; r < cnt; ++r)
        orc_bf16_to_f32_n(x + (int64_t)(perm[r0 + r] / k) * H, xf + r * H, H);
      for (int n = 0; n < I; ++n) {
        const int64_t row = (int64_t)e * I + n;
        dequant_row(w->gate.w + row * wpr_gu, w->gate.scales + row * gpr_gu,
                    w->gate.biases + row * gpr_gu, H, bits, group, rg);
        dequant_row(w->up.w + row * wpr_gu, w->up.scales + row * gpr_gu,
                    w->up.biases + row * gpr_gu, H, bits, group, ru);
        for (int64_t r = 0; r < cnt; ++r) {
          float G = dot8(xf + r * H, rg, H), U = dot8(xf + r * H, ru, H);
          uint16_t *o = hh + (r0 + r) * I + n;
          if (strict) {
            uint16_t gb = orc_f32_to_bf16(G), ub = orc_f32_to_bf16(U);
            orc_swiglu_bf16(&gb, &ub, 1, o);
          } else {
            orc_swiglu_f32(&G, &U, 1, o);
          }
        }
      }
      for (int64_t r = 0; r < cnt; ++r) orc_bf16_to_f32_n(hh + (r0 + r) * I, xf + r * I, I);
      for (int n = 0; n < H; ++n) {
        const int64_t row = (int64_t)e * H + n;
        dequant_row(w->down.w + row * wpr_d, w->down.scales + row * gpr_d,
                    w->down.biases + row * gpr_d, I, bits, group, rg);
        for (int64_t r = 0; r < cnt; ++r)
          y[(r0 + r) * H + n] = orc_f32_to_bf16(dot8(xf + r * I, rg, I));
      }
    }
    free(rg);
    free(xf);
  }
  combine_impl(y, scores, inv, T, k, H, strict, residual, out);

  if (dbg) {
    if (dbg->topk_idx) memcpy(dbg->topk_idx, inds, sizeof(uint32_t) * (size_t)P);
    if (dbg->topk_w) memcpy(dbg->topk_w, scores, sizeof(uint16_t) * (size_t)P);
    if (dbg->counts) memcpy(dbg->counts, counts, sizeof(uint32_t) * (size_t)E);
    if (dbg->offsets) memcpy(dbg->offsets, offsets, sizeof(uint32_t) * (size_t)(E + 1));
    if (dbg->perm) memcpy(dbg->perm, perm, sizeof(uint32_t) * (size_t)P);
    if (dbg->inv_perm) memcpy(dbg->inv_perm, inv, sizeof(uint32_t) * (size_t)P);
  }
done:
  free(inds);
  free(scores);
  free(hh);
  free(y);
  return rc;
}

int orc_moe_forward(const orc_config *cfg, const orc_weights *w, const uint16_t *x,
                    int64_t T, uint16_t *out, const orc_debug_out *dbg, int strict,
                    int n_threads) {
  return moe_forward_impl(cfg, w, x, T, out, dbg, strict, n_threads, NULL);
}

/* RMS normalisation over the last axis: y = weight * x * rsqrt(mean(x^2) + eps)
 * (mlx-rs/src/nn/normalization.rs:233-275 -> fast::rms_norm, mlx-rs/src/fast.rs:190-207).
 * The mean of squares is accumulated in double (exact products, so the value does not depend on
 * the summation order), rounded to float; 1/sqrt in correctly rounded float operations; one
 * rounding to bf16 at the end. */
void orc_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T, int H,
                  uint16_t *out) {
  for (int64_t t = 0; t < T; ++t) {
    const uint16_t *xr = x + t * H;
    double ss = 0.0;
    for (int h = 0; h < H; ++h) {
      const double v = (double)orc_bf16_to_f32(xr[h]);
      ss += v * v;
    }
    const float mean = (float)(ss / (double)H);
    const float rstd = 1.0f / sqrtf(mean + eps);
    for (int h = 0; h < H; ++h) {
      const float xn = orc_bf16_to_f32(xr[h]) * rstd;
      out[t * H + h] = orc_f32_to_bf16(orc_bf16_to_f32(weight[h]) * xn);
    }
  }
}

/* The block between its neighbours in a decoder layer (mlx-lm/src/models/qwen3.rs:310-325):
 * out = x + moe(rms_norm(x, norm_weight, eps)).  strict: the block's result is rounded to bf16
 * before the add (two arrays in MLX); otherwise the add happens in the combine's accumulator. */
int orc_moe_forward_residual(const orc_config *cfg, const orc_weights *w, const uint16_t *x,
                             const uint16_t *norm_weight, float eps, int64_t T, uint16_t *out,
                             const orc_debug_out *dbg, int strict, int n_threads) {
  const int H = cfg->hidden;
  uint16_t *xn = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(T * H + 1));
  if (!xn) return fail("forward_residual: out of memory");
  orc_rms_norm(x, norm_weight, eps, T, H, xn);
  int rc = moe_forward_impl(cfg, w, xn, T, out, dbg, strict, n_threads, x);
  free(xn);
  return rc;
}

