/*
 * moe_oracle.h -- CPU restatement of the quantized mixture-of-experts block that
 * mlx-rs / mlx-lm compose from MLX primitives.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are compared
 * with, and the host-CPU baseline a benchmark times beside the GPU.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * The reference (oxiglade/mlx-rs) only *binds* these operations; the arithmetic
 * lives in ml-explore/mlx-c -> ml-explore/mlx, an un-vendored git submodule
 * (.gitmodules:1-3, directory empty; mlx-sys/Cargo.toml:3 says version 0.2.0
 * "should follow that of mlx-c", the workspace is 0.25.3, the exact commit is not
 * recoverable).  Each function below therefore restates the *published contract*
 * of the op and cites the reference binding, docs and tests it follows.
 *
 * Pinning status (what independent check each function has, tests/test_oracle_*.py):
 *   orc_quantize / orc_dequantize  pinned: reference KAT ops/quantization.rs:298-315
 *                                  (arange 128x512, group 128, bits 2/4/8: shapes +
 *                                  max error bound), nearest-code property by brute force
 *                                  over all codes, exact zero in groups that straddle
 *                                  zero, special groups (zero, constant, negative-
 *                                  dominant), packing order against a bit-by-bit numpy
 *                                  unpack.
 *                                  The exact bits of mlx.quantize on arbitrary input
 *                                  (eps clamp, rint mode, cast timing) are
 *                                  "parity unpinned": MLX is not importable here.  They
 *                                  do not enter kernel parity: packed weights are inputs.
 *   orc_router_logits              pinned: fp64 numpy/torch matmul, exact-rational
 *                                  brute force on tiny inputs.
 *   orc_softmax                    pinned: torch.softmax(float32).bfloat16(), row sums,
 *                                  reference test nn/activation.rs:1156-1185 (rows sum
 *                                  to one), monotonicity.
 *   orc_topk                       pinned: brute-force full sort, tie fixtures.
 *                                  MLX leaves tie choice and in-partition order
 *                                  undefined (ops/sort.rs:114,188,231); the order
 *                                  (value desc, expert id asc) is this build's.
 *   orc_scores                     pinned: closed forms in numpy/torch.
 *   orc_dispatch                   pinned: numpy.argsort(kind="stable"), bincount.
 *   orc_gather_qmm                 pinned: identity of ops/quantization.rs:345-423
 *                                  (== gather_mm on dequantised weights), fp64 numpy,
 *                                  E=1 -> torch matmul, unit-scale integer case (exact).
 *   orc_gather_qmm_nt              pinned: the identity of ops/quantization.rs:318-342
 *                                  (== x @ dequantize(w)) in fp64 numpy, and agreement with
 *                                  orc_gather_qmm on the transposed, re-quantised-free case K = N
 *                                  groups aligned (unit scales).
 *   orc_swiglu                     pinned: closed form, sigmoid KATs
 *                                  ops/arithmetic.rs:2577-2600.
 *   orc_combine                    pinned: closed form, slot-permutation invariance.
 *   orc_rms_norm                   pinned: closed form in float64 numpy, torch (float32 compute), the
 *                                  statistic of the reference test fast.rs:304-324 (uniform(0,1)
 *                                  input, unit weight: mean 0.8729 +- 0.0175).  Where MLX rounds
 *                                  inside its kernel (once at the end here) is "parity unpinned".
 *   orc_moe_forward_residual       pinned: composition of orc_rms_norm, orc_moe_forward and an add.
 *   orc_moe_forward                pinned: composition of the above vs an independent
 *                                  fp64 numpy restatement of the whole block.  No test
 *                                  in the reference exercises an MoE composition
 *                                  (mlx-lm/src/models/mod.rs:1-2 has only dense models),
 *                                  so block-level parity with MLX itself is unpinned.
 */
#ifndef MOE_ORACLE_H
#define MOE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* score modes (what the router does with the selected experts) */
enum {
  ORC_SCORE_SOFTMAX_TOPK_RENORM = 0, /* Qwen3-MoE, norm_topk_prob = true  */
  ORC_SCORE_SOFTMAX_TOPK = 1,        /* Qwen3-MoE, norm_topk_prob = false */
  ORC_SCORE_TOPK_SOFTMAX = 2         /* Mixtral: softmax over the k selected logits */
};

typedef struct {
  int32_t hidden, n_experts, top_k, intermediate, bits, group_size, score_mode;
} orc_config;

typedef struct {
  const uint32_t *w;      /* [E, N, K*bits/32] */
  const uint16_t *scales; /* bf16 [E, N, K/group] */
  const uint16_t *biases; /* bf16 [E, N, K/group] */
} orc_qmat;

typedef struct {
  const uint16_t *router_w;  /* bf16 [E, H] */
  const float *router_bias;  /* f32 [E] or NULL */
  orc_qmat gate, up, down;   /* gate/up: N=I,K=H ; down: N=H,K=I */
} orc_weights;

typedef struct {
  uint32_t *topk_idx; /* [T,k] */
  uint16_t *topk_w;   /* bf16 [T,k] */
  uint32_t *counts;   /* [E] */
  uint32_t *offsets;  /* [E+1] */
  uint32_t *perm;     /* [P] */
  uint32_t *inv_perm; /* [P] */
} orc_debug_out;

/* bfloat16 <-> float32, round to nearest even */
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);
void orc_f32_to_bf16_n(const float *src, uint16_t *dst, int64_t n);
void orc_bf16_to_f32_n(const uint16_t *src, float *dst, int64_t n);

/* exp() used by every softmax here: built from fmaf/rintf only, so that a GPU
 * restatement of the same formula gives the same bits. */
float orc_expf(float x);

/* W: MLX-affine quantisation (mlx-rs/src/ops/quantization.rs:31-83,124-158). */
int orc_quantize_f32(const float *w, int64_t rows, int64_t cols, int bits, int group,
                     uint32_t *q, float *scales, float *biases);
int orc_quantize(const float *w, int64_t rows, int64_t cols, int bits, int group,
                 uint32_t *q, uint16_t *scales, uint16_t *biases);
int orc_dequantize_f32(const uint32_t *q, const float *scales, const float *biases,
                       int64_t rows, int64_t cols, int bits, int group, float *out);
int orc_dequantize(const uint32_t *q, const uint16_t *scales, const uint16_t *biases,
                   int64_t rows, int64_t cols, int bits, int group, float *out);

/* R1 router logits: g = bf16(x . Wg^T (+ bias)), nn/linear.rs:84-96. */
void orc_router_logits(const uint16_t *x, const uint16_t *wg, const float *bias,
                       int64_t T, int H, int E, uint16_t *g);
/* same dot products accumulated in fp32 in index order (how far the bf16 logits move
 * under another summation order; used only to document that distance) */
void orc_router_logits_f32seq(const uint16_t *x, const uint16_t *wg, const float *bias,
                              int64_t T, int H, int E, uint16_t *g);
/* R2 softmax(precise=true) over the last axis, ops/arithmetic.rs:1291-1327. */
void orc_softmax(const uint16_t *g, int64_t T, int E, uint16_t *p);
/* R3 indices of the k largest, (value desc, id asc), ops/sort.rs:211-260. */
void orc_topk(const uint16_t *v, int64_t T, int E, int k, uint32_t *inds);
/* R4 scores of the selected experts, ops/indexing/mod.rs:433-453 + renorm. */
void orc_scores(const uint16_t *g, const uint16_t *p, const uint32_t *inds, int64_t T,
                int E, int k, int score_mode, uint16_t *scores);
/* R1-R4 together */
void orc_route(const orc_config *cfg, const uint16_t *router_w, const float *router_bias,
               const uint16_t *x, int64_t T, uint32_t *inds, uint16_t *scores);
/* R5 dispatch: stable sort of the pairs by expert, ops/sort.rs:75-109. */
int orc_dispatch(const uint32_t *flat, int64_t P, int E, uint32_t *counts,
                 uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm);
/* R6 gather_qmm, ops/quantization.rs:160-230.  x: bf16 [x_batch, M, K];
 * w: [E, N, K*bits/32]; out row-block j = x[lhs[j]] . W_hat[rhs[j]]^T, lhs == NULL
 * means lhs[j] = j.  y_f32 (fp32 accumulators) and y_bf16 may each be NULL. */
int orc_gather_qmm(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                   const uint16_t *biases, const uint32_t *lhs, const uint32_t *rhs,
                   int64_t n_idx, int64_t x_batch, int M, int N, int K, int E, int bits,
                   int group, float *y_f32, uint16_t *y_bf16, int n_threads);
/* the same with transpose = false: w [E, K, N*bits/32] holds K x N matrices quantised along N */
int orc_gather_qmm_nt(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                      const uint16_t *biases, const uint32_t *lhs, const uint32_t *rhs,
                      int64_t n_idx, int64_t x_batch, int M, int N, int K, int E, int bits,
                      int group, float *y_f32, uint16_t *y_bf16);
/* R7 silu(gate) * up.  strict != 0: bf16 round after every MLX op
 * (nn/activation.rs:142-144,876-880), else one round at the end. */
void orc_swiglu_bf16(const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out);
void orc_swiglu_f32(const float *gate, const float *up, int64_t n, uint16_t *out);
/* R8 combine: out[t] = sum_s score[t,s] * y[row(t,s)], row = inv_perm[t*k+s] or
 * t*k+s when inv_perm == NULL.  ops/reduction.rs:260-276. */
void orc_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                 int64_t T, int k, int H, int strict, uint16_t *out);

/* M: the whole block.  strict = 1 rounds to bf16 wherever MLX would materialise a
 * bf16 array between ops; strict = 0 rounds where fused kernels write memory. */
int orc_moe_forward(const orc_config *cfg, const orc_weights *w, const uint16_t *x,
                    int64_t T, uint16_t *out, const orc_debug_out *dbg, int strict,
                    int n_threads);

/* next to the path: RMS normalisation (mlx-rs/src/nn/normalization.rs:233-275, fast.rs:190-207) and
 * the block between its neighbours in a decoder layer, out = x + moe(rms_norm(x))
 * (mlx-lm/src/models/qwen3.rs:310-325). */
void orc_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T, int H,
                  uint16_t *out);
int orc_moe_forward_residual(const orc_config *cfg, const orc_weights *w, const uint16_t *x,
                             const uint16_t *norm_weight, float eps, int64_t T, uint16_t *out,
                             const orc_debug_out *dbg, int strict, int n_threads);

const char *orc_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
