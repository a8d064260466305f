/*
 * mi_moe.h -- C ABI of the MI355X (gfx950) quantized mixture-of-experts block.
 *
 * One call, mi_moe_forward, replaces the ~25 mlx-sys dispatches an mlx-rs Module
 * makes for a sparse MoE layer (router Linear, softmax, argpartition, take_along_axis,
 * renormalise, argsort x2, take, gather_qmm x3, silu, multiply, unsort, multiply,
 * sum).  Stage-level entry points expose each primitive family on its own so that
 * each has an individually testable counterpart.
 *
 * Conventions follow what mlx-rs expects from mlx-sys:
 *  - every entry point returns int: 0 = success, non-zero = failure
 *    (mlx-rs/src/utils/mod.rs:13-14, mlx-rs/src/utils/guard.rs:20-49);
 *  - the message of the last failure is kept per thread and can also be delivered to
 *    a registered handler (mlx-rs/src/error.rs:226-280 installs such a handler through
 *    mlx_set_error_handler and stores the text in a thread-local slot);
 *  - no exception or unwinding crosses the boundary; on failure outputs are untouched;
 *  - arrays are row-major and contiguous (an mlx-rs Array after eval,
 *    mlx-rs/src/array/mod.rs:384-403); bfloat16 is passed as raw uint16_t, packed
 *    weights and indices as uint32_t, sizes as int64_t; every pointer is DEVICE memory
 *    unless the comment says host, and must be 16-byte aligned;
 *  - calls are asynchronous on the hipStream_t passed as `void* stream` (NULL = the
 *    default stream): the analogue of MLX's lazy evaluation, the caller synchronises
 *    where mlx-rs would call eval (mlx-rs/src/transforms/mod.rs:66-92);
 *  - the library keeps no input pointer after a call returns except the weight
 *    pointers registered with mi_moe_create; one handle is used by one host thread at
 *    a time (MLX itself is not thread safe, .github/workflows/validate.yml:46), and
 *    forwards through one handle must not overlap on the GPU (use one stream per handle):
 *    a handle owns 260 bytes of device memory (arrival counters of the decode router
 *    kernel), allocated by mi_moe_create on the current device and released by
 *    mi_moe_destroy.  Each GPU has ONE set of three streams and five events (default
 *    priority) for the whole process, created by the first mi_moe_create on that GPU and kept
 *    until the process ends, however many handles exist: a forward with an average of 6 rows
 *    per expert or more (17 with 8-bit weights) forks its independent kernel chains onto
 *    them from `stream` and joins them back before it returns, which is also what a graph
 *    capture of `stream` records (so two captures that are open at the same time on one GPU
 *    must not both hold such a forward: a stream belongs to one capture at a time).  The
 *    host-side fork-to-join sequence runs under a per-GPU lock.  No other entry point
 *    allocates device memory or creates streams.
 *
 * Weight format = MLX "affine" quantisation (mlx-rs/src/ops/quantization.rs:31-47,
 * 85-87, 306-309): element c of a row lives in uint32 word c/(32/bits) at bit
 * (c mod (32/bits))*bits; w_hat = scale*q + bias with one bf16 (scale, bias) per
 * group_size consecutive elements of the row.
 */
#ifndef MI_MOE_H
#define MI_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi_moe_s *mi_moe_handle;

typedef enum {
  MI_MOE_SCORE_SOFTMAX_THEN_TOPK_RENORM = 0, /* Qwen3-MoE, norm_topk_prob = true  */
  MI_MOE_SCORE_SOFTMAX_THEN_TOPK = 1,        /* Qwen3-MoE, norm_topk_prob = false */
  MI_MOE_SCORE_TOPK_THEN_SOFTMAX = 2         /* Mixtral: softmax over the selected logits */
} mi_moe_score_mode;

/* element type of activations, scales, biases and outputs of the *_typed entry points (MLX takes
 * any floating type there, mlx-rs/src/dtype.rs:206-256; the reference's own tests of these ops run in
 * float32, mlx-rs/src/ops/quantization.rs:318-423) */
typedef enum {
  MI_MOE_DTYPE_BF16 = 0,
  MI_MOE_DTYPE_F16 = 1,
  MI_MOE_DTYPE_F32 = 2
} mi_moe_dtype;

typedef struct {
  int32_t hidden;       /* H, multiple of group_size */
  int32_t n_experts;    /* E, 1..512 */
  int32_t top_k;        /* k, 1..min(E,32) */
  int32_t intermediate; /* I, multiple of group_size */
  int32_t bits;         /* 4 or 8 (tuned kernels); 2 runs on the plain products */
  int32_t group_size;   /* 64 (tuned kernels); 32 and 128 run on the plain products */
  int32_t score_mode;   /* mi_moe_score_mode */
} mi_moe_config;

/* one bank of E quantized matrices, the layout mlx-rs's QuantizedLinear holds per
 * matrix (mlx-rs/src/nn/quantized.rs:254-279: inner.weight, scales, biases) with a
 * leading expert axis */
typedef struct {
  const uint32_t *w;      /* [E, N, K*bits/32] */
  const uint16_t *scales; /* bf16 [E, N, K/group_size] */
  const uint16_t *biases; /* bf16 [E, N, K/group_size] */
} mi_moe_qmat;

typedef struct {
  const uint16_t *router_w; /* bf16 [E, H]: bias-free Linear, mlx-rs/src/nn/linear.rs:84-96 */
  const float *router_bias; /* f32 [E] added to the logits before the bf16 round, or NULL */
  mi_moe_qmat gate, up;     /* N = I, K = H */
  mi_moe_qmat down;         /* N = H, K = I */
} mi_moe_weights;

/* optional routing outputs of mi_moe_forward; any member may be NULL */
typedef struct {
  uint32_t *topk_idx; /* [T, k] expert ids, slot 0 = best, ties -> lower id */
  uint16_t *topk_w;   /* bf16 [T, k] scores */
  uint32_t *counts;   /* [E] pairs per expert */
  uint32_t *offsets;  /* [E+1] exclusive scan of counts */
  uint32_t *perm;     /* [P] pair index t*k+s of sorted position r (stable by expert) */
  uint32_t *inv_perm; /* [P] sorted position of pair t*k+s */
} mi_moe_debug_out;

/* ---- errors (replaces mlx_set_error_handler + the LAST_MLX_ERROR slot,
 * mlx-rs/src/error.rs:226-280) ---- */
const char *mi_moe_last_error(void); /* thread-local, never NULL */
void mi_moe_set_error_handler(void (*handler)(const char *msg, void *data), void *data,
                              void (*dtor)(void *data));

/* ---- the block (replaces the op sequence a Module<&Array>::forward would issue;
 * forward contract mlx-rs/src/module/module.rs:28-50, dense sibling
 * mlx-lm/src/models/qwen3.rs:204-255, call site :321-324) ---- */
int mi_moe_create(const mi_moe_config *cfg, const mi_moe_weights *weights, mi_moe_handle *out);
int mi_moe_destroy(mi_moe_handle h);
int mi_moe_workspace_size(const mi_moe_config *cfg, int64_t max_tokens, size_t *bytes);
/* x: bf16 [T, H] -> out: bf16 [T, H].  workspace: device memory of at least
 * mi_moe_workspace_size(cfg, T) bytes, 256-byte aligned, contents irrelevant. */
int mi_moe_forward(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out,
                   void *workspace, size_t workspace_bytes, const mi_moe_debug_out *dbg,
                   void *stream);

/* mi_moe_forward for callers that cannot allocate device memory or hand one over: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference (MLX allocates as it evaluates).  The workspace is an array of
 * MI_MOE_STATIC_SCRATCH_BYTES that is part of the library's code object (each GPU the library runs on
 * holds its own copy until the process ends); the call allocates nothing, creates nothing and gives
 * mi_moe_forward's results bit for bit.  It fails, with a message that says how much is missing, when
 * T tokens of the handle's layer need more workspace than that (mi_moe_workspace_size tells: the
 * Qwen3-30B-A3B-shaped layer fits up to 156 tokens, the Mixtral-8x7B-shaped one up to 102, the
 * Qwen3-235B-A22B-shaped one up to 84).  Every call on
 * one GPU uses the same array, whatever the handle: calls that overlap on a GPU race, so keep them
 * on one stream (or order them by events); nothing in the array has to survive between calls. */
#define MI_MOE_STATIC_SCRATCH_BYTES 8388608
int mi_moe_forward_static(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out,
                          const mi_moe_debug_out *dbg, void *stream);

/* The block between its neighbours in a decoder layer (mlx-lm/src/models/qwen3.rs:310-325:
 * r = post_attention_layernorm(h); r = mlp(r); out = h + r): out = x + moe(rms_norm(x, norm_weight,
 * eps)), with the residual add folded into the combine (one rounding) and the normalised rows
 * kept in the workspace.  norm_weight: bf16 [H].  out must not alias x.  Same workspace as
 * mi_moe_forward.  Replaces mlx_fast_rms_norm (mlx-rs/src/fast.rs:190-207) and mlx_add around
 * the block. */
int mi_moe_forward_residual(mi_moe_handle h, const uint16_t *x, const uint16_t *norm_weight,
                            float eps, int64_t T, uint16_t *out, void *workspace,
                            size_t workspace_bytes, const mi_moe_debug_out *dbg, void *stream);

/* RMS normalisation over the last axis on its own: out = weight * x * rsqrt(mean(x^2) + eps)
 * (mlx_fast_rms_norm, mlx-rs/src/fast.rs:190-207; nn::RmsNorm, nn/normalization.rs:233-275).
 * x, out: bf16 [T, hidden]; weight: bf16 [hidden]. */
int mi_moe_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T,
                    int32_t hidden, uint16_t *out, void *stream);

/* The same forward with a HIP event recorded on `stream` before the first launch and
 * after each stage; waits for the last one and returns the MI_MOE_N_STAGES elapsed times
 * in milliseconds (host array): router logits, router select, dispatch, gate/up + SwiGLU,
 * down, combine (an event pair adds several microseconds to what lies between).  kernel_ms (host
 * array of MI_MOE_N_KERNEL_TIMES, or NULL): the durations of the grouped-product kernels themselves,
 * each from the start and end time stamps of its own dispatch (what a profiler reports for the
 * kernel): gate/up + SwiGLU over the 256-row, 128-row and 64-row tile lists and over the streamed
 * segments, then the down product over the same four; 0 where no kernel was launched.  The kernels
 * run one after the other on `stream`.  For measurement; mlx-rs has no counterpart (it times with
 * Instant::now() around eval, mlx-rs/examples/linear_regression.rs:40-59). */
#define MI_MOE_N_STAGES 6
#define MI_MOE_N_KERNEL_TIMES 8
int mi_moe_forward_timed(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out,
                         void *workspace, size_t workspace_bytes, void *stream, float *stage_ms,
                         float *kernel_ms);

/* ---- R1-R4 router: gate Linear + softmax(precise) + argpartition top-k +
 * take_along_axis + renormalise (mlx_matmul, mlx_softmax_axis, mlx_argpartition_axis,
 * mlx_take_along_axis, mlx_sum_axis, mlx_divide; mlx-rs/src/ops/arithmetic.rs:577-603,
 * 1291-1327, ops/sort.rs:211-260, ops/indexing/mod.rs:433-453).
 * logits_out (bf16 [T,E]) may be NULL.  workspace >= mi_moe_route_workspace_size.  A workspace that is larger
 * by mi_moe_router_logits_workspace_size(T, hidden, n_experts) lets batches of more than 64 tokens take the
 * integer route for the logits (same bits; up to 128 experts with the selection in the same kernel). */
int mi_moe_route_workspace_size(int32_t n_experts, int64_t T, size_t *bytes);
int mi_moe_route(const uint16_t *x, const uint16_t *router_w, const float *router_bias,
                 int64_t T, int32_t hidden, int32_t n_experts, int32_t top_k,
                 int32_t score_mode, uint32_t *topk_idx, uint16_t *topk_w,
                 uint16_t *logits_out, void *workspace, size_t workspace_bytes, void *stream);

/* ---- R1 alone: logits = x . router_w^T (+ router_bias), bf16 [T, n_experts]: the gate Linear
 * (mlx_matmul through nn::Linear, mlx-rs/src/nn/linear.rs:84-96, ops/arithmetic.rs:577-603), the way
 * mi_moe_forward computes it: exact bf16 x bf16 products, summed without rounding, then fp64 -> fp32 ->
 * bf16.  Up to 64 tokens in fp64 arithmetic; beyond, in integer arithmetic on the int8 matrix cores with
 * the same bits (csrc/router_exact.hip), which needs workspace >= mi_moe_router_logits_workspace_size
 * (contents irrelevant).  mi_moe_route takes the fp64 route for any T unless its workspace has that much
 * room beyond its own need. ---- */
int mi_moe_router_logits_workspace_size(int64_t T, int32_t hidden, int32_t n_experts, size_t *bytes);
int mi_moe_router_logits(const uint16_t *x, const uint16_t *router_w, const float *router_bias,
                         int64_t T, int32_t hidden, int32_t n_experts, uint16_t *logits,
                         void *workspace, size_t workspace_bytes, void *stream);

/* ---- R5 dispatch: stable sort of the P = T*k pairs by expert (mlx_argsort x2,
 * mlx_floor_divide, mlx_take; mlx-rs/src/ops/sort.rs:75-109).  Every output except
 * perm may be NULL.  workspace >= mi_moe_dispatch_workspace_size. */
int mi_moe_dispatch_workspace_size(int32_t n_experts, int64_t P, size_t *bytes);
int mi_moe_dispatch(const uint32_t *expert_of_pair, int64_t P, int32_t n_experts,
                    uint32_t *counts, uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                    void *workspace, size_t workspace_bytes, void *stream);

/* ---- R6 gather_qmm (mlx_gather_qmm, mlx-rs/src/ops/quantization.rs:160-230):
 * for j < n_idx: y[j] (M x N) = x[lhs[j]] (M x K) . dequantize(w[rhs[j]])^T.
 * x: bf16 [x_batch, M, K]; w: [E, N, K*bits/32]; y: bf16 [n_idx, M, N].
 * lhs_indices NULL = identity (j), as an absent mlx_array; rhs_indices required.  Index arrays of
 * other shapes are broadcast against each other and flattened by the host layers (the op's batch
 * semantics, :160-176); the entry point takes the flat arrays.
 * The tuned path: transpose non-zero (the layout every mlx-lm switch layer uses), group_size 64,
 * bits 4 or 8, K a multiple of 64 (4-bit: 128), N a multiple of 16, at most 512 experts.  Everything
 * else -- transpose = 0 (w [E, K, N*bits/32], scales, biases [E, K, N/group_size], K x N matrices
 * quantised along N), group sizes 32 and 128, 2-bit codes -- is served by plain kernels that need no
 * workspace and no alignment.
 * sorted_indices is a hint, results do not depend on it.
 * Index values live in device memory and cannot be checked by the call: an lhs index beyond
 * x_batch - 1 or an rhs index beyond n_experts - 1 is clamped to the last matrix by the kernels (the
 * output rows it belongs to are then meaningless, but nothing outside the operands is read).
 * x_batch = 0 means "not told" (no clamp on lhs); without lhs_indices, n_idx may not exceed x_batch.
 * workspace >= mi_moe_gather_qmm_workspace_size. */
int mi_moe_gather_qmm_workspace_size(int32_t n_experts, int64_t n_idx, int32_t M, size_t *bytes);
int mi_moe_gather_qmm(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                      const uint16_t *biases, const uint32_t *lhs_indices,
                      const uint32_t *rhs_indices, int64_t n_idx, int64_t x_batch, int32_t M,
                      int32_t N, int32_t K, int32_t n_experts, int32_t transpose,
                      int32_t group_size, int32_t bits, int32_t sorted_indices, uint16_t *y,
                      void *workspace, size_t workspace_bytes, void *stream);
/* the same op with x, scales, biases and y of element type dtype (mi_moe_dtype); bf16 takes the
 * paths above, fp16 and fp32 the plain kernels (fp32 accumulation, one rounding to dtype):
 * test_gather_qmm of the reference (mlx-rs/src/ops/quantization.rs:345-423) runs through this. */
int mi_moe_gather_qmm_typed(const void *x, const uint32_t *w, const void *scales, const void *biases,
                            const uint32_t *lhs_indices, const uint32_t *rhs_indices, int64_t n_idx,
                            int64_t x_batch, int32_t M, int32_t N, int32_t K, int32_t n_experts,
                            int32_t transpose, int32_t group_size, int32_t bits,
                            int32_t sorted_indices, int32_t dtype, void *y, void *workspace,
                            size_t workspace_bytes, void *stream);

/* ---- dense quantized matmul (mlx_quantized_matmul, mlx-rs/src/ops/quantization.rs:91-122, as
 * QuantizedLinear::forward calls it with transpose = true, mlx-rs/src/nn/quantized.rs:363-386):
 * y (M x N) = x (M x K) . dequantize(w)^T on the same kernels as gather_qmm (one matrix, every row).
 * x: bf16 [M, K]; w: [N, K*bits/32]; scales, biases: bf16 [N, K/group_size]; y: bf16 [M, N].
 * transpose = 0 (the op's own default; test_quantized_matmul, ops/quantization.rs:318-342):
 * w [K, N*bits/32], scales, biases [K, N/group_size], y = x . dequantize(w), a plain kernel; so are
 * group sizes 32 / 128 and 2-bit codes.
 * workspace >= mi_moe_quantized_matmul_workspace_size (the plain kernels need none). */
int mi_moe_quantized_matmul_workspace_size(int64_t M, int32_t K, int32_t bits, size_t *bytes);
int mi_moe_quantized_matmul(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                            const uint16_t *biases, int64_t M, int32_t N, int32_t K,
                            int32_t transpose, int32_t group_size, int32_t bits, uint16_t *y,
                            void *workspace, size_t workspace_bytes, void *stream);
/* the same op with x, scales, biases and y of element type dtype (mi_moe_dtype):
 * test_quantized_matmul of the reference (fp32, transpose = false) runs through this. */
int mi_moe_quantized_matmul_typed(const void *x, const uint32_t *w, const void *scales,
                                  const void *biases, int64_t M, int32_t N, int32_t K,
                                  int32_t transpose, int32_t group_size, int32_t bits, int32_t dtype,
                                  void *y, void *workspace, size_t workspace_bytes, void *stream);

/* ---- a quantized linear layer with its optional bias (QuantizedLinear::forward,
 * mlx-rs/src/nn/quantized.rs:363-386: quantized_matmul(x, w, scales, biases, transpose = true), then
 * `+ bias` when the layer has one): y = x . dequantize(w)^T, rounded to dtype, then y + linear_bias,
 * rounded again, as the reference's two ops.  linear_bias: [N] of element type dtype, or NULL (then this
 * is mi_moe_quantized_matmul_typed with transpose = 1).  Same workspace. */
int mi_moe_quantized_linear_typed(const void *x, const uint32_t *w, const void *scales,
                                  const void *biases, const void *linear_bias, int64_t M, int32_t N,
                                  int32_t K, int32_t group_size, int32_t bits, int32_t dtype, void *y,
                                  void *workspace, size_t workspace_bytes, void *stream);

/* ---- R7 silu(gate) * up on bf16 arrays (mlx_sigmoid + mlx_multiply x2,
 * mlx-rs/src/nn/activation.rs:142-144,876-880).  The block itself fuses this into
 * the gate/up product; this entry point is the stand-alone op. ---- */
int mi_moe_swiglu(const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out,
                  void *stream);

/* ---- R8 combine: out[t] = sum_s scores[t,s] * y[row(t,s)] with
 * row = inv_perm[t*k+s], or t*k+s when inv_perm is NULL (mlx_take + mlx_multiply +
 * mlx_sum_axis; mlx-rs/src/ops/reduction.rs:260-276).  y: bf16 [P, H]. ---- */
int mi_moe_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                   int64_t T, int32_t top_k, int32_t hidden, uint16_t *out, void *stream);

/* ---- W: MLX-affine quantize / dequantize of a [rows, cols] fp32 matrix on the
 * device (mlx_quantize / mlx_dequantize, mlx-rs/src/ops/quantization.rs:50-83,
 * 124-158).  q: [rows, cols*bits/32]; scales, biases: bf16 [rows, cols/group_size]. */
int mi_moe_quantize(const float *w, int64_t rows, int64_t cols, int32_t group_size,
                    int32_t bits, uint32_t *q, uint16_t *scales, uint16_t *biases,
                    void *stream);
int mi_moe_dequantize(const uint32_t *q, const uint16_t *scales, const uint16_t *biases,
                      int64_t rows, int64_t cols, int32_t group_size, int32_t bits,
                      float *w_hat, void *stream);
/* the same two with scales and biases of element type dtype (mi_moe_dtype): mlx_quantize gives them
 * the type of its input, float32 in the reference's tests (ops/quantization.rs:298-342).  The codes
 * come from the fp32 scale and bias either way; the cast to dtype happens afterwards. */
int mi_moe_quantize_typed(const float *w, int64_t rows, int64_t cols, int32_t group_size,
                          int32_t bits, int32_t dtype, uint32_t *q, void *scales, void *biases,
                          void *stream);
int mi_moe_dequantize_typed(const uint32_t *q, const void *scales, const void *biases, int64_t rows,
                            int64_t cols, int32_t group_size, int32_t bits, int32_t dtype,
                            float *w_hat, void *stream);

/* mlx_dequantize as the reference returns it (mlx-rs/src/ops/quantization.rs:124-158): w_hat has the
 * element type of scales and biases (dtype), [rows, cols].  The value is the fp32 one of
 * mi_moe_dequantize_typed rounded once more to dtype. */
int mi_moe_dequantize_native(const uint32_t *q, const void *scales, const void *biases, int64_t rows,
                             int64_t cols, int32_t group_size, int32_t bits, int32_t dtype,
                             void *w_hat, void *stream);

/* ---- introspection; no counterpart in the reference.  The library holds one compiled variant of its
 * two grouped-product kernels per combination of bit width, SwiGLU fusion, K split, ring depth, slab
 * staging, token groups and tile height.  mi_moe_debug_kernel_count / _name / _launches list every variant
 * the library contains with the number of times this process has launched it (the name stays valid
 * until the library is unloaded): the test suite uses them to show that no variant is left
 * without a parity-checked launch.  mi_moe_debug_plan_forward / _grouped write, into the host buffer
 * `out` (cap bytes, NUL-terminated, entries separated by ';'), the variants with grid and LDS bytes that
 * a forward of T tokens / one grouped product of the given extents WOULD launch, and launch nothing:
 * they need no GPU and touch no device memory (the host-side launch rules, checked on any machine).
 * _grouped: total_rows rows in max_active segments of at most max_rows_per_expert rows;
 * max_streamed_rows (0 = unknown) bounds the segments that are not tiled; tile_lists non-zero = M-tile
 * lists exist (a batch that mi_moe_forward would tile).
 * mi_moe_debug_side_streams_created: streams the library has created in this process (three per GPU
 * on which a handle was ever created, whatever the number of handles). ---- */
int32_t mi_moe_debug_kernel_count(void);
const char *mi_moe_debug_kernel_name(int32_t index);  /* NULL beyond the last variant */
int64_t mi_moe_debug_kernel_launches(int32_t index);  /* -1 beyond the last variant */
int mi_moe_debug_plan_forward(const mi_moe_config *cfg, int64_t T, char *out, size_t cap);
int mi_moe_debug_plan_grouped(int32_t N, int32_t K, int32_t bits, int32_t glu, int64_t total_rows,
                              int32_t max_active, int64_t max_rows_per_expert,
                              int64_t max_streamed_rows, int32_t tile_lists, int32_t paired_out,
                              char *out, size_t cap);
/* which rows of a forward of T tokens go where: *tiled = M-tile lists are built; *tile_min_rows = a segment of
 * at least that many rows is cut into 256-row tiles, with its remainder in the 256-, 128- or 64-row list that
 * holds it; shorter segments stream */
int mi_moe_debug_tile_rule(const mi_moe_config *cfg, int64_t T, int32_t *tiled, int32_t *tile_min_rows);
int32_t mi_moe_debug_side_streams_created(void);

/* ---- measurement aid; no counterpart in the reference.  A bare streaming kernel with the decode
 * grouped product's access shape (a wave reads a 16 KiB tile from each half of buf, 64 bytes per row
 * and instruction, four pieces in flight, four blocks per CU) over the first `bytes` bytes of buf
 * (a multiple of 32768): what a launch of that size can pull from HBM.  bench.py reports it beside
 * the roofline of the gate/up kernel.  sink: one device word (never written in practice). ---- */
int mi_moe_stream_probe(const void *buf, size_t bytes, uint32_t *sink, void *stream);

/* library version string, e.g. "mi_moe 0.1 gfx950" */
const char *mi_moe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI_MOE_H */
