// Decode-sized batches: router logits, selection and dispatch in ONE launch.
//
// The three stages are separated by grid-wide dependencies (a token's selection needs all of
// its logits, the dispatch needs every token's selection).  Instead of ending the kernel at
// each of them, the workgroup that arrives last does the next stage:
//   - a workgroup computes 16 logits of one token (one per wave), publishes them, and counts
//     itself in for that token; the one that completes the count selects for the token;
//   - it then counts the token in; the workgroup that completes that count runs the dispatch.
// Nobody waits: a workgroup that is not last simply exits, so the scheme cannot deadlock.
// Data that crosses workgroups inside the launch (logits, selected experts, counters) is written
// with device-coherent stores and read with device-coherent loads; a workgroup waits for its own
// stores to be acknowledged before it counts itself in.  No cache-wide write-back or invalidate
// is involved (on this chip those cost microseconds per workgroup).
//
// Why this is safe on gfx950 although it is below what the HIP memory model promises:
//  * an `sc1` store is written through the issuing XCD's L2 to memory, and its acknowledgement
//    (what `s_waitcnt vmcnt(0)` waits for) comes back only when the data is there; an `sc1`
//    load is served from memory, not from a line another XCD's L2 may hold stale.  So a value whose
//    store was acknowledged is what any later `sc1` load on any XCD returns;
//  * the counters are device-scope atomics, executed at the memory side: every workgroup sees one
//    order of them;
//  * therefore: wave stores (sc1) -> every wave waits vmcnt(0) -> barrier -> one thread's atomic
//    increment.  The workgroup that observes the full count runs after every contributor's
//    increment, hence after every contributor's acknowledged stores, and reads them with sc1 loads
//    issued after its own barrier (no earlier load of those addresses exists in the workgroup, so
//    nothing stale sits in its registers, and sc1 loads do not hit in the per-CU cache).
// The wait is written out (`wait_own_stores`): a workgroup-scope release fence does not make the
// compiler emit it when the workgroup runs on one CU.
// The counters return to zero before the kernel ends, so the next launch finds them ready.
// Results are those of the separate kernels bit for bit (same device functions, and none of
// them depends on which workgroup runs it).
#include "dispatch_dev.hpp"
#include "router_dev.hpp"

namespace mi_moe {

// every vector-memory operation of this wave, stores included, has been acknowledged
__device__ __forceinline__ void wait_own_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// counters[0]: tokens selected; counters[1 + t]: logit workgroups of token t that have finished
template <int NV>
__global__ __launch_bounds__(kDispThreads) void router_fused_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ wg, const float *__restrict__ bias,
    const uint16_t *__restrict__ norm_w, float eps, uint16_t *__restrict__ xnorm,
    int T, int H, int E, int k, int mode, uint16_t *logits, uint32_t *topk_idx, uint16_t *topk_w,
    uint32_t *counters, int nbits, uint32_t *counts, uint32_t *offsets, uint32_t *perm,
    uint32_t *inv_perm, uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int cap256, uint32_t big_thr) {
  extern __shared__ uint32_t lds[];
  __shared__ uint32_t last;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int t = blockIdx.x;
  const int e = blockIdx.y * kDispWaves + wave;

  if (e < E) {
    // with a norm weight the token row is normalised first; every wave derives the same
    // normalised values, one of them (first workgroup of the token, first wave) keeps the row
    double s = norm_w ? logit_wave_norm(x + (int64_t)t * H, wg + (int64_t)e * H, norm_w, eps, H,
                                        blockIdx.y == 0 && wave == 0 ? xnorm + (int64_t)t * H : nullptr)
                      : logit_wave(x + (int64_t)t * H, wg + (int64_t)e * H, H);
    if (lane_id() == 0) {
      if (bias) s += (double)bias[e];
      store_agent(logits + (int64_t)t * E + e, f32_to_bf16((float)s));
    }
  }
  // every wave's stores (the logit, the normalised row) have been acknowledged ...
  wait_own_stores();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) {  // ... before the workgroup is counted in
    const uint32_t old = __hip_atomic_fetch_add(counters + 1 + t, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = old == gridDim.y - 1;
    if (last) store_agent(counters + 1 + t, 0u);
  }
  __syncthreads();
  if (!last) return;

  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (wave == 0)
    select_wave<NV, true>(logits + (int64_t)t * E, E, k, mode, topk_idx + (int64_t)t * k,
                          topk_w + (int64_t)t * k);
  wait_own_stores();  // the selected experts are where the dispatching workgroup will read them
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) {
    const uint32_t old = __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = old == gridDim.x - 1;
    if (last) store_agent(counters, 0u);
  }
  __syncthreads();
  if (!last) return;

  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  // at most 64 tokens, distinct experts per token: the mask form of the dispatch (the tiled lists
  // belong to batches far above this kernel's, the host passes none)
  if (mtiles == nullptr && T <= kMaskTokens)
    dispatch_tokens_block(topk_idx, T, k, E, lds, counts, offsets, perm, inv_perm, src_of, work);
  else
    dispatch_block(topk_idx, (int64_t)T * k, E, nbits, k, lds, counts, offsets, perm, inv_perm, src_of,
                   work, mtiles, cap256, big_thr);
}

// The same three stages with ONE exchange, for the smallest batches: every workgroup publishes its
// logits and counts itself in once; the workgroup that completes the count selects for every token
// (a wave per token, the logit rows of all of a wave's tokens fetched before the first selection, so
// that the round trip to memory is paid once) and dispatches from a copy of the selected experts in
// LDS.  Against the kernel above this saves one atomic round trip and the acknowledged store + reload
// of the selected experts, and spends the selections of all tokens on one CU.  Measured (Qwen3-30B
// shape, layer time): 2 and 4 tokens -0.8 us, 16 tokens no change, 32 tokens +4.4 us (two selections
// per wave in sequence): used up to kOneExchangeMaxTokens.  counters[0] is the only counter used.
constexpr int kOneExchangeRows = 1;        // tokens a wave selects for
constexpr int kOneExchangeMaxTokens = 8;
template <int NV>
__global__ __launch_bounds__(kDispThreads) void router_fused1_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ wg, const float *__restrict__ bias,
    const uint16_t *__restrict__ norm_w, float eps, uint16_t *__restrict__ xnorm,
    int T, int H, int E, int k, int mode, uint16_t *logits, uint32_t *topk_idx, uint16_t *topk_w,
    uint32_t *counters, uint32_t *counts, uint32_t *offsets, uint32_t *perm,
    uint32_t *inv_perm, uint32_t *src_of, uint32_t *work) {
  extern __shared__ uint32_t lds[];  // dispatch: 4 E words; selected experts: T k words behind them
  __shared__ uint32_t last;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int t0 = blockIdx.x;
  const int e = blockIdx.y * kDispWaves + wave;

  if (e < E) {
    double s = norm_w ? logit_wave_norm(x + (int64_t)t0 * H, wg + (int64_t)e * H, norm_w, eps, H,
                                        blockIdx.y == 0 && wave == 0 ? xnorm + (int64_t)t0 * H : nullptr)
                      : logit_wave(x + (int64_t)t0 * H, wg + (int64_t)e * H, H);
    if (lane_id() == 0) {
      if (bias) s += (double)bias[e];
      store_agent(logits + (int64_t)t0 * E + e, f32_to_bf16((float)s));
    }
  }
  wait_own_stores();  // every wave's logit has been acknowledged before the workgroup is counted in
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) {
    const uint32_t old = __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = old == gridDim.x * gridDim.y - 1;
    if (last) store_agent(counters, 0u);
  }
  __syncthreads();
  if (!last) return;

  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  uint32_t *const sel = lds + 4 * E;
  uint16_t bits[kOneExchangeRows][NV];
#pragma unroll
  for (int i = 0; i < kOneExchangeRows; ++i) {
    const int t = wave + i * kDispWaves;
    if (t < T) load_logit_row<NV, true>(logits + (int64_t)t * E, E, bits[i]);
  }
#pragma unroll
  for (int i = 0; i < kOneExchangeRows; ++i) {
    const int t = wave + i * kDispWaves;
    if (t < T)
      select_from_bits<NV, false>(bits[i], E, k, mode, topk_idx + (int64_t)t * k, topk_w + (int64_t)t * k,
                                  sel + t * k);
  }
  __syncthreads();
  dispatch_tokens_block<true>(sel, T, k, E, lds, counts, offsets, perm, inv_perm, src_of, work);
}

bool router_fused_applies(int64_t T, int E, int k) {
  return T >= 1 && T <= kFusedRouterMaxTokens && T * k <= kSingleMaxP;
}

hipError_t launch_router_fused(const uint16_t *x, const uint16_t *wg, const float *bias,
                               const uint16_t *norm_w, float eps, uint16_t *xnorm, int64_t T,
                               int H, int E, int k, int mode, uint16_t *logits, uint32_t *topk_idx,
                               uint16_t *topk_w, uint32_t *counters, uint32_t *counts,
                               uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                               uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int cap256,
                               int big_thr, hipStream_t st) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  dim3 grid((unsigned)T, (unsigned)((E + kDispWaves - 1) / kDispWaves));
  const size_t lds = (size_t)(3 + kDispWaves) * E * sizeof(uint32_t);
  static_assert(kOneExchangeMaxTokens <= kOneExchangeRows * kDispWaves && kOneExchangeMaxTokens <= kMaskTokens,
                "a wave selects for kOneExchangeRows tokens; the dispatch from LDS is the one of at most 64 tokens");
  if (T <= kOneExchangeMaxTokens && mtiles == nullptr) {
    const size_t lds1 = ((size_t)4 * E + (size_t)T * k) * sizeof(uint32_t);
#define MI_FUSED1(NV)                                                                             \
  router_fused1_kernel<NV><<<grid, kDispThreads, lds1, st>>>(                                      \
      x, wg, bias, norm_w, eps, xnorm, (int)T, H, E, k, mode, logits, topk_idx, topk_w, counters, counts, offsets,   \
      perm, inv_perm, src_of, work)
    if (E <= 64) MI_FUSED1(1);
    else if (E <= 128) MI_FUSED1(2);
    else if (E <= 256) MI_FUSED1(4);
    else MI_FUSED1(8);
#undef MI_FUSED1
    return hipGetLastError();
  }
#define MI_FUSED(NV)                                                                              \
  router_fused_kernel<NV><<<grid, kDispThreads, lds, st>>>(                                        \
      x, wg, bias, norm_w, eps, xnorm, (int)T, H, E, k, mode, logits, topk_idx, topk_w, counters, nbits, counts,      \
      offsets, perm, inv_perm, src_of, work, mtiles, cap256, (uint32_t)big_thr)
  if (E <= 64) MI_FUSED(1);
  else if (E <= 128) MI_FUSED(2);
  else if (E <= 256) MI_FUSED(4);
  else MI_FUSED(8);
#undef MI_FUSED
  return hipGetLastError();
}

}  // namespace mi_moe
