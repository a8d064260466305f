// Dispatch: stable sort of the (token, slot) pairs by expert id.
//
// Replaces mlx-lm's gather-sort (argsort of the flattened expert indices, argsort of
// that order, floor_divide by k; mlx-rs/src/ops/sort.rs:75-109,
// ops/arithmetic.rs:1006-1014, ops/indexing/mod.rs:386-401) with a stable counting
// sort: per-expert histogram in LDS (ds_add_u32), scans, and a scatter whose ranks are
// computed from wave ballots in pair order, so the permutation is the one a stable
// argsort gives, whatever order blocks and waves run in.  Also emits the list of
// experts that received at least one pair (what the grouped products iterate over).
#include "dispatch_dev.hpp"

namespace mi_moe {

// ---- one block does everything (decode-sized P)
__global__ __launch_bounds__(kDispThreads) void dispatch_single_kernel(
    const uint32_t *flat, int64_t P, int E, int nbits, int k_div,
    uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets, uint32_t *__restrict__ perm,
    uint32_t *__restrict__ inv_perm, uint32_t *__restrict__ src_of,
    uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles, int cap256, uint32_t big_thr) {
  extern __shared__ uint32_t lds[];
  dispatch_block(flat, P, E, nbits, k_div, lds, counts, offsets, perm, inv_perm, src_of, work, mtiles, cap256, big_thr);
}

// ---- three kernels for prefill-sized P: block b owns pairs [b*span, (b+1)*span)
__global__ __launch_bounds__(kDispThreads) void dispatch_hist_kernel(
    const uint32_t *__restrict__ flat, int64_t P, int E, int64_t span,
    uint32_t *__restrict__ blockhist) {
  extern __shared__ uint32_t lds[];
  const int tid = threadIdx.x;
  for (int i = tid; i < E; i += kDispThreads) lds[i] = 0u;
  __syncthreads();
  const int64_t j0 = (int64_t)blockIdx.x * span;
  const int64_t j1 = j0 + span < P ? j0 + span : P;
  for (int64_t j = j0 + tid; j < j1; j += kDispThreads) {
    const uint32_t e = flat[j];
    atomicAdd(&lds[e < (uint32_t)E ? e : (uint32_t)E - 1u], 1u);
  }
  __syncthreads();
  for (int i = tid; i < E; i += kDispThreads) blockhist[(int64_t)blockIdx.x * E + i] = lds[i];
}

// Scatter of block b's pairs, and what used to be a kernel of its own between the histograms and the
// scatter: every block sums the per-block histograms itself (nb x E words, a few loads per thread: the
// blocks are dealt in G = 1024 / E' contiguous ranges, E' = E rounded up to a power of two, to G threads
// per expert), which gives it the counts, their exclusive scan and the number of pairs of each expert in
// the blocks before it, i.e. its own first sorted position per expert.  One more block (blockIdx.x == nb)
// takes no pairs and writes counts, offsets, work records and M tiles instead.
__global__ __launch_bounds__(kDispThreads) void dispatch_scatter_kernel(
    const uint32_t *flat, int64_t P, int E, int nbits, int k_div, int64_t span,
    const uint32_t *__restrict__ blockhist, int nb, uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets,
    uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles, int cap256, uint32_t big_thr,
    uint32_t *__restrict__ perm, uint32_t *__restrict__ inv_perm, uint32_t *__restrict__ src_of) {
  extern __shared__ uint32_t lds[];
  __shared__ uint32_t n_active, total;
  uint32_t *cnt = lds, *tmp = lds + E, *cur = lds + 2 * E, *wcnt = lds + 3 * E;  // tmp: at least kDispWaves words
  const int tid = threadIdx.x;
  const int mine = (int)blockIdx.x;
  int ep = 1;
  while (ep < E) ep <<= 1;
  const int G = kDispThreads / ep;  // E <= 512: at least 2
  const int e = tid % ep, g = tid / ep;
  const int per = (nb + G - 1) / G;
  const int b0 = g * per, b1 = b0 + per < nb ? b0 + per : nb;
  uint32_t *part_all = wcnt, *part_before = wcnt + G * E;  // [G][E] each; the space is wcnt's afterwards
  if (e < E) {
    uint32_t all = 0, before = 0;
    for (int b = b0; b < b1; ++b) {
      const uint32_t c = blockhist[(int64_t)b * E + e];
      all += c;
      before += b < mine ? c : 0u;
    }
    part_all[g * E + e] = all;
    part_before[g * E + e] = before;
  }
  __syncthreads();
  uint32_t before = 0;
  if (tid < E) {
    uint32_t all = 0;
    for (int i = 0; i < G; ++i) {
      all += part_all[i * E + tid];
      before += part_before[i * E + tid];
    }
    cnt[tid] = all;
  }
  __syncthreads();
  if (mine == nb) {
    finish_counts(cnt, tmp, cur, E, counts, offsets, work, mtiles, cap256, big_thr, &n_active);
    return;
  }
  block_exclusive_scan(cnt, tmp, E, &total);
  if (tid < E) cur[tid] = cnt[tid] + before;
  __syncthreads();
  const int64_t j0 = (int64_t)mine * span;
  const int64_t j1 = j0 + span < P ? j0 + span : P;
  scatter_range(flat, j0, j1, E, nbits, k_div, cur, wcnt, perm, inv_perm, src_of);
}

#ifndef MI_DISPATCH_SPAN
#define MI_DISPATCH_SPAN 1024
#endif
constexpr int64_t kSpan = MI_DISPATCH_SPAN;  // pairs per block in the multi-block path

size_t dispatch_workspace_bytes(int E, int64_t P) {
  if (P <= kSingleMaxP) return 256;
  int64_t nb = (P + kSpan - 1) / kSpan;
  return (size_t)nb * E * sizeof(uint32_t) + 256;
}

hipError_t launch_dispatch(const uint32_t *flat, int64_t P, int E, int k_div, uint32_t *counts,
                           uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                           uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int cap256, int big_thr,
                           void *scratch, hipStream_t st) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  if (k_div < 1) k_div = 1;
  if (P <= kSingleMaxP) {
    size_t lds = (size_t)(3 + kDispWaves) * E * sizeof(uint32_t);
    dispatch_single_kernel<<<1, kDispThreads, lds, st>>>(flat, P, E, nbits, k_div, counts, offsets,
                                                        perm, inv_perm, src_of, work, mtiles, cap256, (uint32_t)big_thr);
    return hipGetLastError();
  }
  uint32_t *blockhist = reinterpret_cast<uint32_t *>(scratch);
  const int nb = (int)((P + kSpan - 1) / kSpan);
  dispatch_hist_kernel<<<nb, kDispThreads, (size_t)E * 4, st>>>(flat, P, E, kSpan, blockhist);
  // LDS: cnt, tmp, cur [E] each (tmp also holds kDispWaves words), then the larger of wcnt[16 E] and the two
  // partial-sum arrays [G][E] (G E <= 1024)
  const size_t e3 = (size_t)3 * (E > kDispWaves ? E : kDispWaves);
  const size_t tail = (size_t)kDispWaves * E > 2u * kDispThreads ? (size_t)kDispWaves * E : 2u * kDispThreads;
  dispatch_scatter_kernel<<<nb + 1, kDispThreads, (e3 + tail) * 4, st>>>(flat, P, E, nbits, k_div, kSpan, blockhist, nb, counts,
                                                                        offsets, work, mtiles, cap256, (uint32_t)big_thr, perm,
                                                                        inv_perm, src_of);
  return hipGetLastError();
}

// One dense segment (a plain quantized matmul: every row goes to matrix 0): the work record or, from
// big_thr rows on, its M tiles.
__global__ void dense_records_kernel(uint32_t M, uint32_t big_thr, uint32_t *__restrict__ work,
                                     uint32_t *__restrict__ mtiles, int cap256) {
  const uint32_t tid = threadIdx.x;
  const bool big = big_thr != 0u && M >= big_thr;
  if (tid < kWorkWords) work[tid] = (tid == 2 && !big) ? M : 0u;  // {expert 0, row 0, M rows, no inline rows}
  const TileSplit ts = split_segment(big ? M : 0u);
  uint32_t *const l128 = tile_list(mtiles, 1, cap256, 1), *const l64 = tile_list(mtiles, 2, cap256, 1);
  if (tid == 0) {
    mtiles[0] = ts.n256;
    l128[0] = big && ts.r != 0u && ts.rcls == 1;
    l64[0] = big && ts.r != 0u && ts.rcls == 2;
    if (big && ts.r != 0u && ts.rcls != 0) {
      uint32_t *rec = (ts.rcls == 1 ? l128 : l64) + 4;
      rec[0] = 0u;
      rec[1] = M - ts.r;
      rec[2] = ts.r;
      rec[3] = 0u;
    }
  }
  for (uint32_t i = tid; i < ts.n256; i += blockDim.x) {
    uint32_t *rec = mtiles + 4 + (size_t)i * 4;
    rec[0] = 0u;
    rec[1] = i * kBigTileM;
    rec[2] = M - i * kBigTileM < (uint32_t)kBigTileM ? M - i * kBigTileM : (uint32_t)kBigTileM;
    rec[3] = 0u;
  }
}

hipError_t launch_dense_records(int64_t M, int big_thr, uint32_t *work, uint32_t *mtiles, int cap256,
                                hipStream_t st) {
  dense_records_kernel<<<1, 256, 0, st>>>((uint32_t)M, (uint32_t)big_thr, work, mtiles, cap256);
  return hipGetLastError();
}

// Row maps for the stand-alone gather_qmm: sorted position q of index j = perm[q]
// covers M rows; x rows come from lhs[j]*M + m, outputs go to j*M + m.
__global__ void row_maps_kernel(const uint32_t *__restrict__ perm, const uint32_t *__restrict__ lhs, uint32_t n_lhs,
                                const uint32_t *__restrict__ offsets, int64_t n_idx, int M, int E,
                                uint32_t *__restrict__ src_rows, uint32_t *__restrict__ dst_rows,
                                uint32_t *__restrict__ work) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < E) {  // records count rows, not indices; their inline source rows are not used
    work[i * kWorkWords + 1] *= (uint32_t)M;
    work[i * kWorkWords + 2] *= (uint32_t)M;
    work[i * kWorkWords + 3] = 0u;
  }
  if (i >= n_idx * M) return;
  const int64_t q = i / M;
  const int m = (int)(i % M);
  const uint32_t j = perm[q];
  uint32_t xb = lhs ? lhs[j] : j;
  if (n_lhs && xb >= n_lhs) xb = n_lhs - 1u;  // an index past x's batch is clamped, never followed
  src_rows[i] = xb * (uint32_t)M + m;
  dst_rows[i] = j * (uint32_t)M + m;
}

hipError_t launch_row_maps(const uint32_t *perm, const uint32_t *lhs, uint32_t n_lhs, const uint32_t *offsets,
                           int64_t n_idx, int M, int E, uint32_t *src_rows, uint32_t *dst_rows,
                           uint32_t *work, hipStream_t st) {
  int64_t n = n_idx * M > E ? n_idx * M : E;
  row_maps_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(perm, lhs, n_lhs, offsets, n_idx, M, E,
                                                              src_rows, dst_rows, work);
  return hipGetLastError();
}

}  // namespace mi_moe
