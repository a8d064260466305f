// Dispatch: stable sort of the (token, slot) pairs by expert id.
//
// Replaces mlx-lm's gather-sort (argsort of the flattened expert indices, argsort of
// that order, floor_divide by k; mlx-rs/src/ops/sort.rs:75-109,
// ops/arithmetic.rs:1006-1014, ops/indexing/mod.rs:386-401) with a stable counting
// sort: per-expert histogram in LDS (ds_add_u32), scans, and a scatter whose ranks are
// computed from wave ballots in pair order, so the permutation is the one a stable
// argsort gives, whatever order blocks and waves run in.  Also emits the list of
// experts that received at least one pair (what the grouped products iterate over).
#include "common.hpp"

namespace mi_moe {

constexpr int kDispThreads = 1024;             // 16 waves
constexpr int kDispWaves = kDispThreads / 64;  // pairs per chunk = 1024

__device__ __forceinline__ uint64_t lanemask_lt() {
  return (1ull << lane_id()) - 1ull;
}

// lanes (among `valid` ones) that hold the same expert id as this lane
__device__ __forceinline__ uint64_t match_peers(uint32_t e, int nbits, bool valid) {
  uint64_t peers = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1u;
    const uint64_t bm = __ballot(valid && bit);
    peers &= bit ? bm : ~bm;
  }
  return peers;
}

// exclusive scan of v[0..n) in LDS by one block of kDispThreads threads (n <= 1024);
// tmp: n words.  Returns with v holding the exclusive scan and *total the sum.
__device__ void block_exclusive_scan(uint32_t *v, uint32_t *tmp, int n, uint32_t *total) {
  const int tid = threadIdx.x;
  uint32_t mine = tid < n ? v[tid] : 0u;
  uint32_t *src = v, *dst = tmp;
  for (int off = 1; off < n; off <<= 1) {
    uint32_t val = 0;
    if (tid < n) val = src[tid] + (tid >= off ? src[tid - off] : 0u);
    __syncthreads();
    if (tid < n) dst[tid] = val;
    __syncthreads();
    uint32_t *t = src;
    src = dst;
    dst = t;
  }
  uint32_t incl = tid < n ? src[tid] : 0u;
  __syncthreads();
  if (tid < n) v[tid] = incl - mine;
  if (tid == n - 1) *total = incl;
  __syncthreads();
}

// Scatter the pairs [j0, j1) (j0 a multiple of 1024) given cur[e] = first free sorted
// position of expert e for this range.  LDS: cur[E], wcnt[16*E].
__device__ void scatter_range(const uint32_t *__restrict__ flat, int64_t j0, int64_t j1, int E,
                              int nbits, int k_div, uint32_t *cur, uint32_t *wcnt,
                              uint32_t *__restrict__ perm, uint32_t *__restrict__ inv_perm,
                              uint32_t *__restrict__ src_of) {
  const int tid = threadIdx.x, wave = tid >> 6;
  for (int64_t c0 = j0; c0 < j1; c0 += kDispThreads) {
    for (int i = tid; i < kDispWaves * E; i += kDispThreads) wcnt[i] = 0u;
    __syncthreads();
    const int64_t j = c0 + tid;
    const bool valid = j < j1;
    uint32_t e = valid ? flat[j] : 0u;
    e = e < (uint32_t)E ? e : (uint32_t)E - 1u;  // out-of-range ids are clamped, never written past LDS
    const uint64_t peers = match_peers(e, nbits, valid);
    const uint32_t rank = __popcll(peers & lanemask_lt());
    if (valid && rank == 0) wcnt[wave * E + e] = __popcll(peers);
    __syncthreads();
    for (int x = tid; x < E; x += kDispThreads) {
      uint32_t run = cur[x];
      for (int w = 0; w < kDispWaves; ++w) {
        uint32_t c = wcnt[w * E + x];
        wcnt[w * E + x] = run;
        run += c;
      }
      cur[x] = run;
    }
    __syncthreads();
    if (valid) {
      const uint32_t pos = wcnt[wave * E + e] + rank;
      perm[pos] = (uint32_t)j;
      if (inv_perm) inv_perm[j] = pos;
      if (src_of) src_of[pos] = (uint32_t)j / (uint32_t)k_div;
    }
    __syncthreads();
  }
}

// Work records consumed by the grouped products: one 64-byte record per expert that received
// rows, in ascending expert order, then records with count 0 up to n_experts.
//   [0] expert id  [1] first sorted row  [2] row count  [3] 1 if [4..15] are filled
//   [4..15] source row (pair index / k_div) of the first 12 rows of the segment
constexpr int kWorkWords = 16;
constexpr int kWorkSrc = 12;

// Long segments (at least big_thr rows, big_thr > 0) go to the tiled MFMA kernel instead: they
// are cut into M tiles of kBigTileM rows, listed in `mtiles`:
//   mtiles[0] = number of tiles; tile i at mtiles[4 + 4 i] = {expert id, first sorted row, rows, 0}


// counts -> offsets, work records and M tiles; runs in one block.  LDS cnt[E] in, cur[E] out.
__device__ void finish_counts(uint32_t *cnt, uint32_t *tmp, uint32_t *cur, int E,
                              uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets,
                              uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles,
                              uint32_t big_thr, uint32_t *n_active_lds) {
  __shared__ uint32_t total;
  const int tid = threadIdx.x;
  if (tid < E && counts) counts[tid] = cnt[tid];
  __syncthreads();
  block_exclusive_scan(cnt, tmp, E, &total);
  if (tid < E) {
    cur[tid] = cnt[tid];
    if (offsets) offsets[tid] = cnt[tid];
  }
  if (tid == 0 && offsets) offsets[E] = total;
  __syncthreads();
  // experts with rows, in ascending order, by wave 0
  if (tid < kWave) {
    uint32_t base = 0, tbase = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
      const int e = e0 + tid;
      uint32_t c = 0;
      if (e < E) c = (e + 1 < E ? cnt[e + 1] : total) - cnt[e];
      const bool big = mtiles && big_thr != 0u && c >= big_thr;
      const bool small = c != 0u && !big;
      const uint64_t bm = __ballot(small);
      if (small && work) {
        uint32_t *rec = work + (size_t)(base + __popcll(bm & lanemask_lt())) * kWorkWords;
        rec[0] = (uint32_t)e;
        rec[1] = cnt[e];
        rec[2] = c;
        rec[3] = 0u;
      }
      base += __popcll(bm);
      // M tiles of the long segments: exclusive scan of the tile counts over the wave
      const uint32_t nt = big ? (c + kBigTileM - 1) / kBigTileM : 0u;
      uint32_t incl = nt;
      for (int d = 1; d < kWave; d <<= 1) {
        const uint32_t v = __shfl_up(incl, d, kWave);
        if (tid >= d) incl += v;
      }
      for (uint32_t i = 0; i < nt; ++i) {
        uint32_t *rec = mtiles + 4 + (size_t)(tbase + incl - nt + i) * 4;
        rec[0] = (uint32_t)e;
        rec[1] = cnt[e] + i * kBigTileM;
        rec[2] = c - i * kBigTileM < (uint32_t)kBigTileM ? c - i * kBigTileM : (uint32_t)kBigTileM;
        rec[3] = 0u;
      }
      tbase += __shfl(incl, kWave - 1, kWave);
    }
    if (work)
      for (int sl = base + tid; sl < E; sl += kWave) {
        work[(size_t)sl * kWorkWords + 2] = 0u;
        work[(size_t)sl * kWorkWords + 3] = 0u;
      }
    if (tid == 0) {
      *n_active_lds = base;
      if (mtiles) mtiles[0] = tbase;
    }
  }
  __syncthreads();
}

// ---- one block does everything (decode-sized P)
__global__ __launch_bounds__(kDispThreads) void dispatch_single_kernel(
    const uint32_t *__restrict__ flat, int64_t P, int E, int nbits, int k_div,
    uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets, uint32_t *__restrict__ perm,
    uint32_t *__restrict__ inv_perm, uint32_t *__restrict__ src_of,
    uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles, uint32_t big_thr) {
  extern __shared__ uint32_t lds[];
  __shared__ uint32_t n_active;
  uint32_t *cnt = lds, *tmp = lds + E, *cur = lds + 2 * E, *wcnt = lds + 3 * E;
  const int tid = threadIdx.x;
  for (int i = tid; i < E; i += kDispThreads) cnt[i] = 0u;
  __syncthreads();
  for (int64_t j = tid; j < P; j += kDispThreads) {
    const uint32_t e = flat[j];
    atomicAdd(&cnt[e < (uint32_t)E ? e : (uint32_t)E - 1u], 1u);
  }
  __syncthreads();
  finish_counts(cnt, tmp, cur, E, counts, offsets, work, mtiles, big_thr, &n_active);
  scatter_range(flat, 0, P, E, nbits, k_div, cur, wcnt, perm, inv_perm, src_of);
  // source rows of the first rows of every segment, so that a consumer needs one load
  if (work) {
    __threadfence_block();
    __syncthreads();
    for (int i = tid; i < (int)n_active * kWorkSrc; i += kDispThreads) {
      uint32_t *rec = work + (size_t)(i / kWorkSrc) * kWorkWords;
      const uint32_t j = i % kWorkSrc;
      if (j < rec[2]) rec[4 + j] = perm[rec[1] + j] / (uint32_t)k_div;
      if (j == 0) rec[3] = 1u;
    }
  }
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

__global__ __launch_bounds__(kDispThreads) void dispatch_scan_kernel(
    uint32_t *__restrict__ blockhist, int nb, int E, uint32_t *__restrict__ counts,
    uint32_t *__restrict__ offsets, uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles,
    uint32_t big_thr) {
  extern __shared__ uint32_t lds[];
  __shared__ uint32_t n_active;
  uint32_t *cnt = lds, *tmp = lds + E, *cur = lds + 2 * E;
  const int tid = threadIdx.x;
  if (tid < E) {
    uint32_t run = 0;
    for (int b = 0; b < nb; ++b) run += blockhist[(int64_t)b * E + tid];
    cnt[tid] = run;
  }
  __syncthreads();
  finish_counts(cnt, tmp, cur, E, counts, offsets, work, mtiles, big_thr, &n_active);
  if (tid < E) {  // blockhist[b][e] <- first sorted position of expert e for block b
    uint32_t run = cur[tid];
    for (int b = 0; b < nb; ++b) {
      uint32_t c = blockhist[(int64_t)b * E + tid];
      blockhist[(int64_t)b * E + tid] = run;
      run += c;
    }
  }
}

__global__ __launch_bounds__(kDispThreads) void dispatch_scatter_kernel(
    const uint32_t *__restrict__ flat, int64_t P, int E, int nbits, int k_div, int64_t span,
    const uint32_t *__restrict__ blockbase, uint32_t *__restrict__ perm,
    uint32_t *__restrict__ inv_perm, uint32_t *__restrict__ src_of) {
  extern __shared__ uint32_t lds[];
  uint32_t *cur = lds, *wcnt = lds + E;
  const int tid = threadIdx.x;
  for (int i = tid; i < E; i += kDispThreads) cur[i] = blockbase[(int64_t)blockIdx.x * E + i];
  __syncthreads();
  const int64_t j0 = (int64_t)blockIdx.x * span;
  const int64_t j1 = j0 + span < P ? j0 + span : P;
  scatter_range(flat, j0, j1, E, nbits, k_div, cur, wcnt, perm, inv_perm, src_of);
}

constexpr int64_t kSingleMaxP = 4096;
constexpr int64_t kSpan = 2048;  // pairs per block in the multi-block path

size_t dispatch_workspace_bytes(int E, int64_t P) {
  if (P <= kSingleMaxP) return 256;
  int64_t nb = (P + kSpan - 1) / kSpan;
  return (size_t)nb * E * sizeof(uint32_t) + 256;
}

hipError_t launch_dispatch(const uint32_t *flat, int64_t P, int E, int k_div, uint32_t *counts,
                           uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                           uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int big_thr,
                           void *scratch, hipStream_t st) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  if (k_div < 1) k_div = 1;
  if (P <= kSingleMaxP) {
    size_t lds = (size_t)(3 + kDispWaves) * E * sizeof(uint32_t);
    dispatch_single_kernel<<<1, kDispThreads, lds, st>>>(flat, P, E, nbits, k_div, counts, offsets,
                                                        perm, inv_perm, src_of, work, mtiles, (uint32_t)big_thr);
    return hipGetLastError();
  }
  uint32_t *blockhist = reinterpret_cast<uint32_t *>(scratch);
  const int nb = (int)((P + kSpan - 1) / kSpan);
  dispatch_hist_kernel<<<nb, kDispThreads, (size_t)E * 4, st>>>(flat, P, E, kSpan, blockhist);
  dispatch_scan_kernel<<<1, kDispThreads, (size_t)3 * E * 4, st>>>(blockhist, nb, E, counts,
                                                                  offsets, work, mtiles, (uint32_t)big_thr);
  dispatch_scatter_kernel<<<nb, kDispThreads, (size_t)(1 + kDispWaves) * E * 4, st>>>(
      flat, P, E, nbits, k_div, kSpan, blockhist, perm, inv_perm, src_of);
  return hipGetLastError();
}

// Row maps for the stand-alone gather_qmm: sorted position q of index j = perm[q]
// covers M rows; x rows come from lhs[j]*M + m, outputs go to j*M + m.
__global__ void row_maps_kernel(const uint32_t *__restrict__ perm, const uint32_t *__restrict__ lhs,
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
  src_rows[i] = (lhs ? lhs[j] : j) * (uint32_t)M + m;
  dst_rows[i] = j * (uint32_t)M + m;
}

hipError_t launch_row_maps(const uint32_t *perm, const uint32_t *lhs, const uint32_t *offsets,
                           int64_t n_idx, int M, int E, uint32_t *src_rows, uint32_t *dst_rows,
                           uint32_t *work, hipStream_t st) {
  int64_t n = n_idx * M > E ? n_idx * M : E;
  row_maps_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(perm, lhs, offsets, n_idx, M, E,
                                                              src_rows, dst_rows, work);
  return hipGetLastError();
}

}  // namespace mi_moe
