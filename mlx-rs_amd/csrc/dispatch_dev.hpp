// Device-side building blocks of the dispatch (stable counting sort of the (token, slot) pairs by
// expert), shared by the stand-alone dispatch kernels and the fused decode router kernel.
#pragma once

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
// tmp: at least kDispWaves words.  Returns with v holding the exclusive scan and *total the sum.
// Each wave scans its 64 values with lane shuffles; the waves' totals meet in tmp.
__device__ __forceinline__ void block_exclusive_scan(uint32_t *v, uint32_t *tmp, int n, uint32_t *total) {
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const uint32_t mine = tid < n ? v[tid] : 0u;
  uint32_t incl = mine;
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t up = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += up;
  }
  if (lane == kWave - 1) tmp[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
  for (int w = 0; w < kDispWaves; ++w) {
    const uint32_t t = tmp[w];
    before += w < wave ? t : 0u;
    all += t;
  }
  if (tid < n) v[tid] = before + incl - mine;
  if (tid == 0) *total = all;
  __syncthreads();
}

// Scatter the pairs [j0, j1) (j0 a multiple of 1024) given cur[e] = first free sorted
// position of expert e for this range.  LDS: cur[E], wcnt[16*E].
__device__ __forceinline__ void scatter_range(const uint32_t *flat, int64_t j0, int64_t j1, int E,
                              int nbits, int k_div, uint32_t *cur, uint32_t *wcnt,
                              uint32_t *__restrict__ perm, uint32_t *__restrict__ inv_perm,
                              uint32_t *__restrict__ src_of) {
  const int tid = threadIdx.x, wave = tid >> 6;
  for (int64_t c0 = j0; c0 < j1; c0 += kDispThreads) {
    for (int i = tid; i < kDispWaves * E; i += kDispThreads) wcnt[i] = 0u;
    __syncthreads();
    const int64_t j = c0 + tid;
    const bool valid = j < j1;
    uint32_t e = valid ? load_agent(flat + j) : 0u;
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

// Segments of at least big_thr rows (big_thr > 0) go to the tiled MFMA kernel instead: they are cut
// into M tiles of 256 rows, and what is left over (or a whole shorter segment) goes to the smallest
// of the 256-, 128- and 64-row classes that holds it; one list per class (tile_list()).

// tile classes of a segment of c rows: full 256-row tiles, then one tile for the remainder r
struct TileSplit {
  uint32_t n256;  // tiles in the 256-row list (the last one may be the remainder, if r > 128)
  uint32_t r;     // rows of the remainder tile (0: none)
  int rcls;       // class of the remainder tile: 0, 1, 2
};
__device__ __forceinline__ TileSplit split_segment(uint32_t c) {
  TileSplit t;
  const uint32_t full = c / kBigTileM;
  t.r = c % kBigTileM;
  t.rcls = t.r > 128u ? 0 : (t.r > 64u ? 1 : 2);
  t.n256 = full + (t.r > 128u ? 1u : 0u);
  return t;
}

// counts -> offsets, work records and M tiles; runs in one block.  LDS cnt[E] in, cur[E] out.
__device__ __forceinline__ void finish_counts(uint32_t *cnt, uint32_t *tmp, uint32_t *cur, int E,
                              uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets,
                              uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles, int cap256,
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
    uint32_t *const l256 = mtiles, *const l128 = mtiles ? tile_list(mtiles, 1, cap256, E) : nullptr,
                   *const l64 = mtiles ? tile_list(mtiles, 2, cap256, E) : nullptr;
    uint32_t base = 0, t256 = 0, t128 = 0, t64 = 0;
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
      // M tiles: exclusive scan of the 256-row tile counts over the wave, ballots for the others
      TileSplit ts = split_segment(big ? c : 0u);
      uint32_t incl = ts.n256;
      for (int d = 1; d < kWave; d <<= 1) {
        const uint32_t v = __shfl_up(incl, d, kWave);
        if (tid >= d) incl += v;
      }
      const uint32_t first = big ? cnt[e] : 0u;
      for (uint32_t i = 0; i < ts.n256; ++i) {
        uint32_t *rec = l256 + 4 + (size_t)(t256 + incl - ts.n256 + i) * 4;
        const uint32_t left = c - i * kBigTileM;
        rec[0] = (uint32_t)e;
        rec[1] = first + i * kBigTileM;
        rec[2] = left < (uint32_t)kBigTileM ? left : (uint32_t)kBigTileM;
        rec[3] = 0u;
      }
      t256 += __shfl(incl, kWave - 1, kWave);
      const bool r128 = big && ts.r != 0u && ts.rcls == 1, r64 = big && ts.r != 0u && ts.rcls == 2;
      const uint64_t b128 = __ballot(r128), b64 = __ballot(r64);
      if (r128 || r64) {
        uint32_t *rec = r128 ? l128 + 4 + (size_t)(t128 + __popcll(b128 & lanemask_lt())) * 4
                             : l64 + 4 + (size_t)(t64 + __popcll(b64 & lanemask_lt())) * 4;
        rec[0] = (uint32_t)e;
        rec[1] = first + (c - ts.r);
        rec[2] = ts.r;
        rec[3] = 0u;
      }
      t128 += __popcll(b128);
      t64 += __popcll(b64);
    }
    if (work)
      for (int sl = base + tid; sl < E; sl += kWave) {
        work[(size_t)sl * kWorkWords + 2] = 0u;
        work[(size_t)sl * kWorkWords + 3] = 0u;
      }
    if (tid == 0) {
      *n_active_lds = base;
      if (mtiles) {
        l256[0] = t256;
        l128[0] = t128;
        l64[0] = t64;
      }
    }
  }
  __syncthreads();
}


// The whole dispatch of P <= kSingleMaxP pairs by one block of kDispThreads threads.
// LDS (dynamic, passed in): (3 + kDispWaves) * E words.
__device__ __forceinline__ void dispatch_block(const uint32_t *flat, int64_t P, int E, int nbits, int k_div,
                               uint32_t *lds, uint32_t *__restrict__ counts,
                               uint32_t *__restrict__ offsets, uint32_t *__restrict__ perm,
                               uint32_t *__restrict__ inv_perm, uint32_t *__restrict__ src_of,
                               uint32_t *__restrict__ work, uint32_t *__restrict__ mtiles, int cap256,
                               uint32_t big_thr) {
  __shared__ uint32_t n_active;
  uint32_t *cnt = lds, *tmp = lds + E, *cur = lds + 2 * E, *wcnt = lds + 3 * E;
  const int tid = threadIdx.x;
  for (int i = tid; i < E; i += kDispThreads) cnt[i] = 0u;
  __syncthreads();
  for (int64_t j = tid; j < P; j += kDispThreads) {
    const uint32_t e = load_agent(flat + j);
    atomicAdd(&cnt[e < (uint32_t)E ? e : (uint32_t)E - 1u], 1u);
  }
  __syncthreads();
  finish_counts(cnt, tmp, cur, E, counts, offsets, work, mtiles, cap256, big_thr, &n_active);
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

constexpr int64_t kSingleMaxP = 4096;

// The dispatch of at most 64 tokens whose k experts are distinct per token (what the selection
// produces), by one block.  The stable order by pair index is then the order by token, and a
// pair's place inside its expert's segment is the number of earlier tokens that chose the same
// expert: it is read off a 64-bit token mask per expert.  Three barriers instead of the two dozen
// of the general path; the same outputs bit for bit.
// LDS (dynamic, passed in): 4 * E words.  P = T * k <= kSingleMaxP.
constexpr int kMaskTokens = 64;
// FLAT_LOCAL: `flat` was written by this workgroup (LDS, or memory behind a barrier): plain loads.
template <bool FLAT_LOCAL = false>
__device__ __forceinline__ void dispatch_tokens_block(const uint32_t *flat, int T, int k, int E, uint32_t *lds,
                                      uint32_t *__restrict__ counts, uint32_t *__restrict__ offsets,
                                      uint32_t *__restrict__ perm, uint32_t *__restrict__ inv_perm,
                                      uint32_t *__restrict__ src_of, uint32_t *__restrict__ work) {
  uint32_t *const mlo = lds, *const mhi = lds + E, *const off = lds + 2 * E, *const ridx = lds + 3 * E;
  const int tid = threadIdx.x;
  const int P = T * k;
  constexpr int kPer = (int)(kSingleMaxP / kDispThreads);  // pairs per thread at most
  for (int i = tid; i < 2 * E; i += kDispThreads) lds[i] = 0u;
  __syncthreads();
  uint32_t es[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int j = tid + i * kDispThreads;
    es[i] = 0u;
    if (j < P) {
      uint32_t e = FLAT_LOCAL ? flat[j] : load_agent(flat + j);
      e = e < (uint32_t)E ? e : (uint32_t)E - 1u;  // out-of-range ids are clamped, never written past LDS
      es[i] = e;
      const uint32_t t = (uint32_t)j / (uint32_t)k;
      atomicOr(t < 32u ? &mlo[e] : &mhi[e], 1u << (t & 31u));
    }
  }
  __syncthreads();
  // wave 0: counts, their exclusive scan, one work record per expert with rows (ascending ids)
  if (tid < kWave) {
    uint32_t base = 0, n_active = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
      const int e = e0 + tid;
      const uint32_t c = e < E ? (uint32_t)(__popc(mlo[e]) + __popc(mhi[e])) : 0u;
      uint32_t incl = c;
      for (int d = 1; d < kWave; d <<= 1) {
        const uint32_t v = __shfl_up(incl, d, kWave);
        if (tid >= d) incl += v;
      }
      const uint32_t excl = base + incl - c;
      const uint64_t bm = __ballot(c != 0u);
      if (e < E) {
        off[e] = excl;
        if (counts) counts[e] = c;
        if (offsets) offsets[e] = excl;
        if (c != 0u) {
          const uint32_t r = n_active + __popcll(bm & lanemask_lt());
          ridx[e] = r;
          if (work) {
            uint32_t *rec = work + (size_t)r * kWorkWords;
            rec[0] = (uint32_t)e;
            rec[1] = excl;
            rec[2] = c;
            rec[3] = 1u;  // the source rows follow below
          }
        }
      }
      base += __shfl(incl, kWave - 1, kWave);
      n_active += __popcll(bm);
    }
    if (tid == 0 && offsets) offsets[E] = base;
    if (work)
      for (int sl = (int)n_active + tid; sl < E; sl += kWave) {
        work[(size_t)sl * kWorkWords + 2] = 0u;
        work[(size_t)sl * kWorkWords + 3] = 0u;
      }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int j = tid + i * kDispThreads;
    if (j < P) {
      const uint32_t e = es[i];
      const uint32_t t = (uint32_t)j / (uint32_t)k;
      const uint32_t lo = mlo[e], hi = mhi[e];
      const uint32_t below = t < 32u ? (uint32_t)__popc(lo & ((1u << t) - 1u))
                                     : (uint32_t)(__popc(lo) + __popc(hi & ((1u << (t - 32u)) - 1u)));
      const uint32_t pos = off[e] + below;
      perm[pos] = (uint32_t)j;
      if (inv_perm) inv_perm[j] = pos;
      if (src_of) src_of[pos] = t;
      // source rows of the first rows of every segment, so that a consumer needs one load
      if (work && below < (uint32_t)kWorkSrc) work[(size_t)ridx[e] * kWorkWords + 4 + below] = t;
    }
  }
}

}  // namespace mi_moe
