// Tiled grouped quantized product for long expert segments (prefill).
//
// Same contract as the small-segment kernel (mlx_gather_qmm with transpose = true,
// mlx-rs/src/ops/quantization.rs:160-230; with GLU also nn::silu and multiply,
// nn/activation.rs:142-144,876-880), restricted to the segments the dispatch cut into M tiles
// of 256 rows.  A block computes a 256-token x 128-weight-row tile:
//   * weights stream from HBM as packed codes (one 16-byte load per thread and 64-wide K step),
//     are dequantised ONCE per block to bf16 (w_hat = s q + b, fp32 fma, one rounding) and
//     parked in LDS, so the cost of unpacking is shared by the 256 token rows of the tile;
//   * the token rows are gathered through the sorted-row -> source-row map straight into LDS
//     (no materialised gather);
//   * 4 waves (2 x 2) run v_mfma_f32_32x32x16_bf16 on 128 x 64 sub-tiles, fp32 accumulators;
//   * with GLU the 128 weight rows are 64 gate rows and the matching 64 up rows, each wave owns
//     32 + 32 of them, and the epilogue writes silu(gate) * up without either product ever
//     reaching memory.
// The next K step's global loads are in flight while the current one is multiplied.
#include "common.hpp"

namespace mi_moe {

namespace {

constexpr int BM = kBigTileM;  // token rows per block
constexpr int BK = 64;         // one quantisation group per K step
constexpr int BR = 128;        // weight rows per block (GLU: 64 gate + 64 up)
constexpr int LDK = 72;        // LDS row stride in bf16 (144 bytes: conflict-free 16-byte reads)

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ f32x16_t mfma32(const uint4 &a, const uint4 &b, f32x16_t c) {
  const u32x4_t av = {a.x, a.y, a.z, a.w}, bv = {b.x, b.y, b.z, b.w};
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                 __builtin_bit_cast(bf16x8_t, bv), c, 0, 0, 0);
}

}  // namespace

template <int BITS, bool GLU>
__global__ __launch_bounds__(256, 2) void qmm_large_kernel(GroupedArgs a, int n_ntiles) {
  constexpr int NI = GLU ? 64 : 128;          // distinct output columns per block
  constexpr int BQ = BITS == 4 ? 1 : 2;       // 16-byte weight loads per thread per K step

  // block -> (M tile, N tile): blocks of one M tile share the gathered token rows, so they
  // are given consecutive ids on ONE XCD (ids are dealt round-robin over the 8 XCDs)
  const uint32_t n_mtiles = a.mtiles[0];
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int nt = j % n_ntiles;
  const uint32_t mt_id = (uint32_t)(j / n_ntiles) * 8u + xcd;
  if (mt_id >= n_mtiles) return;
  const uint4 rec = reinterpret_cast<const uint4 *>(a.mtiles)[1 + mt_id];
  const int e = (int)rec.x;
  const int64_t row0 = rec.y;
  const int rows = (int)rec.z;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int N = a.N, K = a.K;
  const int n0 = nt * NI;
  const int row_bytes = K * BITS / 8, gpr = K / 64;

  __shared__ __align__(16) uint16_t As[BM * LDK];
  __shared__ __align__(16) uint16_t Bs[BR * LDK];

  // ---- global -> register stage
  // A: thread covers 8 rows (rg + 32 j) x one 8-element piece (cp) of the K step
  const int cp = tid & 7, rg = tid >> 3;
  const uint16_t *arow[8];
#pragma unroll
  for (int jj = 0; jj < 8; ++jj) {
    int tr = rg + 32 * jj;
    tr = tr < rows ? tr : rows - 1;  // rows past the segment repeat its last row (never stored)
    const int64_t r = row0 + tr;
    const int64_t src = a.src_rows ? (int64_t)a.src_rows[r] : r;
    arow[jj] = a.x + src * K + cp * 8;
  }
  // B: thread covers half a K step (32 codes) of weight row br
  const int br = tid >> 1, bh = tid & 1;
  const int mat = GLU ? (br >> 6) : 0;
  const int nrow = GLU ? n0 + (br & 63) : n0 + br;  // rows >= N read zeros through the descriptor
  const int64_t ebase = (int64_t)e * N;
  const uint32_t *wbase = (mat ? a.w1 : a.w0) + ebase * (row_bytes / 4);
  const uint16_t *sbase = (mat ? a.s1 : a.s0) + ebase * gpr;
  const uint16_t *bbase = (mat ? a.b1 : a.b0) + ebase * gpr;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wbase, (uint32_t)N * row_bytes);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc(sbase, (uint32_t)N * gpr * 2);
  const __amdgpu_buffer_rsrc_t brs = make_rsrc(bbase, (uint32_t)N * gpr * 2);
  const uint32_t w_voff = (uint32_t)nrow * row_bytes + bh * (BITS == 4 ? 16 : 32);
  const uint32_t g_voff = (uint32_t)nrow * gpr * 2;

  uint4 areg[8];
  u32x4_t breg[BQ];
  uint32_t sreg, bireg;
  auto gload = [&](int ks) {
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) areg[jj] = *reinterpret_cast<const uint4 *>(arow[jj] + ks * BK);
#pragma unroll
    for (int q = 0; q < BQ; ++q)
      breg[q] = __builtin_amdgcn_raw_buffer_load_b128(wr, w_voff + q * 16, ks * (BK * BITS / 8), 0);
    sreg = __builtin_amdgcn_raw_buffer_load_b16(sr, g_voff, ks * 2, 0);
    bireg = __builtin_amdgcn_raw_buffer_load_b16(brs, g_voff, ks * 2, 0);
  };

  // ---- register -> LDS stage
  auto stage = [&]() {
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      uint4 v = areg[jj];
      if constexpr (BITS == 4) {  // pair (x_i, x_{i+4}) like the nibble unpacking below
        uint4 p;
        p.x = (v.x & 0xffffu) | (v.z << 16);
        p.y = (v.x >> 16) | (v.z & 0xffff0000u);
        p.z = (v.y & 0xffffu) | (v.w << 16);
        p.w = (v.y >> 16) | (v.w & 0xffff0000u);
        v = p;
      }
      *reinterpret_cast<uint4 *>(&As[(rg + 32 * jj) * LDK + cp * 8]) = v;
    }
    const float sc = bf16lo_to_f32(sreg);
    float bi = bf16lo_to_f32(bireg);
    uint16_t *bdst = &Bs[br * LDK + bh * 32];
    if constexpr (BITS == 4) {
      bi = __builtin_fmaf(-128.0f, sc, bi);  // codes are expanded as 128 + q
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {
        const uint32_t w = breg[0][wi];
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t pr = ((w >> (4 * i)) & 0x000f000fu) | 0x43004300u;  // (128+q_i, 128+q_{i+4})
          o[i] = cvt_pk_bf16(__builtin_fmaf(sc, bf16lo_to_f32(pr), bi), __builtin_fmaf(sc, bf16hi_to_f32(pr), bi));
        }
        *reinterpret_cast<uint4 *>(bdst + wi * 8) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    } else {
#pragma unroll
      for (int q = 0; q < BQ; ++q)
#pragma unroll
        for (int h = 0; h < 2; ++h) {  // 8 codes = two words -> one 16-byte LDS store
          const uint32_t wA = breg[q][2 * h], wB = breg[q][2 * h + 1];
          uint32_t o[4];
          o[0] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wA & 0xffu), bi), __builtin_fmaf(sc, (float)((wA >> 8) & 0xffu), bi));
          o[1] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wA >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wA >> 24), bi));
          o[2] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wB & 0xffu), bi), __builtin_fmaf(sc, (float)((wB >> 8) & 0xffu), bi));
          o[3] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wB >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wB >> 24), bi));
          *reinterpret_cast<uint4 *>(bdst + q * 16 + h * 8) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
  };

  // ---- MFMA stage: wave (wm, wn) owns token rows [128 wm, +128) and two 32-row weight sub-tiles
  f32x16_t acc[4][2];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[m][s][r] = 0.f;
  const int ln = lane & 31, kb = lane >> 5;
  const int brow0 = GLU ? 32 * wn : 64 * wn;       // first sub-tile: gate rows / first 32 rows
  const int brow1 = GLU ? 64 + 32 * wn : 64 * wn + 32;  // second: the matching up rows / next 32
  const uint16_t *ap = &As[(128 * wm + ln) * LDK + kb * 32];
  const uint16_t *bp0 = &Bs[(brow0 + ln) * LDK + kb * 32];
  const uint16_t *bp1 = &Bs[(brow1 + ln) * LDK + kb * 32];

  const int nk = K / BK;
  gload(0);
  for (int ks = 0; ks < nk; ++ks) {
    __syncthreads();  // every wave has finished reading the previous K step
    stage();
    __syncthreads();
    if (ks + 1 < nk) gload(ks + 1);
#pragma unroll
    for (int ss = 0; ss < 4; ++ss) {
      const uint4 b0 = *reinterpret_cast<const uint4 *>(bp0 + ss * 8);
      const uint4 b1 = *reinterpret_cast<const uint4 *>(bp1 + ss * 8);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint4 av = *reinterpret_cast<const uint4 *>(ap + m * 32 * LDK + ss * 8);
        acc[m][0] = mfma32(av, b0, acc[m][0]);
        acc[m][1] = mfma32(av, b1, acc[m][1]);
      }
    }
  }

  // ---- epilogue: D[i][j], lane holds column j = lane % 32 and rows 8 (r/4) + 4 (lane/32) + r%4
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int tr = 128 * wm + 32 * m + 8 * (r >> 2) + 4 * kb + (r & 3);
      if (tr < rows) {
        const int64_t rr = row0 + tr;
        const int64_t dst = a.dst_rows ? (int64_t)a.dst_rows[rr] : rr;
        if constexpr (GLU) {
          const int col = n0 + 32 * wn + ln;
          if (col < N) {
            const float g = acc[m][0][r], u = acc[m][1][r];
            a.y[dst * N + col] = (uint16_t)(cvt_pk_bf16(g / (1.0f + __expf(-g)) * u, 0.f) & 0xffffu);
          }
        } else {
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int col = n0 + 64 * wn + 32 * s + ln;
            if (col < N) a.y[dst * N + col] = (uint16_t)(cvt_pk_bf16(acc[m][s][r], 0.f) & 0xffffu);
          }
        }
      }
    }
}

hipError_t launch_large_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  if (!a.mtiles || a.max_mtiles <= 0) return hipSuccess;
  const int ni = glu ? 64 : 128;
  const int n_ntiles = (a.N + ni - 1) / ni;
  const unsigned grid = (unsigned)((a.max_mtiles + 7) / 8) * 8u * (unsigned)n_ntiles;
  if (a.bits == 4) {
    if (glu) qmm_large_kernel<4, true><<<grid, 256, 0, st>>>(a, n_ntiles);
    else qmm_large_kernel<4, false><<<grid, 256, 0, st>>>(a, n_ntiles);
  } else {
    if (glu) qmm_large_kernel<8, true><<<grid, 256, 0, st>>>(a, n_ntiles);
    else qmm_large_kernel<8, false><<<grid, 256, 0, st>>>(a, n_ntiles);
  }
  return hipGetLastError();
}

}  // namespace mi_moe
