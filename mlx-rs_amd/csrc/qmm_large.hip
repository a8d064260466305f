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
constexpr int BK = 32;         // K step (two steps per quantisation group)
constexpr int BR = 128;        // weight rows per block (GLU: 64 gate + 64 up)

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// LDS tiles hold rows of 32 bf16 (four 16-byte chunks) at a stride of 80 bytes: consecutive
// rows reading the same chunk start 20 banks apart, which keeps 16-byte reads of 8 or 16
// consecutive rows free of bank conflicts (measured: SQ_LDS_BANK_CONFLICT = 0).
constexpr int LDR = 5;  // row stride in uint4 units
__device__ __forceinline__ int tile_off(int row, int chunk) { return row * LDR + chunk; }

}  // namespace

template <int BITS, bool GLU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void qmm_large_kernel(GroupedArgs a, int n_ntiles) {
  constexpr int NI = GLU ? 64 : 128;  // distinct output columns per block

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

  __shared__ u32x4_t As[2][BM * LDR];
  __shared__ u32x4_t Bs[2][BR * LDR];

  // ---- global -> register stage
  // A: the activations arrive with every 8-block already in the (x0,x4,x1,x5,x2,x6,x3,x7) order
  // of the nibble unpacking (4-bit), so a row chunk is copied as it is.  Thread: chunk acp of
  // rows arg + 64 j.
  const int acp = tid & 3, arg = tid >> 2;
  auto a_row_ptr = [&](int tr) {
    tr = tr < rows ? tr : rows - 1;  // rows past the segment repeat its last row (never stored)
    const int64_t r = row0 + tr;
    const int64_t src = a.src_rows ? (int64_t)a.src_rows[r] : r;
    return a.x_perm + src * K + acp * 8;
  };
  const uint16_t *const arow[4] = {a_row_ptr(arg), a_row_ptr(arg + 64), a_row_ptr(arg + 128), a_row_ptr(arg + 192)};
  // B: thread covers 16 codes (half a K step) of weight row br; waves 0,1 / 2,3 hold gate / up
  const int br = tid >> 1, bh = tid & 1;
  const int mat = GLU ? (wave >> 1) : 0;  // wave-uniform
  const int nrow = GLU ? n0 + (br & 63) : n0 + br;  // rows >= N read zeros through the descriptor
  const int64_t ebase = (int64_t)e * N;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc((mat ? a.w1 : a.w0) + ebase * (row_bytes / 4), (uint32_t)N * row_bytes);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc((mat ? a.s1 : a.s0) + ebase * gpr, (uint32_t)N * gpr * 2);
  const __amdgpu_buffer_rsrc_t brs = make_rsrc((mat ? a.b1 : a.b0) + ebase * gpr, (uint32_t)N * gpr * 2);
  const uint32_t w_voff = (uint32_t)nrow * row_bytes + bh * (BITS == 4 ? 8 : 16);
  const uint32_t g_voff = (uint32_t)nrow * gpr * 2;

  // Two sets of staging registers (plain scalars: they must not end up in scratch or LDS), so
  // that global loads are issued two K steps before their data is needed.
  struct Stage {
    u32x4_t a0, a1, a2, a3;
    uint32_t b0w, b1w, b2w, b3w;  // 4-bit: two words used
    uint32_t sreg, bireg;
  };
  auto gload = [&](int ks, Stage &R) __attribute__((always_inline)) {
    R.a0 = *reinterpret_cast<const u32x4_t *>(arow[0] + ks * BK);
    R.a1 = *reinterpret_cast<const u32x4_t *>(arow[1] + ks * BK);
    R.a2 = *reinterpret_cast<const u32x4_t *>(arow[2] + ks * BK);
    R.a3 = *reinterpret_cast<const u32x4_t *>(arow[3] + ks * BK);
    if constexpr (BITS == 4) {
      const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(wr, w_voff, ks * 16, 0);
      R.b0w = v[0];
      R.b1w = v[1];
    } else {
      const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(wr, w_voff, ks * 32, 0);
      R.b0w = v[0];
      R.b1w = v[1];
      R.b2w = v[2];
      R.b3w = v[3];
    }
    R.sreg = __builtin_amdgcn_raw_buffer_load_b16(sr, g_voff, (ks >> 1) * 2, 0);
    R.bireg = __builtin_amdgcn_raw_buffer_load_b16(brs, g_voff, (ks >> 1) * 2, 0);
  };

  // ---- register -> LDS stage: copy A, dequantise B once for the whole block
  auto stage = [&](int buf, const Stage &R) __attribute__((always_inline)) {
    As[buf][tile_off(arg, acp)] = R.a0;
    As[buf][tile_off(arg + 64, acp)] = R.a1;
    As[buf][tile_off(arg + 128, acp)] = R.a2;
    As[buf][tile_off(arg + 192, acp)] = R.a3;
    const float sc = bf16lo_to_f32(R.sreg);
    float bi = bf16lo_to_f32(R.bireg);
    if constexpr (BITS == 4) {
      bi = __builtin_fmaf(-128.0f, sc, bi);  // codes are expanded as 128 + q
#pragma unroll
      for (int wi = 0; wi < 2; ++wi) {
        const uint32_t w = wi == 0 ? R.b0w : R.b1w;
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t pr = ((w >> (4 * i)) & 0x000f000fu) | 0x43004300u;  // (128+q_i, 128+q_{i+4})
          o[i] = cvt_pk_bf16(__builtin_fmaf(sc, bf16lo_to_f32(pr), bi), __builtin_fmaf(sc, bf16hi_to_f32(pr), bi));
        }
        Bs[buf][tile_off(br, 2 * bh + wi)] = u32x4_t{o[0], o[1], o[2], o[3]};
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // 8 codes = two words -> one chunk
        const uint32_t wA = h == 0 ? R.b0w : R.b2w, wB = h == 0 ? R.b1w : R.b3w;
        uint32_t o[4];
        o[0] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wA & 0xffu), bi), __builtin_fmaf(sc, (float)((wA >> 8) & 0xffu), bi));
        o[1] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wA >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wA >> 24), bi));
        o[2] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wB & 0xffu), bi), __builtin_fmaf(sc, (float)((wB >> 8) & 0xffu), bi));
        o[3] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wB >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wB >> 24), bi));
        Bs[buf][tile_off(br, 2 * bh + h)] = u32x4_t{o[0], o[1], o[2], o[3]};
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
  const int brow0 = (GLU ? 32 * wn : 64 * wn) + ln;            // gate rows / first 32 rows
  const int brow1 = (GLU ? 64 + 32 * wn : 64 * wn + 32) + ln;  // the matching up rows / next 32
  const int arow0 = 128 * wm + ln;

  auto mma = [&](int cur) __attribute__((always_inline)) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss) {
      const int c = 2 * kb + ss;
      const u32x4_t b0 = Bs[cur][tile_off(brow0, c)];
      const u32x4_t b1 = Bs[cur][tile_off(brow1, c)];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const u32x4_t av = As[cur][tile_off(arow0 + 32 * m, c)];
        acc[m][0] = mfma32(av, b0, acc[m][0]);
        acc[m][1] = mfma32(av, b1, acc[m][1]);
      }
    }
  };

  // K loop, two steps per trip (nk is even: K is a multiple of 64).  Entering step ks: LDS buffer
  // ks & 1 holds step ks, register set R1/R0 holds step ks + 1, the load of step ks + 2 is in flight.
  const int nk = K / BK;
  Stage R0, R1;
  gload(0, R0);
  gload(1, R1);
  stage(0, R0);
  if (nk > 2) gload(2, R0);
  __syncthreads();
  for (int ks = 0; ks < nk; ks += 2) {
    stage(1, R1);                          // step ks + 1 -> buffer 1 (last read before the previous barrier)
    if (ks + 3 < nk) gload(ks + 3, R1);
    mma(0);                                // step ks
    __syncthreads();
    if (ks + 2 < nk) stage(0, R0);         // step ks + 2 -> buffer 0
    if (ks + 4 < nk) gload(ks + 4, R0);
    mma(1);                                // step ks + 1
    __syncthreads();
  }

  // ---- epilogue: D[i][j], lane holds column j = lane % 32 and rows 8 (r/4) + 4 (lane/32) + r%4.
  // perm_out: columns are written in the paired order within each 8-block (what a 4-bit
  // consumer of these rows expects as its activations).
  auto out_col = [&](int col) {
    if (!a.y_paired) return col;
    const int jj = col & 7;
    return (col & ~7) | (jj < 4 ? 2 * jj : 2 * (jj - 4) + 1);
  };
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
            a.y[dst * N + out_col(col)] = (uint16_t)(cvt_pk_bf16(g / (1.0f + __expf(-g)) * u, 0.f) & 0xffffu);
          }
        } else {
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int col = n0 + 64 * wn + 32 * s + ln;
            if (col < N) a.y[dst * N + out_col(col)] = (uint16_t)(cvt_pk_bf16(acc[m][s][r], 0.f) & 0xffffu);
          }
        }
      }
    }
}

// Activation rows with every 8-block reordered to (x0,x4,x1,x5,x2,x6,x3,x7): the order in which
// one and+or per register unpacks the eight 4-bit codes of a word.
__global__ __launch_bounds__(256) void pair_rows_kernel(const uint4 *__restrict__ x, int64_t n, uint4 *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint4 v = x[i];
  uint4 p;
  p.x = (v.x & 0xffffu) | (v.z << 16);
  p.y = (v.x >> 16) | (v.z & 0xffff0000u);
  p.z = (v.y & 0xffffu) | (v.w << 16);
  p.w = (v.y >> 16) | (v.w & 0xffff0000u);
  out[i] = p;
}

hipError_t launch_pair_rows(const uint16_t *x, int64_t rows, int K, uint16_t *out, hipStream_t st) {
  const int64_t n = rows * K / 8;
  if (n == 0) return hipSuccess;
  pair_rows_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(reinterpret_cast<const uint4 *>(x), n,
                                                               reinterpret_cast<uint4 *>(out));
  return hipGetLastError();
}

hipError_t launch_large_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  if (!a.mtiles || a.max_mtiles <= 0 || !a.x_perm) return hipSuccess;
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
