// Grouped quantized products over expert-sorted row segments.
//
// Replaces mlx_gather_qmm (mlx-rs/src/ops/quantization.rs:160-230, transpose = true):
// for every sorted row r of expert e:  y[dst(r)] = x[src(r)] . dequantize(W[e])^T, with
// W in MLX-affine format (uint32 words, low bits first, one bf16 (scale, bias) per 64
// codes).  With GLU the gate and up products share the x operand and the epilogue
// writes silu(gate) * up (nn/activation.rs:142-144,876-880 + multiply), so neither
// product reaches memory.
//
// Arithmetic: sum_c x_c (s q_c + b) = s sum_c x_c q_c + b sum_c x_c per quantisation
// group, in fp32.  The integer codes are exact in bf16, so the matrix cores multiply raw
// codes (no per-element dequantisation, no rounding of w_hat), and scale and bias are
// applied once per group to the fp32 partial sums.
#include "common.hpp"

namespace mi_moe {

__device__ __forceinline__ f32x4_t mfma16(const uint32_t (&a)[4], const uint32_t (&b)[4],
                                          f32x4_t c) {
  typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
  u32x4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                 __builtin_bit_cast(bf16x8_t, bv), c, 0, 0, 0);
}

__device__ __forceinline__ float silu_mul(float g, float u) {
  return g / (1.0f + __expf(-g)) * u;
}

// ---------------------------------------------------------------------------------
// Small-segment kernel (decode): one 16x16x32 MFMA tile = 16 weight rows x TT tokens.
//
// Lane l = (c = l & 15, kb = l >> 4).  B operand (weights): lane holds 8 codes of weight
// row n0+c; A operand (activations): lane holds 8 values of token slot c; D: lane holds
// D[4*kb + r][c], r = 0..3 (rows = token slots, columns = weight rows).
//
// 4-bit: a lane loads one uint4 = 32 consecutive codes, so the four lanes of a row cover
// 128 codes = two quantisation groups (kb 0,1 -> first, kb 2,3 -> second).  To keep the
// groups apart inside one MFMA, the 16 A rows are used as 2 x 8: rows 0-7 carry the TT = 8
// tokens with data only in lanes kb < 2, rows 8-15 carry the same tokens with data only in
// lanes kb >= 2.  D rows 0-7 are then the first group's sums and rows 8-15 the second's.
// A code q is fed as the bf16 value 128+q (0x4300 | q); the offset is folded into the
// bias term.  The nibbles of a word come out as pairs (q_i, q_{i+4}), the activations are
// paired the same way.
//
// 8-bit: a uint4 = 16 codes, the four lanes of a row cover one group of 64, all 16 A rows
// are tokens (TT = 16), codes are converted with v_cvt_f32_ubyte and truncated (exact).
//
// KW waves of a block split K chunk-wise (wave wk takes chunks wk, wk+KW, ...), the other
// 4/KW waves take further row tiles; partial sums meet in LDS and are added in wave order.
template <int BITS, bool GLU, int KW>
__global__ __launch_bounds__(256) void qmm_small_kernel(GroupedArgs a) {
  constexpr int NW = 4 / KW;                    // row tiles per block
  constexpr int TT = BITS == 4 ? 8 : 16;        // tokens per tile
  constexpr int CH = BITS == 4 ? 128 : 64;      // codes per chunk (one uint4 per lane)
  constexpr int XV = BITS == 4 ? 4 : 2;         // uint4 of activations per lane per chunk
  constexpr int NM = GLU ? 2 : 1;

  if (blockIdx.y >= *a.n_active) return;
  const int e = (int)a.active[blockIdx.y];
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const int wk = wave % KW, wn = wave / KW;
  const int c = lane & 15, kb = lane >> 4;
  const int N = a.N, K = a.K;
  const int64_t r0 = a.row_offsets[e];
  const int cnt = (int)(a.row_offsets[e + 1] - a.row_offsets[e]);
  const int n0 = (blockIdx.x * NW + wn) * 16;
  const bool tile_ok = n0 < N;
  const int n = tile_ok ? n0 + c : 0;  // weight row of this lane (B operand / D column)

  const int words_per_row = K * BITS / 32;
  const int groups_per_row = K / 64;
  const int nchunks = (K + CH - 1) / CH;
  const int64_t wrow = ((int64_t)e * N + n);
  const uint32_t *wp[NM];
  const uint16_t *sp[NM], *bp[NM];
  wp[0] = a.w0 + wrow * words_per_row;
  sp[0] = a.s0 + wrow * groups_per_row;
  bp[0] = a.b0 + wrow * groups_per_row;
  if constexpr (GLU) {
    wp[1] = a.w1 + wrow * words_per_row;
    sp[1] = a.s1 + wrow * groups_per_row;
    bp[1] = a.b1 + wrow * groups_per_row;
  }
  const uint32_t ones[4] = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};

  __shared__ float red[KW > 1 ? KW : 1][KW > 1 ? NW : 1][NM][4][KW > 1 ? 64 : 1];

  for (int t0 = 0; t0 < cnt; t0 += TT) {
    // activation row of this lane (A operand)
    const int ts = BITS == 4 ? (c & 7) : c;
    bool a_on = (t0 + ts < cnt);
    if constexpr (BITS == 4) a_on = a_on && ((kb >> 1) == (c >> 3));
    const uint16_t *xrow = a.x;
    if (a_on) {
      const int64_t r = r0 + t0 + ts;
      const int64_t src = a.src_rows ? (int64_t)a.src_rows[r] : r;
      xrow = a.x + src * K;
    }

    f32x4_t tot[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) tot[m] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    for (int ch = wk; ch < nchunks; ch += KW) {
      const int kbase = ch * CH + kb * (CH / 4);  // first code of this lane
      const bool k_ok = kbase < K;
      uint4 q[NM];
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        q[m] = make_uint4(0, 0, 0, 0);
        if (k_ok && tile_ok) q[m] = *reinterpret_cast<const uint4 *>(wp[m] + kbase * BITS / 32);
      }
      uint4 xv[XV];
#pragma unroll
      for (int i = 0; i < XV; ++i) {
        xv[i] = make_uint4(0, 0, 0, 0);
        if (a_on && k_ok) xv[i] = *reinterpret_cast<const uint4 *>(xrow + kbase + i * 8);
      }
      // scale / bias of the group this lane's D rows belong to
      const int g = BITS == 4 ? ch * 2 + (kb >> 1) : ch;
      float sc[NM], bi[NM];
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        sc[m] = 0.f;
        bi[m] = 0.f;
        if (g < groups_per_row && tile_ok) {
          sc[m] = bf16_to_f32(sp[m][g]);
          bi[m] = bf16_to_f32(bp[m][g]);
        }
        if constexpr (BITS == 4) bi[m] = __builtin_fmaf(-128.0f, sc[m], bi[m]);
      }

      f32x4_t acc[NM], xs = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < NM; ++m) acc[m] = f32x4_t{0.f, 0.f, 0.f, 0.f};

      if constexpr (BITS == 4) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint4 v = xv[s];
          uint32_t av[4];
          av[0] = (v.x & 0xffffu) | (v.z << 16);
          av[1] = (v.x >> 16) | (v.z & 0xffff0000u);
          av[2] = (v.y & 0xffffu) | (v.w << 16);
          av[3] = (v.y >> 16) | (v.w & 0xffff0000u);
          xs = mfma16(av, ones, xs);
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            const uint32_t w = s == 0 ? q[m].x : s == 1 ? q[m].y : s == 2 ? q[m].z : q[m].w;
            uint32_t bv[4];
            bv[0] = (w & 0x000f000fu) | 0x43004300u;
            bv[1] = ((w >> 4) & 0x000f000fu) | 0x43004300u;
            bv[2] = ((w >> 8) & 0x000f000fu) | 0x43004300u;
            bv[3] = ((w >> 12) & 0x000f000fu) | 0x43004300u;
            acc[m] = mfma16(av, bv, acc[m]);
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const uint4 v = xv[s];
          const uint32_t av[4] = {v.x, v.y, v.z, v.w};
          xs = mfma16(av, ones, xs);
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            const uint32_t wA = s == 0 ? q[m].x : q[m].z, wB = s == 0 ? q[m].y : q[m].w;
            uint32_t bv[4];
            bv[0] = (__float_as_uint((float)(wA & 0xffu)) >> 16) |
                    (__float_as_uint((float)((wA >> 8) & 0xffu)) & 0xffff0000u);
            bv[1] = (__float_as_uint((float)((wA >> 16) & 0xffu)) >> 16) |
                    (__float_as_uint((float)(wA >> 24)) & 0xffff0000u);
            bv[2] = (__float_as_uint((float)(wB & 0xffu)) >> 16) |
                    (__float_as_uint((float)((wB >> 8) & 0xffu)) & 0xffff0000u);
            bv[3] = (__float_as_uint((float)((wB >> 16) & 0xffu)) >> 16) |
                    (__float_as_uint((float)(wB >> 24)) & 0xffff0000u);
            acc[m] = mfma16(av, bv, acc[m]);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          tot[m][r] += sc[m] * acc[m][r] + bi[m] * xs[r];
    }

    if constexpr (BITS == 4) {  // rows 8-15 (second group of each chunk) onto rows 0-7
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) tot[m][r] += __shfl_xor(tot[m][r], 32, kWave);
    }

    // cross-wave sum over the K split, in wave order
    constexpr int LR = BITS == 4 ? 32 : 64;  // lanes that hold distinct results
    float res[NM][4];
    if constexpr (KW == 1) {
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) res[m][r] = tot[m][r];
    } else {
      __syncthreads();  // the previous token tile's readers are done with the buffer
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wk][wn][m][r][lane] = tot[m][r];
      __syncthreads();
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < KW; ++w) s += red[w][wn][m][r][lane];
          res[m][r] = s;
        }
    }

    // epilogue: one wave per row tile writes TT x 16 outputs
    if (wk == 0 && tile_ok && lane < LR) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int slot = BITS == 4 ? 4 * (kb & 1) + r : 4 * kb + r;
        if (t0 + slot < cnt) {
          const int64_t rr = r0 + t0 + slot;
          const int64_t dst = a.dst_rows ? (int64_t)a.dst_rows[rr] : rr;
          float v;
          if constexpr (GLU) v = silu_mul(res[0][r], res[1][r]);
          else v = res[0][r];
          a.y[dst * N + n] = f32_to_bf16(v);
        }
      }
    }
  }
}

template <int BITS, bool GLU>
static void launch_small(const GroupedArgs &a, hipStream_t st) {
  // split K over the 4 waves of a block when there are too few row tiles to fill the chip
  const int64_t tiles = (int64_t)(a.N / 16) * a.max_active;
  const int chunks = (a.K + (BITS == 4 ? 127 : 63)) / (BITS == 4 ? 128 : 64);
  int kw = 1;
  if (tiles < 8192 && chunks >= 8) kw = 4;
  else if (tiles < 16384 && chunks >= 4) kw = 2;
  const int nw = 4 / kw;
  dim3 grid((unsigned)((a.N + 16 * nw - 1) / (16 * nw)), (unsigned)a.max_active);
  if (kw == 4) qmm_small_kernel<BITS, GLU, 4><<<grid, 256, 0, st>>>(a);
  else if (kw == 2) qmm_small_kernel<BITS, GLU, 2><<<grid, 256, 0, st>>>(a);
  else qmm_small_kernel<BITS, GLU, 1><<<grid, 256, 0, st>>>(a);
}

hipError_t launch_grouped_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  if (a.max_active <= 0 || a.total_rows <= 0) return hipSuccess;
  if (a.bits == 4) {
    if (glu) launch_small<4, true>(a, st);
    else launch_small<4, false>(a, st);
  } else {
    if (glu) launch_small<8, true>(a, st);
    else launch_small<8, false>(a, st);
  }
  return hipGetLastError();
}

}  // namespace mi_moe
