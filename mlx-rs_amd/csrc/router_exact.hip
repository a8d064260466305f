// Router logits for prefill-sized batches on the int8 matrix cores, with the bits of the fp64 kernels.
//
// Replaces the same op as router.hip's logits kernels: ops::matmul via a bias-free nn::Linear
// (mlx-rs/src/nn/linear.rs:84-96, ops/arithmetic.rs:577-603).  Those accumulate the exact bf16 x bf16
// products in fp64 on the fp64 matrix cores: 2 T E H flops at 78.6 TFLOP/s, 45 us at 4096 tokens x 128
// experts x 2048, as long as a fifth of the expert products.  Here the same VALUE is computed in integer
// arithmetic, which the int8 matrix cores do 60 times faster, and every result that the integer route
// cannot vouch for is recomputed the old way.
//
// A bf16 number is m * 2^e with an 8-bit m.  A row (of x or of the router matrix) is rewritten in fixed
// point on the row's own scale: X_i = m_i shifted so that the row's largest element keeps 14 bits below
// its last place; |X_i| < 2^22.  Elements more than 2^14 times smaller than the row's largest lose low
// bits: their lost parts are summed per row (rsum), which bounds what the row contributes to any error.
// X = a2 2^16 + a1 2^8 + a0 in signed bytes, so  sum_i X_i W_i = sum_{j,l} 2^(8(j+l)) sum_i a_j,i b_l,i:
// nine int8 products with int32 accumulation (|sum| <= 2^14 H: exact for H <= 32768), five accumulators
// (one per j + l), combined exactly in int64.  The logit is that integer times the two rows' units.
// With no element truncated this IS the exact sum; in general it lies within
//     delta = 2 rsum_x |w|max + rsum_w |x|max  (+ the fp64 roundings both routes make)
// of it.  The result is rounded fp64 -> fp32 -> bf16 like the fp64 kernels'.  If a point within delta
// (plus two fp32 ulps for the double rounding) of the value rounds differently, i.e. the value sits that
// close to the midpoint of two bf16 numbers, or a row holds an infinity or a NaN, the logit is
// recomputed by logit_wave (fp64, router_dev.hpp).  For data without extreme dynamic range inside a row
// that happens for a few logits in a hundred thousand.
#include <type_traits>

#include "router_dev.hpp"

namespace mi_moe {

namespace {

constexpr int kFixShift = 14;  // bits kept below the last place of a row's largest element
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

struct RowMeta {
  int32_t unit_exp;   // value of element i = X_i * 2^unit_exp
  float absmax;       // largest |element| of the row
  float rsum;         // upper bound of the sum of the |parts lost to truncation|
  uint32_t nonfinite; // the row holds an infinity or a NaN
};
static_assert(sizeof(RowMeta) == 16, "one 16-byte load per row");

// Byte planes are stored for the matrix kernel's loads: rows in tiles of 32, and inside a tile chunk after chunk
// of 32 bytes per row, [row tile][chunk of 32 h][half of the chunk][row in tile][16 bytes], so that the 32 rows x
// 32 bytes which a wave multiplies at a time are one contiguous KiB in the order of its lanes (lane = half * 32 +
// row, 16 bytes each).  Offset of byte h of `row`:
__host__ __device__ __forceinline__ int64_t plane_off(int64_t row, int h, int H) {
  return ((((row >> 5) * (H >> 5) + (h >> 5)) * 2 + ((h >> 4) & 1)) * 32 + (row & 31)) * 16 + (h & 15);
}
__host__ __device__ __forceinline__ int64_t plane_bytes(int64_t rows, int H) { return ((rows + 31) / 32) * 32 * (int64_t)H; }

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  return ((uint32_t)a & 0xffu) | (((uint32_t)b & 0xffu) << 8) | (((uint32_t)c & 0xffu) << 16) | ((uint32_t)d << 24);
}

}  // namespace

// One wave per row of x (rows 0 .. T-1) or of the router matrix (rows T .. T+E-1): the three byte planes and the
// row's meta data.  NV: 16-byte pieces of the row a lane keeps in registers between the pass that finds the row's
// scale and the pass that writes the planes (NV * 512 >= H), or 0: the row is read twice.
// x_paired (optional): the copy of x with every 8-block in the order (x0,x4,x1,x5,x2,x6,x3,x7) that the 4-bit
// tiled product reads.
template <int NV>
__global__ __launch_bounds__(256) void router_slice_kernel(const uint16_t *__restrict__ x, int64_t T,
                                                           const uint16_t *__restrict__ w, int64_t E, int H,
                                                           int8_t *__restrict__ px, int8_t *__restrict__ pw,
                                                           RowMeta *__restrict__ mx, RowMeta *__restrict__ mw,
                                                           uint16_t *__restrict__ x_paired) {
  const int lane = lane_id();
  int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const bool is_x = row < T;
  if (!is_x) row -= T;
  if (!is_x && row >= E) return;
  const uint16_t *src = (is_x ? x : w) + row * H;
  int8_t *planes = is_x ? px : pw;
  const int64_t plane_stride = plane_bytes(is_x ? T : E, H);
  constexpr int NR = NV > 0 ? NV : 1;
  const int n_iter = NV > 0 ? NV : (H + kWave * 8 - 1) / (kWave * 8);

  // the row's largest exponent field (subnormals count as field 1: same scale, no hidden bit)
  uint4 keep[NR];
  uint32_t emax = 1, nf = 0;
  float absmax = 0.f;
  auto scan = [&](const uint4 v) __attribute__((always_inline)) {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint32_t b = half ? u[q] >> 16 : u[q] & 0xffffu;
        const uint32_t eb = (b >> 7) & 0xffu;
        emax = eb > emax ? eb : emax;
        nf |= eb == 255u;
        absmax = fmaxf(absmax, __uint_as_float((b & 0x7fffu) << 16));
      }
    }
  };
  if constexpr (NV > 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int h = lane * 8 + i * kWave * 8;
      keep[i] = h < H ? *reinterpret_cast<const uint4 *>(src + h) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) scan(keep[i]);
  } else {
    for (int i = 0; i < n_iter; ++i) {
      const int h = lane * 8 + i * kWave * 8;
      if (h < H) scan(*reinterpret_cast<const uint4 *>(src + h));
    }
  }
  emax = wave_max_u32(emax);
  absmax = wave_max_f32(absmax);
  nf = __ballot(nf != 0u) != 0ull;

  // Fixed point by float arithmetic: element * 2^-unit_exp is exact (a power of two), has at most 22 bits before
  // the point, and v_cvt_i32_f32 drops what lies behind it (toward zero); the dropped part is exact as well.
  // Rows whose largest element is below 2^-110 are put on the scale of 2^-110 (the factor must be a float): their
  // small elements lose bits like any others and the bound sees it.
  const uint32_t emax_eff = emax > 24u ? emax : 24u;
  const float to_fixed = __uint_as_float((275u - emax_eff) << 23);  // 2^(148 - emax_eff)
  float rsum = 0.f;  // in units of 2^unit_exp
  auto slice = [&](const uint4 v, int h) __attribute__((always_inline)) {
    if (is_x && x_paired) {
      uint4 p;
      p.x = (v.x & 0xffffu) | (v.z << 16);
      p.y = (v.x >> 16) | (v.z & 0xffff0000u);
      p.z = (v.y & 0xffffu) | (v.w << 16);
      p.w = (v.y >> 16) | (v.w & 0xffff0000u);
      *reinterpret_cast<uint4 *>(x_paired + row * H + h) = p;
    }
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    int d0[8], d1[8], d2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float y = ((i & 1) ? bf16hi_to_f32(u[i >> 1]) : bf16lo_to_f32(u[i >> 1])) * to_fixed;
      const int Xs = (int)y;  // toward zero
      rsum += fabsf(y - (float)Xs);
      const int a0 = __builtin_amdgcn_sbfe(Xs, 0, 8);
      const int X1 = (Xs - a0) >> 8;
      const int a1 = __builtin_amdgcn_sbfe(X1, 0, 8);
      d0[i] = a0;
      d1[i] = a1;
      d2[i] = (X1 - a1) >> 8;
    }
    int8_t *dst = planes + plane_off(row, h, H);
    *reinterpret_cast<uint2 *>(dst) = make_uint2(pack4(d0[0], d0[1], d0[2], d0[3]), pack4(d0[4], d0[5], d0[6], d0[7]));
    *reinterpret_cast<uint2 *>(dst + plane_stride) = make_uint2(pack4(d1[0], d1[1], d1[2], d1[3]), pack4(d1[4], d1[5], d1[6], d1[7]));
    *reinterpret_cast<uint2 *>(dst + 2 * plane_stride) = make_uint2(pack4(d2[0], d2[1], d2[2], d2[3]), pack4(d2[4], d2[5], d2[6], d2[7]));
  };
  if constexpr (NV > 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int h = lane * 8 + i * kWave * 8;
      if (h < H) slice(keep[i], h);
    }
  } else {
    for (int i = 0; i < n_iter; ++i) {
      const int h = lane * 8 + i * kWave * 8;
      if (h < H) slice(*reinterpret_cast<const uint4 *>(src + h), h);
    }
  }
  // (the order of a float sum is not fixed: the bound is raised by more than any order can differ)
  rsum = (float)wave_sum_f64((double)rsum) * 1.0001f * __uint_as_float((emax_eff - 21u) << 23);  // * 2^unit_exp
  if (lane == 0) {
    RowMeta mt;
    mt.unit_exp = (int)emax_eff - 134 - kFixShift;
    mt.absmax = absmax;
    mt.rsum = rsum;
    mt.nonfinite = nf;
    (is_x ? mx : mw)[row] = mt;
  }
}

// A block computes a 32-token x 32-expert tile with v_mfma_i32_32x32x32_i8; its four waves split H (wave w takes the
// chunks of its quarter) and their integer accumulators are added through LDS (integers: any order gives the same sum).
// Lane (ln = lane % 32, kh = lane / 32) holds bytes [32 c + 16 kh, + 16) of row ln of its operand in chunk c, for the
// token rows and the expert rows alike, so the k index inside the instruction never has to be known.  A chunk of an
// operand is one contiguous KiB (plane_off).  Three chunks of loads are in flight per wave.
__global__ __launch_bounds__(256) void router_i8_kernel(const int8_t *__restrict__ px, const int8_t *__restrict__ pw,
                                                        const RowMeta *__restrict__ mx, const RowMeta *__restrict__ mw,
                                                        const float *__restrict__ bias, const uint16_t *__restrict__ x,
                                                        const uint16_t *__restrict__ wg, int64_t T, int H, int E,
                                                        uint16_t *__restrict__ logits) {
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, kh = lane >> 5;
  const int64_t t0 = (int64_t)blockIdx.x * 32;
  const int e0 = blockIdx.y * 32;
  const int nchunks = H / 32;
  const int64_t xs = plane_bytes(T, H), ws = plane_bytes(E, H);  // plane strides
  // chunk c of the block's token tile / expert tile: 1 KiB, this lane's 16 bytes at lane * 16
  const int8_t *ap = px + (int64_t)blockIdx.x * nchunks * 1024 + lane * 16;
  const int8_t *bp = pw + (int64_t)blockIdx.y * nchunks * 1024 + lane * 16;

  v16i_t acc[5];
#pragma unroll
  for (int k = 0; k < 5; ++k)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[k][r] = 0;

  struct Chunk {
    v4i_t a[3], b[3];
  };
  const int per = (nchunks + 3) / 4;
  const int c0 = wave * per, c1 = c0 + per < nchunks ? c0 + per : nchunks;
  auto fetch = [&](int c, Chunk &R) __attribute__((always_inline)) {
    int cc = c < nchunks ? c : nchunks - 1;
    asm volatile("" : "+s"(cc));  // (an opaque index keeps the prefetch where it is written)
#pragma unroll
    for (int p = 0; p < 3; ++p) {
      R.a[p] = *reinterpret_cast<const v4i_t *>(ap + p * xs + (int64_t)cc * 1024);
      R.b[p] = *reinterpret_cast<const v4i_t *>(bp + p * ws + (int64_t)cc * 1024);
    }
  };
  auto multiply = [&](const Chunk &R) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int l = 0; l < 3; ++l) acc[j + l] = __builtin_amdgcn_mfma_i32_32x32x32_i8(R.a[j], R.b[l], acc[j + l], 0, 0, 0);
  };
  constexpr int D = 4;  // chunks of loads in flight per wave
  Chunk ring[D];
#pragma unroll
  for (int d = 0; d < D - 1; ++d) fetch(c0 + d, ring[d]);
  int c = c0;
  for (; c + D <= c1; c += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      fetch(c + d + D - 1, ring[(d + D - 1) % D]);
      __builtin_amdgcn_sched_barrier(0);
      multiply(ring[d]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#pragma unroll
  for (int d = 0; d < D - 1; ++d)  // (up to D - 1 chunks left; they sit in their slots)
    if (c + d < c1) multiply(ring[d]);

  // Each wave's partial tile as exact 64-bit integers (sum_k acc_k 256^k), then wave w adds the four partial tiles
  // for the registers [4 w, 4 w + 4) (token rows 8 w .. 8 w + 7) and finishes those: the conversion, the check and
  // the recomputations are spread over the four waves.
  __shared__ int64_t sred[4][16][64];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int64_t S = 0;
#pragma unroll
    for (int k = 4; k >= 0; --k) S = S * 256 + (int64_t)acc[k][r];
    sred[wave][r][lane] = S;
  }
  __syncthreads();

  // D[i][j]: lane holds column j = ln (expert) and rows i = 8 (r / 4) + 4 kh + r % 4 (tokens)
  const int e = e0 + ln;
  const RowMeta we = mw[e < E ? e : E - 1];
  const float be = bias && e < E ? bias[e] : 0.f;
  uint16_t out[4];
  uint32_t redo = 0;  // bit i: recompute in fp64
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * wave + i;
    const int64_t t = t0 + 8 * (r >> 2) + 4 * kh + (r & 3);
    const RowMeta xt = mx[t < T ? t : T - 1];
    const int64_t S = (sred[0][r][lane] + sred[1][r][lane]) + (sred[2][r][lane] + sred[3][r][lane]);
    double v = ldexp((double)S, xt.unit_exp + we.unit_exp);
    if (bias) v += (double)be;
    const float f = (float)v;
    const uint32_t u = __float_as_uint(f);
    out[i] = f32_to_bf16(f);
    // how far f is from the midpoint of two bf16 numbers, in fp32 ulps, against the error bound in the same unit
    const int dist = abs((int)(u & 0xffffu) - 0x8000);
    const uint32_t ef = (u >> 23) & 0xffu;
    const float ulp = __uint_as_float((ef > 24u ? ef - 23u : 1u) << 23);  // 2^(ef - 150); logits below 2^-102 are recomputed
    // what truncated elements can contribute, and 2^-38 H |x|max |w|max for the fp64 roundings of either route
    const float delta = 2.f * xt.rsum * we.absmax + we.rsum * xt.absmax + 3.64e-12f * (float)H * xt.absmax * we.absmax;
    bool safe = ef > 24u && ef != 255u && (float)dist * ulp > delta * 1.0001f + 2.5f * ulp;
    // a row of zeros (a padding token): every product is zero and the sum is +0 by either route, in any order
    if (xt.absmax == 0.f || we.absmax == 0.f) safe = true;
    safe = safe && !xt.nonfinite && !we.nonfinite;
    if (!safe && t < T && e < E) redo |= 1u << i;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * wave + i;
    uint64_t todo = __ballot((redo >> i) & 1u);
    while (todo) {  // (wave-uniform)
      const int srcl = __builtin_ctzll(todo);
      todo &= todo - 1;
      const int64_t t = t0 + 8 * (r >> 2) + 4 * (srcl >> 5) + (r & 3);
      const int ee = e0 + (srcl & 31);
      double s = logit_wave(x + t * H, wg + (int64_t)ee * H, H);
      if (bias) s += (double)bias[ee];
      if (lane == srcl) out[i] = f32_to_bf16((float)s);
    }
  }
  if (e < E) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * wave + i;
      const int64_t t = t0 + 8 * (r >> 2) + 4 * kh + (r & 3);
      if (t < T) logits[t * E + e] = out[i];
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Up to 128 experts: logits AND selection in one kernel.  A block of eight waves owns 32 tokens and all experts, so
// the byte planes of x never leave the CU and the selection reads the finished logits from LDS:
//   1. every wave scans four token rows (scale, largest element, infinities / NaNs; the paired copy of x goes out here);
//   2. H is walked in slabs of 1024 values: the waves rewrite their rows' part of the slab as byte planes in LDS, in the
//      order of the multiplying lanes ([chunk][half][row][16 bytes], blocks of 512 + 16 bytes: the 16 keep the writing
//      lanes, a block apart each, off each other's banks), then wave (ks, n) multiplies half of the slab's chunks
//      with expert tile n, whose planes (router_slice_kernel, 128 rows) come from L2;
//   3. the two partial tiles of an expert tile meet in LDS as 64-bit integers; each wave finishes eight token rows of
//      its tile (conversion, error bound, fp64 where the bound does not decide), writes the logits out and into LDS;
//   4. every wave selects for four tokens (select_from_bits, the selection of router.hip).
#ifndef MI_TILE_WAVES
#define MI_TILE_WAVES 8   // (sixteen waves: 128 registers each, 26 of them spilled; 4096 tokens 43.1 -> 45.5 us)
#endif
constexpr int kSlab = 1024;                       // values of x per slab
constexpr int kPlaneBlock = 512 + 16;             // bytes from one (chunk, half) block of a plane in LDS to the next
constexpr int kPlaneLds = (kSlab / 16) * kPlaneBlock;  // one plane of a slab
#ifndef MI_TILE_KEEP
#define MI_TILE_KEEP 1
#endif
// LDS: the planes of a slab, later reused for the waves' partial tiles (8 KiB each) and the logits (8 KiB); behind
// both, the token rows' meta data
constexpr int kReuseLds = MI_TILE_WAVES * 8192 + 8192;
constexpr int kMetaOff = 3 * kPlaneLds > kReuseLds ? 3 * kPlaneLds : kReuseLds;
constexpr int kTileLds = kMetaOff + 32 * 32;
struct TokenMeta {
  float to_fixed;   // 2^-unit_exp
  int32_t unit_exp;
  float absmax;
  float rsum;       // in units of 2^unit_exp until the last slab, then in the row's own unit
  uint32_t nonfinite;
  uint32_t pad[3];
};
static_assert(sizeof(TokenMeta) == 32, "meta region");

// NW waves per block: each scans and slices 32 / NW token rows, multiplies one of NW / 4 shares of a slab's chunks
// with one of the four expert tiles, finishes 64 / NW accumulator registers (token rows) and selects for 32 / NW tokens.
// KEEP: the rows a wave scans stay in its registers until they are sliced (H <= 2048: four 16-byte pieces per lane
// and row), else they are read again.
template <int NW, bool KEEP>
__global__ __launch_bounds__(NW * 64) void router_tile_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ pw,
                                                             const RowMeta *__restrict__ mw, const float *__restrict__ bias,
                                                             const uint16_t *__restrict__ wg, int64_t T, int H, int E, int k,
                                                             int mode, uint16_t *__restrict__ logits,
                                                             uint32_t *__restrict__ topk_idx, uint16_t *__restrict__ topk_w,
                                                             uint16_t *__restrict__ x_paired) {
  constexpr int RW = 32 / NW;   // token rows per wave
  constexpr int KS = NW / 4;    // shares of a slab's chunks
  constexpr int FR = 16 / KS;   // accumulator registers a wave finishes
  constexpr int NP = KEEP ? 4 : 1;
  extern __shared__ __align__(16) unsigned char tile_lds[];
  static_assert(NW * 8192 + 8192 <= kMetaOff, "the reused region must end before the meta data");
  TokenMeta *const meta = reinterpret_cast<TokenMeta *>(tile_lds + kMetaOff);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t t0 = (int64_t)blockIdx.x * 32;

  // ---- 1. the rows' scales (all loads of the wave's rows first: one round trip)
  uint4 keep[RW][NP];
  const uint16_t *rowp[RW];
#pragma unroll
  for (int i = 0; i < RW; ++i) {
    const int r = RW * wave + i;
    rowp[i] = x + (t0 + r < T ? t0 + r : T - 1) * H;
    if constexpr (KEEP) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int h = lane * 8 + j * kWave * 8;
        keep[i][j] = h < H ? *reinterpret_cast<const uint4 *>(rowp[i] + h) : make_uint4(0, 0, 0, 0);
      }
    }
  }
  float to_fixed[RW], lost[RW];
#pragma unroll
  for (int i = 0; i < RW; ++i) {
    const int r = RW * wave + i;
    uint32_t emax = 1, nf = 0;
    float absmax = 0.f;
    auto scan = [&](const uint4 v, int h) __attribute__((always_inline)) {
      if (x_paired && t0 + r < T && h < H) {
        uint4 p;
        p.x = (v.x & 0xffffu) | (v.z << 16);
        p.y = (v.x >> 16) | (v.z & 0xffff0000u);
        p.z = (v.y & 0xffffu) | (v.w << 16);
        p.w = (v.y >> 16) | (v.w & 0xffff0000u);
        *reinterpret_cast<uint4 *>(x_paired + (t0 + r) * H + h) = p;
      }
      const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const uint32_t b = half ? u[q] >> 16 : u[q] & 0xffffu;
          const uint32_t eb = (b >> 7) & 0xffu;
          emax = eb > emax ? eb : emax;
          nf |= eb == 255u;
          absmax = fmaxf(absmax, __uint_as_float((b & 0x7fffu) << 16));
        }
      }
    };
    if constexpr (KEEP) {
#pragma unroll
      for (int j = 0; j < 4; ++j) scan(keep[i][j], lane * 8 + j * kWave * 8);
    } else {
      for (int h = lane * 8; h < H; h += kWave * 8) scan(*reinterpret_cast<const uint4 *>(rowp[i] + h), h);
    }
    emax = wave_max_u32(emax);
    absmax = wave_max_f32(absmax);
    const bool any_nf = __ballot(nf != 0u) != 0ull;
    const uint32_t emax_eff = emax > 24u ? emax : 24u;
    to_fixed[i] = __uint_as_float((275u - emax_eff) << 23);
    lost[i] = 0.f;
    if (lane == 0) {
      TokenMeta mt;
      mt.to_fixed = to_fixed[i];
      mt.unit_exp = (int)emax_eff - 134 - kFixShift;
      mt.absmax = absmax;
      mt.rsum = 0.f;
      mt.nonfinite = any_nf;
      mt.pad[0] = mt.pad[1] = mt.pad[2] = 0u;
      meta[r] = mt;
    }
  }

  // ---- 2. slabs: slice into LDS, multiply
  const int ln = lane & 31, kh = lane >> 5;
  const int ks = wave >> 2, n = wave & 3;   // share of a slab's chunks, expert tile
  const int e0 = 32 * n;
  const bool tile_on = e0 < E;
  const int nchunks = H / 32;
  const int64_t ws = plane_bytes(E, H);
  const int8_t *bp = pw + (int64_t)n * nchunks * 1024 + lane * 16;
  v16i_t acc[5];
#pragma unroll
  for (int q = 0; q < 5; ++q)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[q][r] = 0;

  auto do_slab = [&](const int s0, auto slab_index) __attribute__((always_inline)) {
    constexpr int SI = decltype(slab_index)::value;  // (KEEP: which pieces of the kept rows; a constant register index)
    const int sl = H - s0 < kSlab ? H - s0 : kSlab;  // values of this slab (a multiple of 64)
    // slice: a lane's piece j of a row holds the 8 values [lane * 8 + 512 j, + 8): half of block (lane / 2 + 32 j) of
    // the row's planes; the slab takes the pieces 2 (s0 / 1024) and 2 (s0 / 1024) + 1
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      const int r = RW * wave + i;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int h = s0 + lane * 8 + jj * kWave * 8;
        if (h >= s0 + sl) continue;
        uint4 v;
        if constexpr (KEEP) v = keep[i][SI * 2 + jj];
        else v = *reinterpret_cast<const uint4 *>(rowp[i] + h);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
        uint32_t d[3][2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          int a[3][4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int el = 4 * q + j;
            const float y = ((el & 1) ? bf16hi_to_f32(u[el >> 1]) : bf16lo_to_f32(u[el >> 1])) * to_fixed[i];
            const int Xs = (int)y;  // toward zero
            lost[i] += fabsf(y - (float)Xs);
            a[0][j] = __builtin_amdgcn_sbfe(Xs, 0, 8);
            const int X1 = (Xs - a[0][j]) >> 8;
            a[1][j] = __builtin_amdgcn_sbfe(X1, 0, 8);
            a[2][j] = (X1 - a[1][j]) >> 8;
          }
#pragma unroll
          for (int p = 0; p < 3; ++p) d[p][q] = pack4(a[p][0], a[p][1], a[p][2], a[p][3]);
        }
        const int blk = (lane >> 1) + 32 * jj;
#pragma unroll
        for (int p = 0; p < 3; ++p)
          *reinterpret_cast<uint2 *>(tile_lds + p * kPlaneLds + blk * kPlaneBlock + r * 16 + (lane & 1) * 8) = make_uint2(d[p][0], d[p][1]);
      }
    }
    __syncthreads();
    if (tile_on) {
      const int nch = sl / 32;
      const int c_first = ks * nch / KS, c_last = (ks + 1) * nch / KS;
      const int8_t *bslab = bp + (int64_t)(s0 / 32) * 1024;
      struct BChunk {
        v4i_t b[3];
      };
      auto fetch = [&](int c, BChunk &R) __attribute__((always_inline)) {
        int cc = c < nch ? c : nch - 1;
        asm volatile("" : "+s"(cc));
#pragma unroll
        for (int p = 0; p < 3; ++p) R.b[p] = *reinterpret_cast<const v4i_t *>(bslab + p * ws + (int64_t)cc * 1024);
      };
      auto multiply = [&](int c, const BChunk &R) __attribute__((always_inline)) {
        v4i_t a[3];
#pragma unroll
        for (int p = 0; p < 3; ++p)
          a[p] = *reinterpret_cast<const v4i_t *>(tile_lds + p * kPlaneLds + (2 * c + kh) * kPlaneBlock + ln * 16);
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int l = 0; l < 3; ++l) acc[j + l] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[j], R.b[l], acc[j + l], 0, 0, 0);
      };
      constexpr int D = NW > 8 ? 2 : 4;  // (sixteen waves: 128 registers each)
      BChunk ring[D];
#pragma unroll
      for (int dd = 0; dd < D - 1; ++dd) fetch(c_first + dd, ring[dd]);
      int c = c_first;
      for (; c + D <= c_last; c += D) {
#pragma unroll
        for (int dd = 0; dd < D; ++dd) {
          fetch(c + dd + D - 1, ring[(dd + D - 1) % D]);
          __builtin_amdgcn_sched_barrier(0);
          multiply(c + dd, ring[dd]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int dd = 0; dd < D - 1; ++dd)
        if (c + dd < c_last) multiply(c + dd, ring[dd]);
    }
    __syncthreads();  // the planes are rewritten by the next slab (or reused below)
  };
  if constexpr (KEEP) {  // H <= 2048: at most two slabs
    do_slab(0, std::integral_constant<int, 0>{});
    if (H > kSlab) do_slab(kSlab, std::integral_constant<int, 1>{});
  } else {
    for (int s0 = 0; s0 < H; s0 += kSlab) do_slab(s0, std::integral_constant<int, 0>{});
  }
  // what the wave's rows lost to truncation (a row is sliced by one wave)
#pragma unroll
  for (int i = 0; i < RW; ++i) {
    const float ls = (float)wave_sum_f64((double)lost[i]);
    if (lane == 0) meta[RW * wave + i].rsum = ls;
  }

  // ---- 3. partial tiles -> logits
  int64_t(*const sred)[16][64] = reinterpret_cast<int64_t(*)[16][64]>(tile_lds);             // [wave][register][lane]
  uint16_t(*const lg)[128] = reinterpret_cast<uint16_t(*)[128]>(tile_lds + NW * 8192);        // [token row][expert], 8 KiB
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int64_t S = 0;
#pragma unroll
    for (int q = 4; q >= 0; --q) S = S * 256 + (int64_t)acc[q][r];
    sred[wave][r][lane] = S;
  }
  __syncthreads();
  {
    const int e = e0 + ln;
    const RowMeta we = mw[e < E ? e : E - 1];
    const float be = bias && e < E ? bias[e] : 0.f;
    uint16_t out[FR];
    uint32_t redo = 0;
#pragma unroll
    for (int i = 0; i < FR; ++i) {
      const int r = FR * ks + i;
      const int row = 8 * (r >> 2) + 4 * kh + (r & 3);
      const int64_t t = t0 + row;
      const TokenMeta xt = meta[row];
      const float x_rsum = xt.rsum * 1.0001f * __uint_as_float((uint32_t)(xt.unit_exp + 127) << 23);  // in the row's own unit
      int64_t S = 0;
#pragma unroll
      for (int q = 0; q < KS; ++q) S += sred[4 * q + n][r][lane];
      double v = ldexp((double)S, xt.unit_exp + we.unit_exp);
      if (bias) v += (double)be;
      const float f = (float)v;
      const uint32_t u = __float_as_uint(f);
      out[i] = f32_to_bf16(f);
      const int dist = abs((int)(u & 0xffffu) - 0x8000);
      const uint32_t ef = (u >> 23) & 0xffu;
      const float ulp = __uint_as_float((ef > 24u ? ef - 23u : 1u) << 23);
      const float delta = 2.f * x_rsum * we.absmax + we.rsum * xt.absmax + 3.64e-12f * (float)H * xt.absmax * we.absmax;
      bool safe = ef > 24u && ef != 255u && (float)dist * ulp > delta * 1.0001f + 2.5f * ulp;
      if (xt.absmax == 0.f || we.absmax == 0.f) safe = true;
      safe = safe && !xt.nonfinite && !we.nonfinite;
      if (!safe && tile_on && t < T && e < E) redo |= 1u << i;
    }
#pragma unroll
    for (int i = 0; i < FR; ++i) {
      const int r = FR * ks + i;
      uint64_t todo = __ballot((redo >> i) & 1u);
      while (todo) {  // (wave-uniform)
        const int srcl = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int64_t t = t0 + 8 * (r >> 2) + 4 * (srcl >> 5) + (r & 3);
        const int ee = e0 + (srcl & 31);
        double sfix = logit_wave(x + t * H, wg + (int64_t)ee * H, H);
        if (bias) sfix += (double)bias[ee];
        if (lane == srcl) out[i] = f32_to_bf16((float)sfix);
      }
    }
#pragma unroll
    for (int i = 0; i < FR; ++i) {
      const int r = FR * ks + i;
      const int row = 8 * (r >> 2) + 4 * kh + (r & 3);
      lg[row][e0 + ln] = out[i];
      if (tile_on && e < E && t0 + row < T) logits[(t0 + row) * E + e] = out[i];
    }
  }
  __syncthreads();

  // ---- 4. selection: lane l holds experts l and l + 64 of its token
  // (the wave's tokens side by side: their selections are independent chains of wave-wide reductions)
#pragma unroll
  for (int i = 0; i < RW; ++i) {
    const int row = RW * wave + i;
    const int64_t t = t0 + row < T ? t0 + row : T - 1;  // (a row past the batch repeats the last token's: same values stored twice)
    uint16_t bits[2];
    bits[0] = lg[t0 + row < T ? row : (int)(T - 1 - t0)][lane];
    bits[1] = lg[t0 + row < T ? row : (int)(T - 1 - t0)][64 + lane];
    select_from_bits<2, false>(bits, E, k, mode, topk_idx + t * k, topk_w + t * k);
  }
}

bool router_logits_i8_applies(int64_t T, int H, int E) { return T > 64 && H % 64 == 0 && H <= 32768; }

size_t router_logits_i8_bytes(int64_t T, int H, int E) {
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  return up(3 * (size_t)plane_bytes(T, H)) + up(3 * (size_t)plane_bytes(E, H)) + up((size_t)(T + E) * sizeof(RowMeta)) + 256;
}

hipError_t launch_router_logits_i8(const uint16_t *x, const uint16_t *wg, const float *bias, int64_t T, int H, int E,
                                   uint16_t *logits, void *scratch, hipStream_t st, uint16_t *x_paired) {
  if (T == 0) return hipSuccess;
  if (!router_logits_i8_applies(T, H, E)) return hipErrorInvalidValue;
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(scratch) + 255u) & ~(uintptr_t)255u);
  int8_t *px = reinterpret_cast<int8_t *>(base);
  int8_t *pw = reinterpret_cast<int8_t *>(base + up(3 * (size_t)plane_bytes(T, H)));
  RowMeta *mx = reinterpret_cast<RowMeta *>(base + up(3 * (size_t)plane_bytes(T, H)) + up(3 * (size_t)plane_bytes(E, H)));
  RowMeta *mw = mx + T;
  const unsigned sgrid = (unsigned)((T + E + 3) / 4);
  if (H <= 512) router_slice_kernel<1><<<sgrid, 256, 0, st>>>(x, T, wg, E, H, px, pw, mx, mw, x_paired);
  else if (H <= 1024) router_slice_kernel<2><<<sgrid, 256, 0, st>>>(x, T, wg, E, H, px, pw, mx, mw, x_paired);
  else if (H <= 2048) router_slice_kernel<4><<<sgrid, 256, 0, st>>>(x, T, wg, E, H, px, pw, mx, mw, x_paired);
  else if (H <= 4096) router_slice_kernel<8><<<sgrid, 256, 0, st>>>(x, T, wg, E, H, px, pw, mx, mw, x_paired);
  else router_slice_kernel<0><<<sgrid, 256, 0, st>>>(x, T, wg, E, H, px, pw, mx, mw, x_paired);
  dim3 grid((unsigned)((T + 31) / 32), (unsigned)((E + 31) / 32));
  router_i8_kernel<<<grid, 256, 0, st>>>(px, pw, mx, mw, bias, x, wg, T, H, E, logits);
  return hipGetLastError();
}

// logits and selection of T tokens for up to 128 experts in one kernel (after the planes of the router matrix)
bool router_tile_applies(int64_t T, int H, int E, int k) { return router_logits_i8_applies(T, H, E) && E <= 128 && k <= 64; }

hipError_t launch_router_tile(const uint16_t *x, const uint16_t *wg, const float *bias, int64_t T, int H, int E, int k,
                              int mode, uint16_t *logits, uint32_t *topk_idx, uint16_t *topk_w, void *scratch,
                              hipStream_t st, uint16_t *x_paired) {
  if (T == 0) return hipSuccess;
  if (!router_tile_applies(T, H, E, k)) return hipErrorInvalidValue;
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(scratch) + 255u) & ~(uintptr_t)255u);
  // (the same carving as launch_router_logits_i8; the planes of x stay unused)
  int8_t *pw = reinterpret_cast<int8_t *>(base + up(3 * (size_t)plane_bytes(T, H)));
  RowMeta *mx = reinterpret_cast<RowMeta *>(base + up(3 * (size_t)plane_bytes(T, H)) + up(3 * (size_t)plane_bytes(E, H)));
  RowMeta *mw = mx + T;
  const unsigned sgrid = (unsigned)((E + 3) / 4);
  if (H <= 512) router_slice_kernel<1><<<sgrid, 256, 0, st>>>(x, 0, wg, E, H, nullptr, pw, mx, mw, nullptr);
  else if (H <= 1024) router_slice_kernel<2><<<sgrid, 256, 0, st>>>(x, 0, wg, E, H, nullptr, pw, mx, mw, nullptr);
  else if (H <= 2048) router_slice_kernel<4><<<sgrid, 256, 0, st>>>(x, 0, wg, E, H, nullptr, pw, mx, mw, nullptr);
  else if (H <= 4096) router_slice_kernel<8><<<sgrid, 256, 0, st>>>(x, 0, wg, E, H, nullptr, pw, mx, mw, nullptr);
  else router_slice_kernel<0><<<sgrid, 256, 0, st>>>(x, 0, wg, E, H, nullptr, pw, mx, mw, nullptr);
  // more dynamic LDS than a kernel gets without asking: asked for on every launch (the attribute belongs to the
  // current device's copy of the kernel; the call is a table update on the host)
  const unsigned grid = (unsigned)((T + 31) / 32);
#define MI_TILE(NWV, KEEPV)                                                                                              \
  do {                                                                                                                  \
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&router_tile_kernel<NWV, KEEPV>),             \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kTileLds);                      \
        e != hipSuccess)                                                                                                \
      return e;                                                                                                         \
    router_tile_kernel<NWV, KEEPV><<<grid, NWV * 64, kTileLds, st>>>(x, pw, mw, bias, wg, T, H, E, k, mode, logits,      \
                                                                    topk_idx, topk_w, x_paired);                        \
  } while (0)
  if (H <= 2048 && MI_TILE_KEEP) MI_TILE(MI_TILE_WAVES, true);
  else MI_TILE(MI_TILE_WAVES, false);
#undef MI_TILE
  return hipGetLastError();
}

}  // namespace mi_moe
