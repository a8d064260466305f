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

}  // namespace mi_moe
