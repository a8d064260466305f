// MLX-affine quantize / dequantize of a [rows, cols] fp32 matrix
// (mlx_quantize / mlx_dequantize, mlx-rs/src/ops/quantization.rs:50-83,124-158; format
// statement :31-47,85-87; shapes pinned by the reference test :298-315).
//
// One thread produces one packed uint32 word; the lanes that share a quantisation group
// (group_size / (32/bits) of them, a power of two <= 64) find the group's min and max with
// xor-shuffles.  Every step is a correctly rounded fp32 operation in the same order as
// the host-side checker, so codes, scales and biases agree with it bit for bit.
#include "common.hpp"

namespace mi_moe {

// Element types of activations, scales and biases (mi_moe_dtype of the C ABI).  fp16 goes through the
// hardware's round-to-nearest-even conversion, bf16 through the integer rounding every other kernel
// here uses.
template <class T> struct Elem;
template <> struct Elem<uint16_t> {  // bfloat16, raw bits
  static __device__ __forceinline__ float load(const uint16_t *p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(uint16_t *p, float v) { *p = f32_to_bf16(v); }
};
template <> struct Elem<_Float16> {
  static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
  static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float *p) { return *p; }
  static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};

template <class T>
__global__ __launch_bounds__(256) void quantize_kernel(const float *__restrict__ w, int64_t n_words,
                                                       int group, int bits,
                                                       uint32_t *__restrict__ q,
                                                       T *__restrict__ scales,
                                                       T *__restrict__ biases) {
#pragma clang fp contract(off)
  const int per_word = 32 / bits;
  const int lanes_per_group = group / per_word;
  const int64_t wi = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool on = wi < n_words;
  const int64_t wl = on ? wi : n_words - 1;  // keep every lane in the shuffles
  float v[16];
  float w_min = INFINITY, w_max = -INFINITY;
  for (int j = 0; j < per_word; ++j) {
    v[j] = w[wl * per_word + j];
    w_min = fminf(w_min, v[j]);
    w_max = fmaxf(w_max, v[j]);
  }
  for (int m = 1; m < lanes_per_group; m <<= 1) {
    w_min = fminf(w_min, __shfl_xor(w_min, m, kWave));
    w_max = fmaxf(w_max, __shfl_xor(w_max, m, kWave));
  }
  const float n_bins = (float)((1 << bits) - 1);
  const bool mask = fabsf(w_min) > fabsf(w_max);
  float scale = fmaxf((w_max - w_min) / n_bins, 1e-7f);
  scale = mask ? scale : -scale;
  const float edge = mask ? w_min : w_max;
  const float q0 = __builtin_rintf(edge / scale);
  float bias = 0.0f;
  if (q0 != 0.0f) {
    scale = edge / q0;
    bias = edge;
  }
  uint32_t word = 0;
  for (int j = 0; j < per_word; ++j) {
    float c = __builtin_rintf((v[j] - bias) / scale);
    c = fminf(fmaxf(c, 0.0f), n_bins);
    word |= (uint32_t)c << (j * bits);
  }
  if (on) {
    q[wi] = word;
    if (wi % lanes_per_group == 0) {  // the codes come from the fp32 scale and bias; these are cast afterwards
      Elem<T>::store(scales + wi / lanes_per_group, scale);
      Elem<T>::store(biases + wi / lanes_per_group, bias);
    }
  }
}

// O: element type of the result (float, or the type of scales and biases: what mlx_dequantize returns)
template <class T, class O>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t *__restrict__ q,
                                                         const T *__restrict__ scales,
                                                         const T *__restrict__ biases,
                                                         int64_t n_words, int group, int bits,
                                                         O *__restrict__ out) {
#pragma clang fp contract(off)
  const int per_word = 32 / bits;
  const int64_t wi = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (wi >= n_words) return;
  const int64_t g = wi * per_word / group;
  const float s = Elem<T>::load(scales + g), b = Elem<T>::load(biases + g);
  uint32_t word = q[wi];
  const uint32_t m = (1u << bits) - 1u;
  for (int j = 0; j < per_word; ++j) {
    Elem<O>::store(out + wi * per_word + j, s * (float)(word & m) + b);  // two fp32 roundings (contraction is off), then O's
    word >>= bits;
  }
}

// dt: 0 bf16, 1 fp16, 2 fp32 (mi_moe_dtype)
hipError_t launch_quantize(const float *w, int64_t rows, int64_t cols, int group, int bits,
                           uint32_t *q, void *s, void *b, int dt, hipStream_t st) {
  const int64_t n_words = rows * cols * bits / 32;
  if (n_words == 0) return hipSuccess;
  const unsigned grid = (unsigned)((n_words + 255) / 256);
  if (dt == 0) quantize_kernel<uint16_t><<<grid, 256, 0, st>>>(w, n_words, group, bits, q, (uint16_t *)s, (uint16_t *)b);
  else if (dt == 1) quantize_kernel<_Float16><<<grid, 256, 0, st>>>(w, n_words, group, bits, q, (_Float16 *)s, (_Float16 *)b);
  else quantize_kernel<float><<<grid, 256, 0, st>>>(w, n_words, group, bits, q, (float *)s, (float *)b);
  return hipGetLastError();
}

// native_out: the result has the element type of scales and biases (dt); otherwise float
hipError_t launch_dequantize(const uint32_t *q, const void *s, const void *b,
                             int64_t rows, int64_t cols, int group, int bits, void *out, int dt, bool native_out,
                             hipStream_t st) {
  const int64_t n_words = rows * cols * bits / 32;
  if (n_words == 0) return hipSuccess;
  const unsigned grid = (unsigned)((n_words + 255) / 256);
  if (dt == 0 && native_out) dequantize_kernel<uint16_t, uint16_t><<<grid, 256, 0, st>>>(q, (const uint16_t *)s, (const uint16_t *)b, n_words, group, bits, (uint16_t *)out);
  else if (dt == 0) dequantize_kernel<uint16_t, float><<<grid, 256, 0, st>>>(q, (const uint16_t *)s, (const uint16_t *)b, n_words, group, bits, (float *)out);
  else if (dt == 1 && native_out) dequantize_kernel<_Float16, _Float16><<<grid, 256, 0, st>>>(q, (const _Float16 *)s, (const _Float16 *)b, n_words, group, bits, (_Float16 *)out);
  else if (dt == 1) dequantize_kernel<_Float16, float><<<grid, 256, 0, st>>>(q, (const _Float16 *)s, (const _Float16 *)b, n_words, group, bits, (float *)out);
  else dequantize_kernel<float, float><<<grid, 256, 0, st>>>(q, (const float *)s, (const float *)b, n_words, group, bits, (float *)out);
  return hipGetLastError();
}

// y[m][n] += bias[n], one rounding to T: the add that follows the product in a linear layer with a bias
// (mlx-rs/src/nn/quantized.rs:363-386: quantized_matmul, then add, each rounded to the element type)
template <class T>
__global__ __launch_bounds__(256) void add_row_bias_kernel(T *__restrict__ y, const T *__restrict__ bias, int64_t n, int N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  Elem<T>::store(y + i, Elem<T>::load(y + i) + Elem<T>::load(bias + i % N));
}

hipError_t launch_add_row_bias(void *y, const void *bias, int64_t M, int N, int dt, hipStream_t st) {
  const int64_t n = M * N;
  if (n == 0) return hipSuccess;
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (dt == 0) add_row_bias_kernel<uint16_t><<<grid, 256, 0, st>>>((uint16_t *)y, (const uint16_t *)bias, n, N);
  else if (dt == 1) add_row_bias_kernel<_Float16><<<grid, 256, 0, st>>>((_Float16 *)y, (const _Float16 *)bias, n, N);
  else add_row_bias_kernel<float><<<grid, 256, 0, st>>>((float *)y, (const float *)bias, n, N);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Plain quantized products: every combination the tuned kernels do not take -- activations, scales
// and biases in fp32 or fp16 (mlx_quantized_matmul and mlx_gather_qmm accept any floating type; the
// reference's own tests run them in fp32, mlx-rs/src/ops/quantization.rs:318-423), group sizes 32 and
// 128, 2-bit codes, and the untransposed weight layout (transpose = false, the default of
// ops::quantized_matmul, :91-122).  Correct and simple, not tuned: fp32 accumulation, weights
// dequantised as fma(scale, q, bias) in fp32, one rounding to the output type.
//
// Output row r = j * M + m (j: index pair, m: row of the M x K matrix):
//   expert e = rhs[rhs_map ? rhs_map[j] : j] (0 without rhs), x row = (lhs ? lhs[j] : j) * M + m,
//   destination row = dst_map ? dst_map[r] : r.
struct PlainMaps {
  const uint32_t *lhs, *rhs, *rhs_map, *dst_map;
  uint32_t n_lhs, n_rhs;  // matrices behind lhs / rhs (0 = unknown): indices beyond are clamped, never followed
};

__device__ __forceinline__ int64_t clamped_index(uint32_t v, uint32_t n) { return n && v >= n ? n - 1u : v; }

// transpose = true: w [E, N, K*bits/32], scales / biases [E, N, K/group].  One wave per output
// element, lanes over the packed words of the weight row, sum over the lanes in a fixed order.
template <class T, int BITS>
__global__ __launch_bounds__(256) void qmm_plain_t_kernel(const T *__restrict__ x, const uint32_t *__restrict__ w,
                                                          const T *__restrict__ scales, const T *__restrict__ biases,
                                                          PlainMaps mp, int M, int N, int K, int group,
                                                          T *__restrict__ y) {
  constexpr int CPW = 32 / BITS;
  const int64_t r = blockIdx.x;
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const int lane = lane_id();
  const int64_t j = r / M;
  const int m = (int)(r % M);
  const int64_t e = mp.rhs ? clamped_index(mp.rhs[mp.rhs_map ? mp.rhs_map[j] : j], mp.n_rhs) : 0;
  const int64_t xb = mp.lhs ? clamped_index(mp.lhs[j], mp.n_lhs) : j;
  const T *xr = x + (xb * M + m) * K;
  const int wpr = K / CPW, gpr = K / group;
  const uint32_t *wp = w + (e * N + n) * wpr;
  const T *sp = scales + (e * N + n) * gpr, *bp = biases + (e * N + n) * gpr;
  float acc = 0.f;
  for (int wi = lane; wi < wpr; wi += kWave) {
    const uint32_t word = wp[wi];
    const int k0 = wi * CPW;
    const float sc = Elem<T>::load(sp + k0 / group), bi = Elem<T>::load(bp + k0 / group);  // a word never straddles groups
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const float qv = (float)((word >> (c * BITS)) & ((1u << BITS) - 1u));
      acc = __builtin_fmaf(Elem<T>::load(xr + k0 + c), __builtin_fmaf(sc, qv, bi), acc);
    }
  }
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) acc += __shfl_xor(acc, d, kWave);
  const int64_t dr = mp.dst_map ? (int64_t)mp.dst_map[r] : r;
  if (lane == 0) Elem<T>::store(y + dr * N + n, acc);
}

// transpose = false: w [E, K, N*bits/32], scales / biases [E, K, N/group] (K x N matrices quantised
// along N).  One thread per packed word of an output row, fp32 accumulation in k order.
template <class T, int BITS>
__global__ __launch_bounds__(256) void qmm_plain_n_kernel(const T *__restrict__ x, const uint32_t *__restrict__ w,
                                                          const T *__restrict__ scales, const T *__restrict__ biases,
                                                          PlainMaps mp, int M, int N, int K, int group,
                                                          T *__restrict__ y) {
  constexpr int CPW = 32 / BITS;  // codes per word
  const int64_t r = blockIdx.x;   // output row = j * M + m
  const int wi = blockIdx.y * 256 + threadIdx.x;
  const int wpr = N / CPW;
  if (wi >= wpr) return;
  const int64_t j = r / M;
  const int m = (int)(r % M);
  const int64_t e = mp.rhs ? clamped_index(mp.rhs[mp.rhs_map ? mp.rhs_map[j] : j], mp.n_rhs) : 0;
  const int64_t xb = mp.lhs ? clamped_index(mp.lhs[j], mp.n_lhs) : j;
  const T *xr = x + (xb * M + m) * K;
  const int gpr = N / group, g = wi * CPW / group;
  const uint32_t *wp = w + e * K * wpr + wi;
  const T *sp = scales + e * K * gpr + g, *bp = biases + e * K * gpr + g;
  float acc[CPW];
#pragma unroll
  for (int c = 0; c < CPW; ++c) acc[c] = 0.f;
  for (int k = 0; k < K; ++k) {
    const uint32_t word = wp[(int64_t)k * wpr];
    const float sc = Elem<T>::load(sp + (int64_t)k * gpr), bi = Elem<T>::load(bp + (int64_t)k * gpr);
    const float xv = Elem<T>::load(xr + k);
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const float qv = (float)((word >> (c * BITS)) & ((1u << BITS) - 1u));
      acc[c] = __builtin_fmaf(xv, __builtin_fmaf(sc, qv, bi), acc[c]);
    }
  }
  const int64_t dr = mp.dst_map ? (int64_t)mp.dst_map[r] : r;
  T *yo = y + dr * N + (int64_t)wi * CPW;
#pragma unroll
  for (int c = 0; c < CPW; ++c) Elem<T>::store(yo + c, acc[c]);
}

template <class T>
static hipError_t launch_plain_t(const void *x, const uint32_t *w, const void *s, const void *b, const PlainMaps &mp,
                                 int64_t rows, int M, int N, int K, int group, int bits, void *y, bool transpose,
                                 hipStream_t st) {
  const T *xs = static_cast<const T *>(x), *ss = static_cast<const T *>(s), *bs = static_cast<const T *>(b);
  T *ys = static_cast<T *>(y);
  if (transpose) {
    dim3 grid((unsigned)rows, (unsigned)((N + 3) / 4));
    if (bits == 2) qmm_plain_t_kernel<T, 2><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
    else if (bits == 4) qmm_plain_t_kernel<T, 4><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
    else qmm_plain_t_kernel<T, 8><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
  } else {
    const int wpr = N * bits / 32;
    dim3 grid((unsigned)rows, (unsigned)((wpr + 255) / 256));
    if (bits == 2) qmm_plain_n_kernel<T, 2><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
    else if (bits == 4) qmm_plain_n_kernel<T, 4><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
    else qmm_plain_n_kernel<T, 8><<<grid, 256, 0, st>>>(xs, w, ss, bs, mp, M, N, K, group, ys);
  }
  return hipGetLastError();
}

// dt: 0 bf16, 1 fp16, 2 fp32.  rows = n_idx * M output rows (at most 2^31 - 1: they are the grid's x extent).
hipError_t launch_qmm_plain(const void *x, const uint32_t *w, const void *scales, const void *biases,
                            const uint32_t *lhs, const uint32_t *rhs, const uint32_t *rhs_map,
                            const uint32_t *dst_map, uint32_t n_lhs, uint32_t n_rhs, int64_t rows, int M, int N,
                            int K, int group, int bits, bool transpose, int dt, void *y, hipStream_t st) {
  if (rows == 0) return hipSuccess;
  if (transpose && (N + 3) / 4 > 65535) return hipErrorInvalidValue;  // the grid's y extent
  const PlainMaps mp{lhs, rhs, rhs_map, dst_map, n_lhs, n_rhs};
  if (dt == 0) return launch_plain_t<uint16_t>(x, w, scales, biases, mp, rows, M, N, K, group, bits, y, transpose, st);
  if (dt == 1) return launch_plain_t<_Float16>(x, w, scales, biases, mp, rows, M, N, K, group, bits, y, transpose, st);
  return launch_plain_t<float>(x, w, scales, biases, mp, rows, M, N, K, group, bits, y, transpose, st);
}

}  // namespace mi_moe
