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

__global__ __launch_bounds__(256) void quantize_kernel(const float *__restrict__ w, int64_t n_words,
                                                       int group, int bits,
                                                       uint32_t *__restrict__ q,
                                                       uint16_t *__restrict__ scales,
                                                       uint16_t *__restrict__ biases) {
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
    if (wi % lanes_per_group == 0) {
      scales[wi / lanes_per_group] = f32_to_bf16(scale);
      biases[wi / lanes_per_group] = f32_to_bf16(bias);
    }
  }
}

__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t *__restrict__ q,
                                                         const uint16_t *__restrict__ scales,
                                                         const uint16_t *__restrict__ biases,
                                                         int64_t n_words, int group, int bits,
                                                         float *__restrict__ out) {
#pragma clang fp contract(off)
  const int per_word = 32 / bits;
  const int64_t wi = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (wi >= n_words) return;
  const int64_t g = wi * per_word / group;
  const float s = bf16_to_f32(scales[g]), b = bf16_to_f32(biases[g]);
  uint32_t word = q[wi];
  const uint32_t m = (1u << bits) - 1u;
  for (int j = 0; j < per_word; ++j) {
    out[wi * per_word + j] = s * (float)(word & m) + b;  // two roundings (contraction is off)
    word >>= bits;
  }
}

hipError_t launch_quantize(const float *w, int64_t rows, int64_t cols, int group, int bits,
                           uint32_t *q, uint16_t *s, uint16_t *b, hipStream_t st) {
  const int64_t n_words = rows * cols * bits / 32;
  if (n_words == 0) return hipSuccess;
  quantize_kernel<<<(unsigned)((n_words + 255) / 256), 256, 0, st>>>(w, n_words, group, bits, q, s, b);
  return hipGetLastError();
}

hipError_t launch_dequantize(const uint32_t *q, const uint16_t *s, const uint16_t *b,
                             int64_t rows, int64_t cols, int group, int bits, float *out,
                             hipStream_t st) {
  const int64_t n_words = rows * cols * bits / 32;
  if (n_words == 0) return hipSuccess;
  dequantize_kernel<<<(unsigned)((n_words + 255) / 256), 256, 0, st>>>(q, s, b, n_words, group, bits, out);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Quantized product with an UNTRANSPOSED weight (transpose = false, the default of
// ops::quantized_matmul, mlx-rs/src/ops/quantization.rs:91-122, and the layout of the reference's
// test_quantized_matmul, :318-342): w holds K x N matrices quantised along N,
//   w [E, K, N*bits/32], scales / biases [E, K, N/group];  y[r] (N) = x[src(r)] (K) . W_hat[e(r)].
// Not a layout any mlx-lm switch layer uses: a plain, correct kernel (one thread per packed word
// of an output row, fp32 accumulation in k order), not a tuned one.
template <int BITS>
__global__ __launch_bounds__(256) void qmm_nt_kernel(const uint16_t *__restrict__ x,
                                                     const uint32_t *__restrict__ w,
                                                     const uint16_t *__restrict__ scales,
                                                     const uint16_t *__restrict__ biases,
                                                     const uint32_t *__restrict__ lhs,
                                                     const uint32_t *__restrict__ rhs, int M, int N, int K,
                                                     int group, uint16_t *__restrict__ y) {
  constexpr int CPW = 32 / BITS;  // codes per word
  const int64_t r = blockIdx.x;   // output row = j * M + m
  const int wi = blockIdx.y * 256 + threadIdx.x;
  const int wpr = N / CPW;
  if (wi >= wpr) return;
  const int64_t j = r / M;
  const int m = (int)(r % M);
  const int64_t e = rhs ? (int64_t)rhs[j] : 0;
  const int64_t xb = lhs ? (int64_t)lhs[j] : j;
  const uint16_t *xr = x + (xb * M + m) * K;
  const int gpr = N / group, g = wi * CPW / group;
  const uint32_t *wp = w + e * K * wpr + wi;
  const uint16_t *sp = scales + e * K * gpr + g, *bp = biases + e * K * gpr + g;
  float acc[CPW];
#pragma unroll
  for (int c = 0; c < CPW; ++c) acc[c] = 0.f;
  for (int k = 0; k < K; ++k) {
    const uint32_t word = wp[(int64_t)k * wpr];
    const float sc = bf16_to_f32(sp[(int64_t)k * gpr]), bi = bf16_to_f32(bp[(int64_t)k * gpr]);
    const float xv = bf16_to_f32(xr[k]);
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const float qv = (float)((word >> (c * BITS)) & ((1u << BITS) - 1u));
      acc[c] = __builtin_fmaf(xv, __builtin_fmaf(sc, qv, bi), acc[c]);
    }
  }
  uint16_t *yo = y + r * N + (int64_t)wi * CPW;
#pragma unroll
  for (int c = 0; c < CPW; c += 2)
    *reinterpret_cast<uint32_t *>(yo + c) = pack_bf16x2(acc[c], acc[c + 1]);
}

hipError_t launch_qmm_nt(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                         const uint16_t *biases, const uint32_t *lhs, const uint32_t *rhs, int64_t rows,
                         int M, int N, int K, int group, int bits, uint16_t *y, hipStream_t st) {
  if (rows == 0) return hipSuccess;
  const int wpr = N * bits / 32;
  dim3 grid((unsigned)rows, (unsigned)((wpr + 255) / 256));
  if (bits == 4) qmm_nt_kernel<4><<<grid, 256, 0, st>>>(x, w, scales, biases, lhs, rhs, M, N, K, group, y);
  else qmm_nt_kernel<8><<<grid, 256, 0, st>>>(x, w, scales, biases, lhs, rhs, M, N, K, group, y);
  return hipGetLastError();
}

}  // namespace mi_moe
