// Weighted combine back to token order, and the stand-alone SwiGLU elementwise op.
//
// combine replaces take(inv_order) + unflatten + squeeze + multiply(scores) + sum_axis(-2)
// (mlx-rs/src/ops/indexing/mod.rs:386-401, ops/shapes.rs:398-415,466-484,
// ops/arithmetic.rs:138-160, ops/reduction.rs:260-276): every output element is one
// thread's fp32 sum over the k slots in slot order: no atomics, run-to-run identical.
#include "router_dev.hpp"

namespace mi_moe {

__global__ __launch_bounds__(256) void combine_kernel(
    const uint16_t *__restrict__ y, const uint16_t *__restrict__ scores,
    const uint32_t *__restrict__ inv_perm, int64_t T, int k, int H,
    const uint16_t *__restrict__ residual, uint16_t *__restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (h >= H) return;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < k; ++s) {
    const int64_t r = inv_perm ? (int64_t)inv_perm[t * k + s] : t * k + s;
    const float sc = bf16_to_f32(scores[t * k + s]);
    const uint4 v = *reinterpret_cast<const uint4 *>(y + r * H + h);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[2 * i] += sc * bf16lo_to_f32(u[i]);
      acc[2 * i + 1] += sc * bf16hi_to_f32(u[i]);
    }
  }
  if (residual) {  // h + mlp(...): the block's neighbour in a decoder layer, added before the one rounding
    const uint4 v = *reinterpret_cast<const uint4 *>(residual + t * H + h);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[2 * i] = bf16lo_to_f32(u[i]) + acc[2 * i];
      acc[2 * i + 1] = bf16hi_to_f32(u[i]) + acc[2 * i + 1];
    }
  }
  uint4 o;
  o.x = pack_bf16x2(acc[0], acc[1]);
  o.y = pack_bf16x2(acc[2], acc[3]);
  o.z = pack_bf16x2(acc[4], acc[5]);
  o.w = pack_bf16x2(acc[6], acc[7]);
  *reinterpret_cast<uint4 *>(out + t * H + h) = o;
}

hipError_t launch_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                          int64_t T, int k, int H, const uint16_t *residual, uint16_t *out,
                          hipStream_t st) {
  if (T == 0) return hipSuccess;
  dim3 grid((unsigned)T, (unsigned)((H / 8 + 255) / 256));
  combine_kernel<<<grid, 256, 0, st>>>(y, scores, inv_perm, T, k, H, residual, out);
  return hipGetLastError();
}

// RMS normalisation over the last axis (mlx_fast_rms_norm, mlx-rs/src/fast.rs:190-207;
// nn::RmsNorm, mlx-rs/src/nn/normalization.rs:233-275): one wave per row.  The mean of squares is
// accumulated in double over exact products (any order gives the same float), 1 / sqrt in
// correctly rounded float operations, one rounding to bf16: the bits of the host-side checker,
// which the selection of experts downstream depends on.
__global__ __launch_bounds__(256) void rms_norm_kernel(const uint16_t *__restrict__ x,
                                                       const uint16_t *__restrict__ weight, float eps,
                                                       int64_t T, int H, uint16_t *__restrict__ out) {
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const uint16_t *xr = x + t * H;
  const float rstd = row_rstd_wave(xr, H, eps);
  for (int h = lane_id() * 8; h < H; h += kWave * 8)
    *reinterpret_cast<uint4 *>(out + t * H + h) =
        rms_norm8(*reinterpret_cast<const uint4 *>(xr + h), *reinterpret_cast<const uint4 *>(weight + h), rstd);
}

hipError_t launch_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T, int H,
                           uint16_t *out, hipStream_t st) {
  if (T == 0) return hipSuccess;
  rms_norm_kernel<<<(unsigned)((T + 3) / 4), 256, 0, st>>>(x, weight, eps, T, H, out);
  return hipGetLastError();
}

// silu(gate) * up on bf16 arrays, one rounding at the end
// (mlx-rs/src/nn/activation.rs:142-144,876-880 followed by multiply).
__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t *__restrict__ g,
                                                     const uint16_t *__restrict__ u, int64_t n,
                                                     uint16_t *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float gv = bf16_to_f32(g[i]), uv = bf16_to_f32(u[i]);
  out[i] = f32_to_bf16(gv / (1.0f + __expf(-gv)) * uv);
}

hipError_t launch_swiglu(const uint16_t *g, const uint16_t *u, int64_t n, uint16_t *out,
                         hipStream_t st) {
  if (n == 0) return hipSuccess;
  swiglu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(g, u, n, out);
  return hipGetLastError();
}

}  // namespace mi_moe
