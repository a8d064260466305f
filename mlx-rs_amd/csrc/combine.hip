// Weighted combine back to token order, and the stand-alone SwiGLU elementwise op.
//
// combine replaces take(inv_order) + unflatten + squeeze + multiply(scores) + sum_axis(-2)
// (mlx-rs/src/ops/indexing/mod.rs:386-401, ops/shapes.rs:398-415,466-484,
// ops/arithmetic.rs:138-160, ops/reduction.rs:260-276): every output element is one
// thread's fp32 sum over the k slots in slot order: no atomics, run-to-run identical.
#include "router_dev.hpp"

namespace mi_moe {

// One thread per 8 output columns, kCombineThreads threads per block (a token's row is spread over
// several blocks: at decode sizes the launch is latency, and a block per token would leave most of
// the chip idle).  The k rows of a token are fetched eight at a time, all loads of a batch in flight
// before the first is used; the sum itself runs in slot order.
constexpr int kCombineThreads = 64;
__global__ __launch_bounds__(kCombineThreads) void combine_kernel(
    const uint16_t *__restrict__ y, const uint16_t *__restrict__ scores,
    const uint32_t *__restrict__ inv_perm, int64_t T, int k, int H,
    const uint16_t *__restrict__ residual, uint16_t *__restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = (blockIdx.y * kCombineThreads + threadIdx.x) * 8;
  if (h >= H) return;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < k; s0 += 8) {
    uint4 v[8];
    float sc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < k ? s0 + j : k - 1;  // (clamped: loads without a condition stay in flight together)
      const int64_t r = inv_perm ? (int64_t)inv_perm[t * k + s] : t * k + s;
      sc[j] = bf16_to_f32(scores[t * k + s]);
      v[j] = *reinterpret_cast<const uint4 *>(y + r * H + h);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (s0 + j < k) {
        const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[2 * i] += sc[j] * bf16lo_to_f32(u[i]);
          acc[2 * i + 1] += sc[j] * bf16hi_to_f32(u[i]);
        }
      }
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
  dim3 grid((unsigned)T, (unsigned)((H / 8 + kCombineThreads - 1) / kCombineThreads));
  combine_kernel<<<grid, kCombineThreads, 0, st>>>(y, scores, inv_perm, T, k, H, residual, out);
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

// Bare streaming kernel with the decode grouped product's access shape: a wave reads a 16 KiB tile
// (16 rows of 1 KiB) from each of two arrays, 64 bytes per row and instruction, four pieces of
// each in flight, and does nothing with them.  What a launch of a given size can pull from HBM.
__global__ __launch_bounds__(256) void stream_probe_kernel(const uint32_t *__restrict__ p0,
                                                           const uint32_t *__restrict__ p1,
                                                           size_t n_tiles, uint32_t *sink) {
  typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
  extern __shared__ unsigned char probe_lds[];
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wave >= n_tiles) return;
  const uint32_t voff = (lane & 15) * 1024 + (lane >> 4) * 16;
  __amdgpu_buffer_rsrc_t r0 = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p0 + wave * 4096), 0, 16384, 0x00020000);
  __amdgpu_buffer_rsrc_t r1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p1 + wave * 4096), 0, 16384, 0x00020000);
  constexpr int D = 4;
  u32x4_t ring[D][2];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    ring[d][0] = __builtin_amdgcn_raw_buffer_load_b128(r0, voff, d * 64, 0);
    ring[d][1] = __builtin_amdgcn_raw_buffer_load_b128(r1, voff, d * 64, 0);
  }
  uint32_t acc = 0;
  for (int base = 0; base < 16; base += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const u32x4_t a = ring[d][0], b = ring[d][1];
      acc += a[0] ^ a[1] ^ a[2] ^ a[3] ^ b[0] ^ b[1] ^ b[2] ^ b[3];
      if (base + d + D < 16) {
        ring[d][0] = __builtin_amdgcn_raw_buffer_load_b128(r0, voff, (base + d + D) * 64, 0);
        ring[d][1] = __builtin_amdgcn_raw_buffer_load_b128(r1, voff, (base + d + D) * 64, 0);
      }
    }
  }
  if (acc == 0x12345678u) sink[0] = acc + probe_lds[0];  // keeps the loads alive; the buffer never holds such data
}

hipError_t launch_stream_probe(const void *buf, size_t bytes, uint32_t *sink, hipStream_t st) {
  const size_t n_tiles = bytes / 32768;
  if (n_tiles == 0) return hipSuccess;
  const uint32_t *p0 = static_cast<const uint32_t *>(buf);
  // 38000 bytes of LDS: four blocks per CU, as the product kernel at decode
  stream_probe_kernel<<<(unsigned)((n_tiles + 3) / 4), 256, 38000, st>>>(p0, p0 + bytes / 8, n_tiles, sink);
  return hipGetLastError();
}

}  // namespace mi_moe
