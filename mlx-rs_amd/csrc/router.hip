// Router: gate Linear -> softmax(precise) -> top-k -> scores.
//
// Replaces, for one MoE layer, the MLX primitives a Module would call through
// mlx-rs: ops::matmul via nn::Linear (mlx-rs/src/nn/linear.rs:84-96,
// ops/arithmetic.rs:577-603), ops::softmax_axis(precise) (ops/arithmetic.rs:1291-1327),
// ops::argpartition_axis + slice (ops/sort.rs:211-260), take_along_axis
// (ops/indexing/mod.rs:433-453), sum_axis + divide (ops/reduction.rs:260-276).
//
// Selection must be reproducible bit for bit, so every value the selection depends on
// is computed in a way that does not depend on summation order:
//   logits  - fp64 accumulation of exact bf16*bf16 products, rounded fp64->fp32->bf16;
//   softmax - det_expf terms, fp64 sum, one IEEE fp32 division, rounded to bf16;
//   top-k   - total order (value descending, expert id ascending), slot 0 = best.
#include "router_dev.hpp"

namespace mi_moe {

// ------------------------------------------------------------------ logits
// One wave computes a TM x EM tile of logits: lanes split H in 16-byte pieces, fp64
// fused multiply-adds, then a butterfly sum.  A block is 4 waves side by side along E.
template <int TM, int EM>
__global__ __launch_bounds__(256) void router_logits_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ wg,
    const float *__restrict__ bias, int64_t T, int H, int E, uint16_t *__restrict__ logits) {
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * TM;
  const int e0 = (blockIdx.y * 4 + wave) * EM;
  if (e0 >= E) return;

  const uint16_t *xr[TM];
  const uint16_t *wr[EM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int64_t t = t0 + i < T ? t0 + i : T - 1;
    xr[i] = x + t * H;
  }
#pragma unroll
  for (int j = 0; j < EM; ++j) {
    int e = e0 + j < E ? e0 + j : E - 1;
    wr[j] = wg + (int64_t)e * H;
  }
  double acc[TM][EM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < EM; ++j) acc[i][j] = 0.0;

  for (int h = lane * 8; h < H; h += kWave * 8) {
    double xd[TM][8], wd[EM][8];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      uint4 v = *reinterpret_cast<const uint4 *>(xr[i] + h);
      uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        xd[i][2 * q] = (double)bf16lo_to_f32(u[q]);
        xd[i][2 * q + 1] = (double)bf16hi_to_f32(u[q]);
      }
    }
#pragma unroll
    for (int j = 0; j < EM; ++j) {
      uint4 v = *reinterpret_cast<const uint4 *>(wr[j] + h);
      uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        wd[j][2 * q] = (double)bf16lo_to_f32(u[q]);
        wd[j][2 * q + 1] = (double)bf16hi_to_f32(u[q]);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < EM; ++j)
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[i][j] = __builtin_fma(xd[i][q], wd[j][q], acc[i][j]);
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < EM; ++j) {
      double s = wave_sum_f64(acc[i][j]);
      if (lane == 0 && t0 + i < T && e0 + j < E) {
        if (bias) s += (double)bias[e0 + j];
        logits[(t0 + i) * E + e0 + j] = f32_to_bf16((float)s);
      }
    }
}

// Prefill-sized T: the same fp64 accumulation on the matrix cores (v_mfma_f64_16x16x4_f64).
// A block computes a 32-token x 32-expert tile; its 4 waves split H in 32-wide chunks and the
// partial tiles are added in wave order through LDS.  Lane (i = lane & 15, kq = lane >> 4)
// loads 8 consecutive h of row i per chunk; MFMA step s multiplies element s of every lane, so
// the four kq lanes of a row cover 32 consecutive h in 8 steps (any K order gives the same sum).
typedef __attribute__((__vector_size__(4 * sizeof(double)))) double f64x4_t;

// NT: 16-row sub-tiles per side of a block's tile (2: 32 tokens x 32 experts, 1: 16 x 16).
template <int NT>
__global__ __launch_bounds__(256) void router_logits_mfma_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ wg,
    const float *__restrict__ bias, int64_t T, int H, int E, uint16_t *__restrict__ logits,
    uint16_t *__restrict__ x_paired) {
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, kq = lane >> 4;
  const int64_t t0 = (int64_t)blockIdx.x * (16 * NT);
  const int e0 = blockIdx.y * (16 * NT);
  const uint16_t *xr[NT], *wr[NT];
#pragma unroll
  for (int a = 0; a < NT; ++a) {
    const int64_t t = t0 + 16 * a + i;
    const int e = e0 + 16 * a + i;
    xr[a] = x + (t < T ? t : T - 1) * H + kq * 8;
    wr[a] = wg + (int64_t)(e < E ? e : E - 1) * H + kq * 8;
  }
  f64x4_t acc[NT][NT];
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b) acc[a][b] = f64x4_t{0.0, 0.0, 0.0, 0.0};

  // Two register sets take turns: the loads of the next chunk are issued before the current
  // chunk is multiplied and waited for after it.  (Every load is unconditional, its index clamped
  // and opaque: a load under a condition makes the compiler wait for all loads in flight, and a
  // transparent index lets it fold the prefetch back into the next iteration's top.)
  const int nchunks = H / 32;
  struct Chunk {
    uint4 x[NT], w[NT];
  };
  auto fetch = [&](int c, Chunk &R) __attribute__((always_inline)) {
    int cc = c < nchunks ? c : nchunks - 1;
    asm volatile("" : "+s"(cc));
#pragma unroll
    for (int a = 0; a < NT; ++a) {
      R.x[a] = *reinterpret_cast<const uint4 *>(xr[a] + cc * 32);
      R.w[a] = *reinterpret_cast<const uint4 *>(wr[a] + cc * 32);
    }
  };
  // x_paired (optional): a copy of x with every 8-block in the order (x0,x4,x1,x5,x2,x6,x3,x7), which the
  // 4-bit tiled product reads.  The blocks of the first expert tile write it from the pieces they hold
  // anyway (the four waves of a block cover every chunk of its token rows between them).
  const bool pair_out = x_paired != nullptr && blockIdx.y == 0;  // block-uniform
  auto multiply = [&](const Chunk &R, int cidx) __attribute__((always_inline)) {
    if (pair_out) {
#pragma unroll
      for (int a = 0; a < NT; ++a) {
        const int64_t t = t0 + 16 * a + i;
        if (t < T) {
          const uint4 v = R.x[a];
          uint4 p;
          p.x = (v.x & 0xffffu) | (v.z << 16);
          p.y = (v.x >> 16) | (v.z & 0xffff0000u);
          p.z = (v.y & 0xffffu) | (v.w << 16);
          p.w = (v.y >> 16) | (v.w & 0xffff0000u);
          *reinterpret_cast<uint4 *>(x_paired + t * H + kq * 8 + cidx * 32) = p;
        }
      }
    }
    uint32_t xa[NT][4], wb[NT][4];
#pragma unroll
    for (int a = 0; a < NT; ++a) {
      xa[a][0] = R.x[a].x; xa[a][1] = R.x[a].y; xa[a][2] = R.x[a].z; xa[a][3] = R.x[a].w;
      wb[a][0] = R.w[a].x; wb[a][1] = R.w[a].y; wb[a][2] = R.w[a].z; wb[a][3] = R.w[a].w;
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      double av[NT], bv[NT];
#pragma unroll
      for (int a = 0; a < NT; ++a) {
        av[a] = (double)((s & 1) ? bf16hi_to_f32(xa[a][s >> 1]) : bf16lo_to_f32(xa[a][s >> 1]));
        bv[a] = (double)((s & 1) ? bf16hi_to_f32(wb[a][s >> 1]) : bf16lo_to_f32(wb[a][s >> 1]));
      }
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[a], bv[b], acc[a][b], 0, 0, 0);
    }
  };
  Chunk r0, r1;
  fetch(wave, r0);
  int c = wave;
  for (; c + 4 < nchunks; c += 8) {  // two chunks per turn, both multiplied without a condition
    fetch(c + 4, r1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(r0, c);
    __builtin_amdgcn_sched_barrier(0);
    fetch(c + 8, r0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(r1, c + 4);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (c < nchunks) multiply(r0, c);  // an odd chunk left over (already fetched)

  __shared__ double part[4][NT * NT][4][64];  // [wave][tile][r][lane]
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) part[wave][a * NT + b][r][lane] = acc[a][b][r];
  __syncthreads();
  // wave w finishes sub-tile w = (a, b) = (w / NT, w % NT); a lane's register r holds D[4 r + kq][i]
  // (fp64 tiles interleave the rows over the four lane groups, unlike the fp32 16x16 layout)
  if (wave >= NT * NT) return;
  const int a = wave / NT, b = wave % NT;
  const int e = e0 + 16 * b + i;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    double s = ((part[0][wave][r][lane] + part[1][wave][r][lane]) + part[2][wave][r][lane]) +
               part[3][wave][r][lane];
    const int64_t t = t0 + 16 * a + 4 * r + kq;
    if (t < T && e < E) {
      if (bias) s += (double)bias[e];
      logits[t * E + e] = f32_to_bf16((float)s);
    }
  }
}

bool router_logits_pairs_rows(int64_t T, int H) { return T > 64 && H % 32 == 0; }

hipError_t launch_router_logits(const uint16_t *x, const uint16_t *wg, const float *bias,
                                int64_t T, int H, int E, uint16_t *logits, hipStream_t st, uint16_t *x_paired) {
  if (T == 0) return hipSuccess;
  if (x_paired && !router_logits_pairs_rows(T, H)) return hipErrorInvalidValue;
  if (T <= 64) {
    dim3 grid((unsigned)T, (unsigned)((E + 3) / 4));
    router_logits_kernel<1, 1><<<grid, 256, 0, st>>>(x, wg, bias, T, H, E, logits);
  } else {
    // A block is bound by its CU's fp64 matrix rate whatever its number of waves, so what counts
    // is the number of blocks: 32 x 32 tiles when they fill the chip, 16 x 16 (four times the
    // blocks, each a quarter of the work) when they would not (512 tokens x 128 experts: 64 tiles).
    dim3 grid((unsigned)((T + 31) / 32), (unsigned)((E + 31) / 32));
    if ((int64_t)grid.x * grid.y >= 256) {
      router_logits_mfma_kernel<2><<<grid, 256, 0, st>>>(x, wg, bias, T, H, E, logits, x_paired);
    } else {
      grid = dim3((unsigned)((T + 15) / 16), (unsigned)((E + 15) / 16));
      router_logits_mfma_kernel<1><<<grid, 256, 0, st>>>(x, wg, bias, T, H, E, logits, x_paired);
    }
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------ select
// One wave per token.
template <int NV>
__global__ __launch_bounds__(256) void router_select_kernel(
    const uint16_t *__restrict__ logits, int64_t T, int E, int k, int mode,
    uint32_t *__restrict__ topk_idx, uint16_t *__restrict__ topk_w) {
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  select_wave<NV, false>(logits + t * E, E, k, mode, topk_idx + t * k, topk_w + t * k);
}

hipError_t launch_router_select(const uint16_t *logits, int64_t T, int E, int k, int mode,
                                uint32_t *topk_idx, uint16_t *topk_w, hipStream_t st) {
  if (T == 0) return hipSuccess;
  dim3 grid((unsigned)((T + 3) / 4));
#define MI_SEL(NV) \
  router_select_kernel<NV><<<grid, 256, 0, st>>>(logits, T, E, k, mode, topk_idx, topk_w)
  if (E <= 64) MI_SEL(1);
  else if (E <= 128) MI_SEL(2);
  else if (E <= 256) MI_SEL(4);
  else MI_SEL(8);  // E <= 512
#undef MI_SEL
  return hipGetLastError();
}

}  // namespace mi_moe
