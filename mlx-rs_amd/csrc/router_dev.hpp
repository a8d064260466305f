// Device-side building blocks of the router, shared by the stand-alone router kernels and the
// fused decode router kernel: one logit per wave, and softmax / top-k / scores of one token per wave.
#pragma once

#include "common.hpp"

namespace mi_moe {

// logit of (token row xr, expert row wr): lanes split H in 16-byte pieces, exact bf16 x bf16
// products accumulated in fp64, butterfly sum.  Every lane returns the sum.
__device__ __forceinline__ double logit_wave(const uint16_t *__restrict__ xr,
                                             const uint16_t *__restrict__ wr, int H) {
  double acc = 0.0;
  // four pieces of each row per pass, all eight loads in flight before the first is used (a pass
  // covers 2048 values: one memory round trip for a row of that length instead of four); the
  // additions keep the order of a plain loop over the pieces
  for (int h0 = lane_id() * 8; h0 < H; h0 += 4 * kWave * 8) {
    uint4 xv[4], wv[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int h = h0 + p * kWave * 8;
      const int hc = h < H ? h : h0;  // (clamped: the loads carry no condition)
      xv[p] = *reinterpret_cast<const uint4 *>(xr + hc);
      wv[p] = *reinterpret_cast<const uint4 *>(wr + hc);
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      if (h0 + p * kWave * 8 < H) {
        const uint32_t xu[4] = {xv[p].x, xv[p].y, xv[p].z, xv[p].w}, wu[4] = {wv[p].x, wv[p].y, wv[p].z, wv[p].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc = __builtin_fma((double)bf16lo_to_f32(xu[q]), (double)bf16lo_to_f32(wu[q]), acc);
          acc = __builtin_fma((double)bf16hi_to_f32(xu[q]), (double)bf16hi_to_f32(wu[q]), acc);
        }
      }
    }
  }
  return wave_sum_f64(acc);
}

// 1 / sqrt(mean(x^2) + eps) of a row, by one wave: the mean of squares in fp64 over exact products,
// the rest in correctly rounded float operations (the bits of the host-side checker).
__device__ __forceinline__ float row_rstd_wave(const uint16_t *__restrict__ xr, int H, float eps) {
  double ss = 0.0;
  for (int h = lane_id() * 8; h < H; h += kWave * 8) {
    const uint4 v = *reinterpret_cast<const uint4 *>(xr + h);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const double a = (double)bf16lo_to_f32(u[i]), b = (double)bf16hi_to_f32(u[i]);
      ss = __builtin_fma(a, a, ss);
      ss = __builtin_fma(b, b, ss);
    }
  }
  ss = wave_sum_f64(ss);
  return 1.0f / sqrtf((float)(ss / (double)H) + eps);
}
// eight normalised values of a row: bf16(weight * (x * rstd)), packed
__device__ __forceinline__ uint4 rms_norm8(uint4 v, uint4 w, float rstd) {
  const uint32_t u[4] = {v.x, v.y, v.z, v.w}, wu[4] = {w.x, w.y, w.z, w.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = bf16lo_to_f32(u[i]) * rstd, hi = bf16hi_to_f32(u[i]) * rstd;
    o[i] = pack_bf16x2(bf16lo_to_f32(wu[i]) * lo, bf16hi_to_f32(wu[i]) * hi);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}
// logit of (rms_norm(token row), expert row); the wave optionally writes the normalised row
__device__ __forceinline__ double logit_wave_norm(const uint16_t *__restrict__ xr,
                                                  const uint16_t *__restrict__ wr,
                                                  const uint16_t *__restrict__ norm_w, float eps, int H,
                                                  uint16_t *xn_out) {
  const float rstd = row_rstd_wave(xr, H, eps);
  double acc = 0.0;
  for (int h = lane_id() * 8; h < H; h += kWave * 8) {
    const uint4 xv = rms_norm8(*reinterpret_cast<const uint4 *>(xr + h),
                               *reinterpret_cast<const uint4 *>(norm_w + h), rstd);
    if (xn_out) *reinterpret_cast<uint4 *>(xn_out + h) = xv;
    const uint4 wv = *reinterpret_cast<const uint4 *>(wr + h);
    const uint32_t xu[4] = {xv.x, xv.y, xv.z, xv.w}, wu[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      acc = __builtin_fma((double)bf16lo_to_f32(xu[q]), (double)bf16lo_to_f32(wu[q]), acc);
      acc = __builtin_fma((double)bf16hi_to_f32(xu[q]), (double)bf16hi_to_f32(wu[q]), acc);
    }
  }
  return wave_sum_f64(acc);
}

// float -> unsigned key whose unsigned order is the float order; -0 is mapped to +0 so
// that the two zeros tie (and the lower expert id wins) as they do in a float compare.
__device__ __forceinline__ uint32_t ordered_key(float f) {
  uint32_t u = __float_as_uint(f);
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}
// Softmax, top-k and scores of one token by one wave.  Lane l holds experts l, l+64, ... (NV of
// them).  COHERENT: the logits were written by other workgroups of the same launch.
// The values the selection compares are exact in bf16 (rounded probabilities, or the logits
// themselves), so value and expert id fit one 32-bit key: the upper half is the order-preserving
// key of the bf16 value, the lower half 0xffff - expert id (lower id wins a tie).
// a token's logits as the selecting wave holds them: lane l takes experts l, l + 64, ...
template <int NV, bool COHERENT>
__device__ __forceinline__ void load_logit_row(const uint16_t *row, int E, uint16_t (&bits)[NV]) {
  const int lane = lane_id();
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int e = j * kWave + lane;
    bits[j] = 0;
    if (e < E) bits[j] = COHERENT ? load_agent(row + e) : row[e];
  }
}

// COHERENT: the selected experts are read by another workgroup of the same launch.  idx_lds (optional):
// a second copy of the selected experts for a dispatch that follows in the same workgroup.
template <int NV, bool COHERENT>
__device__ __forceinline__ void select_from_bits(const uint16_t (&bits)[NV], int E, int k, int mode,
                                                 uint32_t *idx_out, uint16_t *__restrict__ w_out,
                                                 uint32_t *idx_lds = nullptr) {
  const int lane = lane_id();
  float g[NV], v[NV];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int e = j * kWave + lane;
    g[j] = e < E ? bf16_to_f32(bits[j]) : -INFINITY;
    m = fmaxf(m, g[j]);
  }
  if (mode != 2) {
    m = wave_max_f32(m);
    float ex[NV];
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = j * kWave + lane;
      ex[j] = e < E ? det_expf(g[j] - m) : 0.0f;
      sum += (double)ex[j];
    }
    sum = wave_sum_f64(sum);
    const float sf = (float)sum;
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = bf16_to_f32(f32_to_bf16(ex[j] / sf));
  } else {
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = g[j];
  }

  uint32_t key[NV];  // 0 = not a candidate (no real key is 0: the id half of a real key is >= 0xfe00)
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int e = j * kWave + lane;
    key[j] = e < E ? ((ordered_key(v[j]) & 0xffff0000u) | (0xffffu - (uint32_t)e)) : 0u;
  }
  // k rounds of wave-wide arg-max
  uint32_t my_key = 0;
  for (int s = 0; s < k; ++s) {
    uint32_t best = 0;
#pragma unroll
    for (int j = 0; j < NV; ++j) best = key[j] > best ? key[j] : best;
    best = wave_max_u32(best);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (key[j] == best) key[j] = 0u;  // keys are distinct: exactly one lane drops its candidate
    if (lane == s) my_key = best;
  }
  const uint32_t my_idx = 0xffffu - (my_key & 0xffffu);
  const uint32_t hi = my_key & 0xffff0000u;
  const float my_val = key_to_float((hi & 0x80000000u) ? hi : (hi | 0xffffu));

  // scores; lane s holds slot s
  float score;
  if (mode == 2) {
    const float mx = __shfl(my_val, 0, kWave);  // slot 0 is the largest logit
    const float e_s = lane < k ? det_expf(my_val - mx) : 0.0f;
    double sum = 0.0;
    for (int s = 0; s < k; ++s) sum += (double)__shfl(e_s, s, kWave);
    score = e_s / (float)sum;
  } else {
    score = my_val;
    if (mode == 0) {
      float sum = 0.0f;
      for (int s = 0; s < k; ++s) sum += __shfl(my_val, s, kWave);
      const float denom = bf16_to_f32(f32_to_bf16(sum));
      score = my_val / denom;
    }
  }
  if (lane < k) {
    if (COHERENT) store_agent(idx_out + lane, my_idx);  // read by another workgroup of this launch
    else idx_out[lane] = my_idx;
    if (idx_lds) idx_lds[lane] = my_idx;
    w_out[lane] = f32_to_bf16(score);
  }
}

template <int NV, bool COHERENT>
__device__ __forceinline__ void select_wave(const uint16_t *row, int E, int k, int mode,
                                            uint32_t *idx_out,
                                            uint16_t *__restrict__ w_out) {
  uint16_t bits[NV];
  load_logit_row<NV, COHERENT>(row, E, bits);
  select_from_bits<NV, COHERENT>(bits, E, k, mode, idx_out, w_out);
}

}  // namespace mi_moe
