// Shared device helpers and internal launcher declarations of libmi_moe (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

namespace mi_moe {

constexpr int kWave = 64;
// Which rows go to the tiled MFMA kernel.  A batch with an average of at least tiled_avg_rows(bits)
// rows per expert is "heavy": most segments are worth a tile, those of tile_min_rows(bits, true) rows
// or more (beyond one pass of the streaming kernel) are cut into M tiles, shorter ones stream.
// From light_avg_rows(bits) on a batch is "light": with even routing nearly every segment is cheaper
// on the streaming kernel, but a popular expert's segment is many passes long there (250 rows of a
// 256-token batch: 30 passes over that expert's weights), so segments of tile_min_rows(bits, false)
// rows or more (beyond two passes) are tiled.  Below light_avg_rows everything streams and the tile
// lists are not built.  Measured crossovers: see the design notes.
#ifndef MI_TMR4
#define MI_TMR4 9
#endif
#ifndef MI_TMR8
#define MI_TMR8 17
#endif
#ifndef MI_TAVG4
#define MI_TAVG4 20
#endif
#ifndef MI_TAVG8
#define MI_TAVG8 17
#endif
#ifndef MI_TLIGHT4
#define MI_TLIGHT4 6
#endif
#ifndef MI_TLIGHT8
#define MI_TLIGHT8 17
#endif
#ifndef MI_TMRL4
#define MI_TMRL4 17
#endif
#ifndef MI_TMRL8
#define MI_TMRL8 17
#endif
__host__ __device__ constexpr int tile_min_rows(int bits, bool heavy) {
  return bits == 4 ? (heavy ? MI_TMR4 : MI_TMRL4) : (heavy ? MI_TMR8 : MI_TMRL8);
}
__host__ __device__ constexpr int tiled_avg_rows(int bits) { return bits == 4 ? MI_TAVG4 : MI_TAVG8; }
__host__ __device__ constexpr int light_avg_rows(int bits) { return bits == 4 ? MI_TLIGHT4 : MI_TLIGHT8; }
inline bool heavy_batch(int64_t pairs, int n_experts, int bits) {
  return pairs >= (int64_t)tiled_avg_rows(bits) * n_experts;
}
inline bool tiled_batch(int64_t pairs, int n_experts, int bits) {
  return pairs >= (int64_t)light_avg_rows(bits) * n_experts || heavy_batch(pairs, n_experts, bits);
}
constexpr int kBigTileM = 256;       // rows of the largest M tile
constexpr int kFusedRouterMaxTokens = 64;  // up to here router + dispatch run as one launch

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

// ---------------------------------------------------------------- bfloat16
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float((uint32_t)h << 16);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) {
  return __uint_as_float(w & 0xffff0000u);
}
// round to nearest even; NaN stays NaN (quiet).  Integer arithmetic only: the bits are the
// same as the host-side checker's on every input.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u) ? ((u >> 16) | 0x40u) : r);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}
// two floats -> packed bf16 with the hardware converter (v_cvt_pk_bf16_f32, round to nearest
// even): for values that only have to be within tolerance
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// ---------------------------------------------------------------- exp for softmax
// 2^n * e^r with n = rint(x*log2 e), r by two-step Cody-Waite reduction and a degree-7
// polynomial, written with explicit fmaf so that no contraction choice of the compiler
// can change a bit.  Arguments below -80 give 0.  Same formula as the host-side checker.
__device__ __forceinline__ float det_expf(float x) {
  if (!(x >= -80.0f)) return 0.0f;
  if (x > 80.0f) x = 80.0f;
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, x);
  r = __builtin_fmaf(n, -1.42860682030941723e-6f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  float e = __builtin_fmaf(p, r2, r);
  e = e + 1.0f;
  int ni = (int)n;
  float s = __uint_as_float((uint32_t)(ni + 127) << 23);
  return e * s;
}

// ---------------------------------------------------------------- wave helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Wave-wide reductions whose result every lane holds.  Inside a row of 16 lanes the partners come
// through DPP (quad permutes, then the half-row and row mirrors: a few cycles each, no LDS traffic);
// the four row results are read as scalars and combined in the same fixed order by every lane.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
  const int lo = __builtin_amdgcn_mov_dpp(__double2loint(v), CTRL, 0xf, 0xf, true);
  const int hi = __builtin_amdgcn_mov_dpp(__double2hiint(v), CTRL, 0xf, 0xf, true);
  return __hiloint2double(hi, lo);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;

__device__ __forceinline__ double readlane_f64(double v, int l) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), l),
                          __builtin_amdgcn_readlane(__double2loint(v), l));
}
__device__ __forceinline__ double wave_sum_f64(double v) {
  v += dpp_f64<kDppXor1>(v);
  v += dpp_f64<kDppXor2>(v);
  v += dpp_f64<kDppHalfMirror>(v);
  v += dpp_f64<kDppMirror>(v);
  return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}
__device__ __forceinline__ float wave_max_f32(float v) {
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppXor1>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppXor2>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppHalfMirror>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppMirror>(__float_as_uint(v))));
  const uint32_t u = __float_as_uint(v);
  const float a = __uint_as_float(__builtin_amdgcn_readlane(u, 0)), b = __uint_as_float(__builtin_amdgcn_readlane(u, 16));
  const float c = __uint_as_float(__builtin_amdgcn_readlane(u, 32)), d = __uint_as_float(__builtin_amdgcn_readlane(u, 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  uint32_t o;
  o = dpp_u32<kDppXor1>(v); v = o > v ? o : v;
  o = dpp_u32<kDppXor2>(v); v = o > v ? o : v;
  o = dpp_u32<kDppHalfMirror>(v); v = o > v ? o : v;
  o = dpp_u32<kDppMirror>(v); v = o > v ? o : v;
  const uint32_t a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
  const uint32_t c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

// ---------------------------------------------------------------- M-tile lists
// Three lists, for tiles of 256, 128 and 64 rows, back to back in one buffer: a segment of at least
// tile_min_rows(bits, heavy) rows is cut into 256-row tiles; what is left goes to the smallest class that holds
// it.  List layout: word 0 = number of tiles, tile i at words 4 + 4 i = {expert, first sorted row,
// rows, 0}.  Capacities: cap256 for the first list, n_experts for the other two (a segment leaves
// at most one remainder).
__host__ __device__ inline size_t tile_list_words(int cap256, int n_experts) {
  return (4 + 4 * (size_t)cap256) + 2 * (4 + 4 * (size_t)n_experts);
}
template <class P>
__host__ __device__ inline P *tile_list(P *base, int cls, int cap256, int n_experts) {
  if (cls == 0) return base;
  if (cls == 1) return base + 4 + 4 * (size_t)cap256;
  return base + 4 + 4 * (size_t)cap256 + 4 + 4 * (size_t)n_experts;
}

// ---------------------------------------------------------------- device-coherent accesses
// A load that observes what other workgroups have written before an agent-scope release
// (bypasses the per-CU cache).  Used for data produced earlier in the same launch.
template <class T>
__device__ __forceinline__ T load_agent(const T *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The matching store: written through to where every workgroup's load_agent reads.
template <class T>
__device__ __forceinline__ void store_agent(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------- kernel timing (measurement only)
// While a timer is installed on the calling thread (mi_moe_forward_timed does that), a grouped-product
// launch goes through hipExtLaunchKernelGGL with the timer's two events: they then carry the start
// and end time stamps of that dispatch itself, which is what a profiler reports as the kernel's
// duration (an event recorded before and after a launch measures several microseconds more).
struct KernelTimer {
  hipEvent_t start = nullptr, stop = nullptr;
  bool used = false;  // a kernel was launched with these events
};
extern thread_local KernelTimer *g_kernel_timer;

// ---------------------------------------------------------------- which kernels the library holds, and which ran
// Every instantiation of a grouped-product kernel that a launcher can reach owns one slot (a static of
// the launcher's template, registered when the library is loaded), so the list is complete whether or
// not a kernel has ever run.  launch_kernel counts the launch in the slot.  With a plan installed on the
// calling thread (mi_moe_debug_plan) nothing is launched: the slot's name, grid and LDS size are
// written to the plan instead, which lets the launchers' host-side choices be checked without a GPU.
struct KernelSlot {
  char name[96];
  unsigned long long launches = 0;  // updated with __atomic builtins
  KernelSlot *next = nullptr;
  KernelSlot(const char *fmt, ...) __attribute__((format(printf, 2, 3)));
};
KernelSlot *kernel_slots();  // head of the list
struct LaunchPlan {
  char *out;
  size_t cap, len = 0;
  int n = 0;
};
extern thread_local LaunchPlan *g_launch_plan;
void plan_note(const KernelSlot &slot, dim3 grid, dim3 block, size_t lds);
inline bool planning() { return g_launch_plan != nullptr; }

template <class Kernel, class... Args>
inline void launch_kernel(KernelSlot &slot, Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t st, Args... args) {
  if (planning()) {
    plan_note(slot, grid, block, lds);
    return;
  }
  __atomic_fetch_add(&slot.launches, 1ull, __ATOMIC_RELAXED);
  if (KernelTimer *t = g_kernel_timer) {
    hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds, st, t->start, t->stop, 0, args...);
    t->used = true;
  } else {
    kernel<<<grid, block, lds, st>>>(args...);
  }
}

// ---------------------------------------------------------------- launchers (host)
// Each returns hipSuccess or the launch error.  All pointers are device pointers.
struct GroupedArgs {
  const uint16_t *x;        // bf16 rows of length K
  const uint16_t *x_perm;   // the same rows in the order the tiled kernel reads (4-bit: 8-blocks paired
                            // as x0,x4,x1,x5,x2,x6,x3,x7; 8-bit: identical to x)
  bool x_paired;            // x itself is already in the paired order
  bool y_paired;            // write the output columns in the paired order
  const uint32_t *src_rows; // x row of sorted row r, or nullptr = r
  bool src_in_work;         // the records' inline source rows equal src_rows (saves a dependent load)
  const uint32_t *dst_rows; // output row of sorted row r, or nullptr = r
  const uint32_t *work;        // 16-word records {expert, first row, rows, has_src, src[12]}, count 0 = end
  int max_active;              // upper bound of the number of records known on the host
  const uint32_t *mtiles;      // M-tile lists (tiled MFMA kernel), or nullptr
  int max_mtiles;              // capacity of the 256-row list
  int tile_cap_e;              // capacity of the 128- and 64-row lists (the number of experts)
  const uint32_t *w0, *w1;     // packed weights [E,N,K*bits/32]; w1 only for GLU
  const uint16_t *s0, *b0, *s1, *b1;
  uint16_t *y;                 // bf16 [rows, N]
  int N, K, bits;
  int64_t total_rows;          // host upper bound on rows (for tile selection)
  int64_t max_rows_per_expert; // host upper bound on the longest segment
  int64_t max_streamed_rows;   // host upper bound on the longest segment that is not tiled (0: no bound known)
};

// x_paired (optional, only where router_logits_pairs_rows says so): the kernel also writes the copy of x with
// paired 8-blocks that launch_pair_rows would make.
bool router_logits_pairs_rows(int64_t T, int H);
hipError_t launch_router_logits(const uint16_t *x, const uint16_t *wg, const float *bias,
                                int64_t T, int H, int E, uint16_t *logits, hipStream_t st,
                                uint16_t *x_paired = nullptr);
// the same logits (bit for bit) on the int8 matrix cores, for prefill-sized batches: router_exact.hip.
// scratch: router_logits_i8_bytes(T, H, E) bytes, contents irrelevant.
bool router_logits_i8_applies(int64_t T, int H, int E);
size_t router_logits_i8_bytes(int64_t T, int H, int E);
hipError_t launch_router_logits_i8(const uint16_t *x, const uint16_t *wg, const float *bias, int64_t T, int H, int E,
                                   uint16_t *logits, void *scratch, hipStream_t st, uint16_t *x_paired = nullptr);
// logits and selection in one kernel, up to 128 experts (router_exact.hip); scratch as for launch_router_logits_i8
bool router_tile_applies(int64_t T, int H, int E, int k);
hipError_t launch_router_tile(const uint16_t *x, const uint16_t *wg, const float *bias, int64_t T, int H, int E, int k,
                              int mode, uint16_t *logits, uint32_t *topk_idx, uint16_t *topk_w, void *scratch,
                              hipStream_t st, uint16_t *x_paired = nullptr);
hipError_t launch_router_select(const uint16_t *logits, int64_t T, int E, int k, int mode,
                                uint32_t *topk_idx, uint16_t *topk_w, hipStream_t st);
size_t dispatch_workspace_bytes(int E, int64_t P);
hipError_t launch_dispatch(const uint32_t *flat, int64_t P, int E, int k_div, uint32_t *counts,
                           uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                           uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int cap256, int big_thr,
                           void *scratch, hipStream_t st);
// decode-sized batches: logits + selection + dispatch in one launch.  counters: 1 +
// kFusedRouterMaxTokens zero-initialised words that the kernel leaves zeroed again.  norm_w != nullptr:
// the rows are RMS-normalised first (weight norm_w, eps) and kept in xnorm.
bool router_fused_applies(int64_t T, int E, int k);
hipError_t launch_router_fused(const uint16_t *x, const uint16_t *wg, const float *bias,
                               const uint16_t *norm_w, float eps, uint16_t *xnorm, int64_t T,
                               int H, int E, int k, int mode, uint16_t *logits, uint32_t *topk_idx,
                               uint16_t *topk_w, uint32_t *counters, uint32_t *counts,
                               uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm,
                               uint32_t *src_of, uint32_t *work, uint32_t *mtiles, int cap256,
                               int big_thr, hipStream_t st);
hipError_t launch_grouped_qmm(const GroupedArgs &a, bool glu, hipStream_t st);
hipError_t launch_large_qmm(const GroupedArgs &a, bool glu, hipStream_t st);
// the same work in its independent parts: one tile class (0, 1, 2 = 256-, 128-, 64-row tiles) of
// the tiled kernel, or the streaming kernel alone.  No part reads what another one writes.
bool large_qmm_applies(const GroupedArgs &a);
hipError_t launch_large_qmm_class(const GroupedArgs &a, bool glu, int cls, hipStream_t st);
hipError_t launch_small_qmm(const GroupedArgs &a, bool glu, hipStream_t st);
hipError_t launch_pair_rows(const uint16_t *x, int64_t rows, int K, uint16_t *out, hipStream_t st);
hipError_t launch_row_maps(const uint32_t *perm, const uint32_t *lhs, uint32_t n_lhs, const uint32_t *offsets,
                           int64_t n_idx, int M, int E, uint32_t *src_rows, uint32_t *dst_rows,
                           uint32_t *work, hipStream_t st);
hipError_t launch_dense_records(int64_t M, int big_thr, uint32_t *work, uint32_t *mtiles, int cap256,
                                hipStream_t st);
hipError_t launch_swiglu(const uint16_t *g, const uint16_t *u, int64_t n, uint16_t *out,
                         hipStream_t st);
hipError_t launch_stream_probe(const void *buf, size_t bytes, uint32_t *sink, hipStream_t st);
hipError_t launch_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm,
                          int64_t T, int k, int H, const uint16_t *residual, uint16_t *out,
                          hipStream_t st);
hipError_t launch_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T, int H,
                           uint16_t *out, hipStream_t st);
// plain products (any float type, group sizes 32 / 64 / 128, 2 / 4 / 8 bits, both weight layouts);
// dt: 0 bf16, 1 fp16, 2 fp32.  Output row r = j * M + m: expert rhs[rhs_map ? rhs_map[j] : j] (0 without
// rhs), x row (lhs ? lhs[j] : j) * M + m, destination row dst_map ? dst_map[r] : r.  n_lhs / n_rhs: how many
// matrices the lhs / rhs indices may address (0 = unknown); an index beyond is clamped to the last one.
hipError_t launch_qmm_plain(const void *x, const uint32_t *w, const void *scales, const void *biases,
                            const uint32_t *lhs, const uint32_t *rhs, const uint32_t *rhs_map,
                            const uint32_t *dst_map, uint32_t n_lhs, uint32_t n_rhs, int64_t rows, int M, int N,
                            int K, int group, int bits, bool transpose, int dt, void *y, hipStream_t st);
hipError_t launch_quantize(const float *w, int64_t rows, int64_t cols, int group, int bits,
                           uint32_t *q, void *s, void *b, int dt, hipStream_t st);
hipError_t launch_dequantize(const uint32_t *q, const void *s, const void *b,
                             int64_t rows, int64_t cols, int group, int bits, void *out, int dt, bool native_out,
                             hipStream_t st);
hipError_t launch_add_row_bias(void *y, const void *bias, int64_t M, int N, int dt, hipStream_t st);

}  // namespace mi_moe
