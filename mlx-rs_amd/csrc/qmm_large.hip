// Tiled grouped quantized product for expert segments of more than 8 rows (prefill).
//
// Same contract as the small-segment kernel (mlx_gather_qmm with transpose = true,
// mlx-rs/src/ops/quantization.rs:160-230; with GLU also nn::silu and multiply,
// nn/activation.rs:142-144,876-880), restricted to the segments the dispatch cut into M tiles
// of 256, 128 or 64 rows.  A block of 8 waves computes a (256 | 128 | 64)-token x 256-weight-row tile:
//   * weights stream from HBM as packed codes (one 8- or 16-byte load per thread and K step; scales
//     and biases in 8-byte pieces that last 16 K steps),
//     are dequantised ONCE per block to bf16 (w_hat = s q + b, fp32 fma, one rounding) and
//     parked in LDS, so the cost of unpacking is shared by the 256 token rows of the tile;
//   * the token rows are gathered through the sorted-row -> source-row map straight into LDS
//     (no materialised gather);
//   * 8 waves (2 x 4) run v_mfma_f32_32x32x16_bf16 on 128 x 64 sub-tiles, fp32 accumulators;
//   * with GLU the 256 weight rows are 128 gate rows and the matching 128 up rows, each wave owns
//     32 + 32 of them, and the epilogue writes silu(gate) * up without either product ever
//     reaching memory.
// Three K steps of global loads are in flight while the current one is multiplied.
#include <type_traits>

#include <atomic>

#include "common.hpp"

#ifndef MI_MOE_WEAVE
#define MI_MOE_WEAVE 1
#endif
// VALU instructions of the stage woven in after each MFMA of a step, per 32-row token sub-tile of a wave
// (256-row tiles / shorter ones; measured: 16 / 12, with 12 / 12 the 256-row class loses 1 %, with 16 / 16 the
// 128-row class 7 %)
#ifndef MI_WEAVE_VALU
#define MI_WEAVE_VALU 16
#endif
#ifndef MI_WEAVE_VALU_SHORT
#define MI_WEAVE_VALU_SHORT 12
#endif

namespace mi_moe {

namespace {

constexpr int BK = 32;         // K step (two steps per quantisation group)
constexpr int BR = 256;        // weight rows per block (GLU: 128 gate + 128 up)
constexpr int NTHREADS = 512;  // 8 waves: 2 (token halves) x 4 (weight-row quarters)
constexpr int DEPTH = 4;       // register stages: three K steps of global loads in flight
#ifndef MI_SPREAD_BELOW
#define MI_SPREAD_BELOW 64
#endif
constexpr int kSpreadBelow = MI_SPREAD_BELOW;  // M tiles in a list below which its N tiles are dealt over the XCDs
static_assert(kSpreadBelow >= 1, "the launcher sizes the grid for kSpreadBelow - 1 M tiles");

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// LDS tiles hold rows of 32 bf16 (four 16-byte chunks) at a stride of 80 bytes: consecutive
// rows reading the same chunk start 20 banks apart, which keeps 16-byte reads of 8 or 16
// consecutive rows clear of each other.
constexpr int LDR = 5;  // row stride in uint4 units
__device__ __forceinline__ int tile_off(int row, int chunk) { return row * LDR + chunk; }
constexpr size_t large_lds_bytes(int bm) { return (size_t)2 * (bm + BR) * LDR * 16; }  // two steps of A and B tiles

}  // namespace

// Why this shape.  Measured on the 256 x 128 / 4-wave predecessor of this kernel: its global loads
// alone (no LDS, no MFMA) took 0.9 us per K step against 0.43 us of MFMA work, because a step could
// not start before loads issued only one to two steps earlier had come back (~1 us under load).
// A 256 x 256 tile halves the activation bytes per MFMA, 512 threads halve the staging registers a
// thread needs per step, and the registers saved pay for four stages, i.e. three steps of loads in
// flight.  Per-step 2-byte gathers of scales and biases (more expensive than all other loads of
// that kernel together) became one 8-byte load per 16 steps.
//
// MT = token rows per block / 64 (4, 2 or 1): the same kernel on 256-, 128- and 64-row M tiles, so
// that a short segment or the short end of a long one does not pay for 256 rows of MFMA work.  The
// weight side (256 rows dequantised per step) is the same for all three; with 64 rows the kernel is
// bound by that dequantisation, which is still far cheaper than streaming the weights once per
// 8 tokens.
template <int BITS, bool GLU, int MT>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, MT == 4 ? 2 : 4))) void qmm_large_kernel(GroupedArgs a, const uint32_t *__restrict__ tiles, int n_ntiles, int cap, int chunk, int sub_log2) {
  constexpr int NI = GLU ? 128 : 256;  // distinct output columns per block
  constexpr int BM = 64 * MT;          // token rows per block
  constexpr int NA = MT >= 2 ? MT / 2 : 1;  // 16-byte activation loads per thread and step

  // block -> (M tile, N tile).  Block ids are dealt round-robin over the 8 XCDs, each with its own
  // L2.  Many M tiles: the blocks of one M tile share its gathered token rows, so they get
  // consecutive ids on ONE XCD.  Few M tiles (a small batch, or few experts with wide matrices):
  // whole tiles per XCD would leave XCDs idle (one M tile of a 14336-wide GLU is 112 blocks, all on
  // one XCD's 32 CUs), so the N tiles of an M tile are dealt over the XCDs in chunks of `chunk`.
  // Both candidate records are fetched along with the count (indices clamped to the list's capacity).
  // sub_log2 > 0: the list's tiles are larger than this kernel's; each is taken as 2 or 4 M tiles of
  // BM rows (the launcher does that when even so the chip has blocks to spare: a 64-row block's
  // K step is shorter than a 256-row block's).
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int n_chunks = (n_ntiles + chunk - 1) / chunk;
  const uint32_t whole_id = (uint32_t)(j / n_ntiles) * 8u + xcd;
  const uint32_t unit = (uint32_t)(j / chunk) * 8u + xcd;
  const uint32_t spread_id = unit / (uint32_t)n_chunks;
  const uint4 *const recs = reinterpret_cast<const uint4 *>(tiles) + 1;
  const uint32_t whole_rec = whole_id >> sub_log2, spread_rec = spread_id >> sub_log2;
  const uint4 rec_whole = recs[whole_rec < (uint32_t)cap ? whole_rec : (uint32_t)cap - 1u];
  const uint4 rec_spread = recs[spread_rec < (uint32_t)cap ? spread_rec : (uint32_t)cap - 1u];
  const uint32_t n_mtiles = tiles[0] << sub_log2;
  const bool spread = n_mtiles < (uint32_t)kSpreadBelow;
  const uint32_t mt_id = spread ? spread_id : whole_id;
  const int nt = spread ? (int)(unit % (uint32_t)n_chunks) * chunk + j % chunk : j % n_ntiles;
  const uint4 rec = spread ? rec_spread : rec_whole;
  if (mt_id >= n_mtiles || nt >= n_ntiles) return;
  const int part = (int)(mt_id & ((1u << sub_log2) - 1u)) * BM;  // first row of this block's piece of the tile
  const int e = (int)rec.x;
  const int64_t row0 = (int64_t)rec.y + part;
  const int rows = (int)rec.z - part < BM ? (int)rec.z - part : BM;
  if (rows <= 0) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int N = a.N, K = a.K;
  const int n0 = nt * NI;
  const int row_bytes = K * BITS / 8, gpr = K / 64;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  u32x4_t *const lds = reinterpret_cast<u32x4_t *>(lds_raw);
  // [A step-parity 0][A parity 1][B parity 0][B parity 1]
  auto As = [&](int buf) { return lds + buf * (BM * LDR); };
  auto Bs = [&](int buf) { return lds + 2 * BM * LDR + buf * (BR * LDR); };

  // ---- global -> register stage
  // A: the activations arrive with every 8-block already in the (x0,x4,x1,x5,x2,x6,x3,x7) order
  // of the nibble unpacking (4-bit), so a row chunk is copied as it is.  Thread: chunk acp of
  // rows arg, arg + 128 (64-row tiles: the first four waves only).
  const int acp = tid & 3, arg = tid >> 2;
  const bool a_loader = MT >= 2 || wave < 4;  // wave-uniform
  auto a_row_ptr = [&](int tr) {
    tr = tr < rows ? tr : rows - 1;  // rows past the segment repeat its last row (never stored)
    const int64_t r = row0 + tr;
    const int64_t src = a.src_rows ? (int64_t)a.src_rows[r] : r;
    return a.x_perm + src * K + acp * 8;
  };
  const uint16_t *arow[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) arow[i] = a_row_ptr(arg + 128 * i);
  // B: thread covers 16 codes (half a K step) of weight row br; waves 0-3 / 4-7 hold gate / up
  const int br = tid >> 1, bh = tid & 1;
  const int mat = GLU ? (wave >> 2) : 0;  // wave-uniform
  // paired output (columns of every 8-block in the order 0,4,1,5,2,6,3,7, what a 4-bit consumer
  // of these rows expects as its activations): the thread at position p of an 8-block stages the
  // weight row whose result belongs there, and the epilogue has nothing to permute
  const int brp = a.y_paired ? ((br & ~7) | (((br & 7) >> 1) + ((br & 1) ? 4 : 0))) : br;
  const int nrow = GLU ? n0 + (brp & 127) : n0 + brp;  // rows >= N read zeros through the descriptor
  const int64_t ebase = (int64_t)e * N;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc((mat ? a.w1 : a.w0) + ebase * (row_bytes / 4), (uint32_t)N * row_bytes);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc((mat ? a.s1 : a.s0) + ebase * gpr, (uint32_t)N * gpr * 2);
  const __amdgpu_buffer_rsrc_t brs = make_rsrc((mat ? a.b1 : a.b0) + ebase * gpr, (uint32_t)N * gpr * 2);
  const uint32_t w_voff = (uint32_t)nrow * row_bytes + bh * (BITS == 4 ? 8 : 16);
  // scales / biases: a thread keeps a window of 8 groups (16 K steps) of its row, half of it in
  // its own registers (groups 4 bh .. 4 bh + 3 of the window, one 8-byte load per tensor) and half
  // in its neighbour's (the other thread of the row).
  const uint32_t g_voff = (uint32_t)nrow * gpr * 2 + bh * 8;
  struct SbWindow {
    u32x2_t s, b;
  };
  auto load_window = [&](int w) __attribute__((always_inline)) {
    SbWindow v;
    v.s = __builtin_amdgcn_raw_buffer_load_b64(sr, g_voff, w * 16, 0);
    v.b = __builtin_amdgcn_raw_buffer_load_b64(brs, g_voff, w * 16, 0);
    return v;
  };

  struct Stage {
    u32x4_t av[NA];
    u32x4_t bw;  // 4-bit: two words used
  };
  // every load is unconditional (indices are clamped by the caller): the compiler can then count
  // the loads in flight and wait for exactly the stage it needs
  auto gload = [&](int ks, Stage &R) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NA; ++i) R.av[i] = *reinterpret_cast<const u32x4_t *>(arow[i] + ks * BK);
    if constexpr (BITS == 4) {
      const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(wr, w_voff, ks * 16, 0);
      R.bw[0] = v[0];
      R.bw[1] = v[1];
    } else {
      R.bw = __builtin_amdgcn_raw_buffer_load_b128(wr, w_voff, ks * 32, 0);
    }
  };

  // ---- register -> LDS stage: copy A, dequantise B once for the whole block
  auto stage = [&](int buf, const Stage &R, const SbWindow &sb, int step) __attribute__((always_inline)) {
    u32x4_t *const At = As(buf), *const Bt = Bs(buf);
    if (a_loader) {
#pragma unroll
      for (int i = 0; i < NA; ++i) At[tile_off(arg + 128 * i, acp)] = R.av[i];
    }
    // group of this step inside the window: which thread of the row holds it, which word, which half
    const int gi = (step >> 1) & 7;
    uint32_t sw = (gi & 2) ? sb.s[1] : sb.s[0];
    uint32_t bw = (gi & 2) ? sb.b[1] : sb.b[0];
    const uint32_t sn = (uint32_t)__builtin_amdgcn_mov_dpp((int)sw, 0xB1, 0xf, 0xf, true);  // lane ^ 1
    const uint32_t bn = (uint32_t)__builtin_amdgcn_mov_dpp((int)bw, 0xB1, 0xf, 0xf, true);
    if ((gi >> 2) != bh) {
      sw = sn;
      bw = bn;
    }
    const float sc = (gi & 1) ? bf16hi_to_f32(sw) : bf16lo_to_f32(sw);
    float bi = (gi & 1) ? bf16hi_to_f32(bw) : bf16lo_to_f32(bw);
    if constexpr (BITS == 4) {
      // codes are expanded as the fp16 values 1024 + q (exact: 0x6400 is 1024.0 with a last place of 1), a pair
      // (q_i, q_{i+4}) per register in one shift and one and-or; the mixed-precision fma reads the halves as
      // they are, so no conversion instruction stands between the codes and w_hat
      typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
      bi = __builtin_fmaf(-1024.0f, sc, bi);
#pragma unroll
      for (int wi = 0; wi < 2; ++wi) {
        const uint32_t w = R.bw[wi];
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t pr = __builtin_amdgcn_bitop3_b32(w >> (4 * i), 0x000f000fu, 0x64006400u, 0xEA);  // (a & b) | c
          const half2_t h = __builtin_bit_cast(half2_t, pr);
          o[i] = cvt_pk_bf16(__builtin_fmaf(sc, (float)h.x, bi), __builtin_fmaf(sc, (float)h.y, bi));
        }
        Bt[tile_off(br, 2 * bh + wi)] = u32x4_t{o[0], o[1], o[2], o[3]};
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // 8 codes = two words -> one chunk
        const uint32_t wA = R.bw[2 * h], wB = R.bw[2 * h + 1];
        uint32_t o[4];
        o[0] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wA & 0xffu), bi), __builtin_fmaf(sc, (float)((wA >> 8) & 0xffu), bi));
        o[1] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wA >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wA >> 24), bi));
        o[2] = cvt_pk_bf16(__builtin_fmaf(sc, (float)(wB & 0xffu), bi), __builtin_fmaf(sc, (float)((wB >> 8) & 0xffu), bi));
        o[3] = cvt_pk_bf16(__builtin_fmaf(sc, (float)((wB >> 16) & 0xffu), bi), __builtin_fmaf(sc, (float)(wB >> 24), bi));
        Bt[tile_off(br, 2 * bh + h)] = u32x4_t{o[0], o[1], o[2], o[3]};
      }
    }
  };

  // ---- MFMA stage: wave (wm, wn) owns token rows [BM/2 wm, + BM/2) and two 32-row weight
  // sub-tiles.  64-row tiles: one 32-row sub-tile per wave.
  constexpr int MS = MT >= 2 ? MT : 1;  // 32-row token sub-tiles per wave
  f32x16_t acc[MS][2];
#pragma unroll
  for (int m = 0; m < MS; ++m)
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[m][s][r] = 0.f;
  const int ln = lane & 31, kb = lane >> 5;
  const int brow0 = (GLU ? 32 * wn : 64 * wn) + ln;             // gate rows / first 32 rows
  const int brow1 = (GLU ? 128 + 32 * wn : 64 * wn + 32) + ln;  // the matching up rows / next 32
  const int arow0 = (BM / 2) * wm + ln;

  auto mma = [&](int cur) __attribute__((always_inline)) {
    const u32x4_t *const At = As(cur), *const Bt = Bs(cur);
#pragma unroll
    for (int ss = 0; ss < 2; ++ss) {
      const int c = 2 * kb + ss;
      const u32x4_t b0 = Bt[tile_off(brow0, c)];
      const u32x4_t b1 = Bt[tile_off(brow1, c)];
#pragma unroll
      for (int m = 0; m < MS; ++m) {
        const u32x4_t av = At[tile_off(arow0 + 32 * m, c)];
        acc[m][0] = mfma32(av, b0, acc[m][0]);
        acc[m][1] = mfma32(av, b1, acc[m][1]);
      }
    }
  };

  // K loop.  nk is a multiple of 4 (the launcher takes K in multiples of 128 only).  Step ks:
  // stage step ks from register set ks & 3 into LDS buffer ks & 1 (last read two steps ago, before
  // the previous barrier), reload the set freed one step ago with step ks + 3, multiply step ks - 1
  // from the other buffer.  Steps ks + 1 .. ks + 3 are in flight meanwhile.  Outer loop: one window
  // of scales / biases (16 steps), whose loads sit outside any condition for the same reason the
  // step loads do, and which is only read in the iteration after the one that loaded it.
  const int nk = K / BK;
  Stage R[DEPTH];
  SbWindow sb_cur, sb_next = load_window(0);
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d) gload(d, R[d]);

  // four steps, register sets and LDS buffers by constant index.  FIRST: steps 0..3, where step 0
  // has nothing to multiply yet.  Inside a step the dequantisation arithmetic of the stage is
  // independent of the MFMAs (they work on the other LDS buffer), and the two waves of a SIMD run
  // their steps in phase (same block, same barriers), so the scheduler is asked to weave the
  // stage's VALU work between the MFMAs instead of running the two phases one after the other.
  auto group = [&](int kq, auto first) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first)::value;
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int ks = kq + d;
      gload(ks + DEPTH - 1 < nk ? ks + DEPTH - 1 : nk - 1, R[(d + DEPTH - 1) & 3]);  // a repeat at the very end
      // the multiply comes first in program order: its LDS reads must not queue behind the stage's
      // LDS writes (the compiler cannot tell the two buffers apart), which hang on the stage's VALU work
      if (!(FIRST && d == 0)) mma((d + 1) & 1);
      stage(d & 1, R[d], sb_cur, ks);
#if MI_MOE_WEAVE
      if (!(FIRST && d == 0)) {
        __builtin_amdgcn_sched_group_barrier(0x100, 2 + MS, 0);  // first operands from LDS
#pragma unroll
        for (int i = 0; i < 4 * MS; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, (MT == 4 ? MI_WEAVE_VALU : MI_WEAVE_VALU_SHORT) / MS, 0);  // its share of the stage's VALU work
          if (i < 2 + MS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // the remaining LDS reads
        }
      }
#endif
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);  // nothing moves between steps: a stage hoisted across would
                                          // wait for its loads one step early
    }
  };
  sb_cur = sb_next;
  sb_next = load_window(1);
  group(0, std::true_type{});
  for (int kq = DEPTH; kq < (16 < nk ? 16 : nk); kq += DEPTH) group(kq, std::false_type{});
  for (int k0 = 16; k0 < nk; k0 += 16) {
    sb_cur = sb_next;
    sb_next = load_window((k0 >> 4) + 1);
    const int k1 = k0 + 16 < nk ? k0 + 16 : nk;
    for (int kq = k0; kq < k1; kq += DEPTH) group(kq, std::false_type{});
  }
  mma(1);  // step nk - 1 (odd)

  // ---- epilogue: D[i][j], lane holds column j = lane % 32 and rows 8 (r/4) + 4 (lane/32) + r%4:
  // stored from there, a wave's store instruction would write 2 bytes per lane (measured: 50 to
  // 70 us per launch of the 256-row class at 4096 tokens, a third of the kernel).  Each wave turns
  // its 32-row sub-tiles round in a private piece of LDS instead and stores 16 bytes per lane, whole
  // 64- or 128-byte pieces of output rows.
  constexpr int CW = GLU ? 32 : 64;   // output columns of a wave
  constexpr int ROWB = CW * 2 + 16;   // bytes per staged row (the 16 keep rows off each other's banks)
  constexpr int CPR = CW / 8;         // 16-byte pieces per row
  constexpr int RPI = 64 / CPR;       // rows one store instruction covers
  static_assert(8 * 32 * ROWB <= large_lds_bytes(64), "staging does not fit the smallest tile's LDS");
  __syncthreads();  // every wave has read its last operands: the space is free
  unsigned char *const mine = lds_raw + wave * (32 * ROWB);
  const int col0 = n0 + CW * wn;
  const int my_piece = lane % CPR, my_row = lane / CPR;
  const bool piece_ok = col0 + 8 * my_piece < N;  // N is a multiple of 16: a piece is inside or outside
  // where the rows of this wave's half of the tile go: lane l fetches rows l and 64 + l of the
  // half (one latency for all of them), a lane shuffle hands them out below
  constexpr int NH = BM / 2 > 64 ? BM / 128 : 1;
  uint32_t dst_half[NH];
#pragma unroll
  for (int h = 0; h < NH; ++h) {
    int tr = (BM / 2) * wm + 64 * h + lane;
    tr = tr < rows ? tr : rows - 1;
    const int64_t rr = row0 + tr;
    dst_half[h] = a.dst_rows ? a.dst_rows[rr] : (uint32_t)rr;
  }
#pragma unroll
  for (int m = 0; m < MS; ++m) {
    // two rows of a column become one register (bf16 pair); neighbouring lanes (columns c, c + 1)
    // swap halves, so that the even lane holds row r and the odd lane row r + 1 of both columns:
    // one 4-byte LDS write per two results
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const int row = 8 * (r >> 2) + 4 * kb + (r & 3) + (ln & 1);
#pragma unroll
      for (int s = 0; s < (GLU ? 1 : 2); ++s) {
        uint32_t mine2;
        if constexpr (GLU) {
          const float g0 = acc[m][0][r], u0 = acc[m][1][r], g1 = acc[m][0][r + 1], u1 = acc[m][1][r + 1];
          mine2 = cvt_pk_bf16(g0 / (1.0f + __expf(-g0)) * u0, g1 / (1.0f + __expf(-g1)) * u1);
        } else {
          mine2 = cvt_pk_bf16(acc[m][s][r], acc[m][s][r + 1]);
        }
        const uint32_t theirs = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine2, 0xB1, 0xf, 0xf, true);  // lane ^ 1
        // even lane: (mine.lo, theirs.lo) = row r, columns c, c + 1; odd: (theirs.hi, mine.hi) = row r + 1
        const uint32_t both = __builtin_amdgcn_perm(theirs, mine2, (ln & 1) ? 0x03020706u : 0x05040100u);
        *reinterpret_cast<uint32_t *>(mine + row * ROWB + (32 * s + (ln & ~1)) * 2) = both;
      }
    }
    // LDS serves a wave's accesses in order; the fence and the barrier only pin the program order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = RPI * i + my_row;
      const int tr = (BM / 2) * wm + 32 * m + row;
      const u32x4_t v = *reinterpret_cast<const u32x4_t *>(mine + row * ROWB + my_piece * 16);
      // row 32 m + row of the half is held by lane (32 m + row) % 64 of dst_half[(32 m + row) / 64]
      const uint32_t dst = (uint32_t)__shfl((int)dst_half[(32 * m + RPI * i) >> 6], (32 * m + row) & 63, 64);
      if (tr < rows && piece_ok) *reinterpret_cast<u32x4_t *>(a.y + (int64_t)dst * N + col0 + 8 * my_piece) = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// Activation rows with every 8-block reordered to (x0,x4,x1,x5,x2,x6,x3,x7): the order in which
// one and+or per register unpacks the eight 4-bit codes of a word.
__global__ __launch_bounds__(256) void pair_rows_kernel(const uint4 *__restrict__ x, int64_t n, uint4 *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint4 v = x[i];
  uint4 p;
  p.x = (v.x & 0xffffu) | (v.z << 16);
  p.y = (v.x >> 16) | (v.z & 0xffff0000u);
  p.z = (v.y & 0xffffu) | (v.w << 16);
  p.w = (v.y >> 16) | (v.w & 0xffff0000u);
  out[i] = p;
}

hipError_t launch_pair_rows(const uint16_t *x, int64_t rows, int K, uint16_t *out, hipStream_t st) {
  const int64_t n = rows * K / 8;
  if (n == 0) return hipSuccess;
  pair_rows_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(reinterpret_cast<const uint4 *>(x), n,
                                                               reinterpret_cast<uint4 *>(out));
  return hipGetLastError();
}

template <int BITS, bool GLU, int MT>
KernelSlot large_slot("qmm_large_kernel<%d,%d,%d>", BITS, (int)GLU, MT);

template <int BITS, bool GLU, int MT>
static hipError_t launch_one(const GroupedArgs &a, const uint32_t *tiles, int list_cap, int sub_log2, hipStream_t st) {
  const int cap = list_cap << sub_log2;  // M tiles of this kernel's size
  const int ni = GLU ? 128 : 256;
  const int n_ntiles = (a.N + ni - 1) / ni;
  // ids for either dealing of the tiles (see the kernel): whole M tiles per XCD, or chunks of an
  // M tile's N tiles when the list holds fewer than kSpreadBelow M tiles
  const int chunk = (n_ntiles + 7) / 8, n_chunks = (n_ntiles + chunk - 1) / chunk;
  const unsigned whole = (unsigned)((cap + 7) / 8) * 8u * (unsigned)n_ntiles;
  const unsigned few = (unsigned)(cap < kSpreadBelow - 1 ? cap : kSpreadBelow - 1);
  const unsigned spread = (few * (unsigned)n_chunks + 7u) / 8u * 8u * (unsigned)chunk;
  const unsigned grid = whole > spread ? whole : spread;
  constexpr size_t lds = large_lds_bytes(64 * MT);
  // more LDS per block than a kernel gets without asking: asked for once per device (the attribute
  // belongs to the device's copy of the kernel); two threads asking at once is harmless
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> raised[kMaxDevices];
  int dev = 0;
  if (!planning())
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (!planning() && (dev < 0 || dev >= kMaxDevices || !raised[dev].load(std::memory_order_acquire))) {
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&qmm_large_kernel<BITS, GLU, MT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        e != hipSuccess)
      return e;
    if (dev >= 0 && dev < kMaxDevices) raised[dev].store(true, std::memory_order_release);
  }
  launch_kernel(large_slot<BITS, GLU, MT>, qmm_large_kernel<BITS, GLU, MT>, dim3(grid), dim3(NTHREADS), lds, st, a, tiles,
                n_ntiles, list_cap, chunk, sub_log2);
  return planning() ? hipSuccess : hipGetLastError();
}

// class 0 / 1 / 2 = the 256- / 128- / 64-row tile list.  A segment is at most max_rows_per_expert
// long: a class that cannot occur is not launched.  When even 64-row (128-row) tiles throughout
// could not give the chip more than MI_FEW_BLOCKS blocks, one per CU (few experts, a narrow output:
// Mixtral's down product at a few hundred tokens is a few dozen 256-row blocks of 448 K steps each,
// bound by the length of a step), the larger lists are run by the smaller kernel, 2 or 4 blocks
// per tile (measured: 256 / 512 tokens of that shape -5 / -6 %; with a bound of 384 or 512 blocks
// other batch sizes gain 3 % and 512 tokens lose 6 %).
#ifndef MI_FEW_BLOCKS
#define MI_FEW_BLOCKS 256
#endif
template <int BITS, bool GLU>
static hipError_t launch_class(const GroupedArgs &a, int cls, hipStream_t st) {
  const uint32_t *const list = tile_list(a.mtiles, cls, a.max_mtiles, a.tile_cap_e);
  const int ni = GLU ? 128 : 256;
  const int64_t n_ntiles = (a.N + ni - 1) / ni;
  auto blocks_with = [&](int rows_per_tile) { return (a.total_rows / rows_per_tile + a.max_active) * n_ntiles; };
  const int mt_max = blocks_with(64) <= MI_FEW_BLOCKS ? 1 : (blocks_with(128) <= MI_FEW_BLOCKS ? 2 : 4);
  if (cls == 0) {
    if (a.max_rows_per_expert <= 128) return hipSuccess;
    if (mt_max == 1) return launch_one<BITS, GLU, 1>(a, list, a.max_mtiles, 2, st);
    if (mt_max == 2) return launch_one<BITS, GLU, 2>(a, list, a.max_mtiles, 1, st);
    return launch_one<BITS, GLU, 4>(a, list, a.max_mtiles, 0, st);
  }
  if (cls == 1) {
    if (a.max_rows_per_expert <= 64) return hipSuccess;
    if (mt_max == 1) return launch_one<BITS, GLU, 1>(a, list, a.tile_cap_e, 1, st);
    return launch_one<BITS, GLU, 2>(a, list, a.tile_cap_e, 0, st);
  }
  return launch_one<BITS, GLU, 1>(a, list, a.tile_cap_e, 0, st);
}

bool large_qmm_applies(const GroupedArgs &a) { return a.mtiles && a.tile_cap_e > 0 && a.x_perm; }

hipError_t launch_large_qmm_class(const GroupedArgs &a, bool glu, int cls, hipStream_t st) {
  if (!large_qmm_applies(a)) return hipSuccess;
  if (a.bits == 4) return glu ? launch_class<4, true>(a, cls, st) : launch_class<4, false>(a, cls, st);
  return glu ? launch_class<8, true>(a, cls, st) : launch_class<8, false>(a, cls, st);
}

hipError_t launch_large_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  for (int cls = 0; cls < 3; ++cls)
    if (hipError_t e = launch_large_qmm_class(a, glu, cls, st); e != hipSuccess) return e;
  return hipSuccess;
}

}  // namespace mi_moe
