// Grouped quantized products over expert-sorted row segments.
//
// Replaces mlx_gather_qmm (mlx-rs/src/ops/quantization.rs:160-230, transpose = true):
// for every sorted row r of expert e:  y[dst(r)] = x[src(r)] . dequantize(W[e])^T, with
// W in MLX-affine format (uint32 words, low bits first, one bf16 (scale, bias) per 64
// codes).  With GLU the gate and up products share the x operand and the epilogue
// writes silu(gate) * up (nn/activation.rs:142-144,876-880 + multiply), so neither
// product reaches memory.
//
// Arithmetic: sum_c x_c (s q_c + b) = s sum_c x_c q_c + b sum_c x_c per quantisation
// group, in fp32.  The integer codes are exact in bf16, so the matrix cores multiply raw
// codes (no per-element dequantisation, no rounding of w_hat), and scale and bias are
// applied once per group to the fp32 partial sums.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>

#include "common.hpp"

namespace mi_moe {

thread_local KernelTimer *g_kernel_timer = nullptr;
thread_local LaunchPlan *g_launch_plan = nullptr;

// the list of kernel slots: its head is constant-initialised, so slots may register in any order
// while the library's static objects are constructed
static KernelSlot *g_slot_head = nullptr;
KernelSlot *kernel_slots() { return g_slot_head; }
KernelSlot::KernelSlot(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(name, sizeof name, fmt, ap);
  va_end(ap);
  next = g_slot_head;
  g_slot_head = this;
}
void plan_note(const KernelSlot &slot, dim3 grid, dim3 block, size_t lds) {
  LaunchPlan *p = g_launch_plan;
  if (!p) return;
  ++p->n;
  if (p->out && p->len < p->cap) {
    const int w = snprintf(p->out + p->len, p->cap - p->len, "%s%s grid=%ux%u block=%u lds=%zu", p->len ? ";" : "", slot.name,
                           grid.x, grid.y, block.x, lds);
    if (w > 0) p->len = p->len + (size_t)w < p->cap ? p->len + (size_t)w : p->cap - 1;
  }
}

__device__ __forceinline__ f32x4_t mfma16(const uint32_t (&a)[4], const uint32_t (&b)[4],
                                          f32x4_t c) {
  typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
  u32x4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                 __builtin_bit_cast(bf16x8_t, bv), c, 0, 0, 0);
}

// (a & mask) | orv.  With mask and orv held in registers (see opaque_reg) this is one
// v_and_or_b32; as literals it would be two instructions (VOP3 takes no 32-bit literals).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
  return (a & mask) | orv;
}
// hide a constant from the optimiser so that it stays in a register
__device__ __forceinline__ uint32_t opaque_reg(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

__device__ __forceinline__ float silu_mul(float g, float u) {
  return g / (1.0f + __expf(-g)) * u;
}

// ---------------------------------------------------------------------------------
// Small-segment kernel (decode): one 16x16x32 MFMA tile = 16 weight rows x TT tokens.
//
// Lane l = (c = l & 15, kb = l >> 4).  B operand (weights): lane holds 8 codes of weight
// row n0+c; A operand (activations): lane holds 8 values of token slot c; D: lane holds
// D[4*kb + r][c], r = 0..3 (rows = token slots, columns = weight rows).
//
// 4-bit: a lane loads one uint4 = 32 consecutive codes, so the four lanes of a row cover
// 128 codes = two quantisation groups (kb 0,1 -> first, kb 2,3 -> second).  To keep the
// groups apart inside one MFMA, the 16 A rows are used as 2 x 8: rows 0-7 carry the TT = 8
// tokens with data only in lanes kb < 2, rows 8-15 carry the same tokens with data only in
// lanes kb >= 2.  D rows 0-7 are then the first group's sums and rows 8-15 the second's.
// A code q is fed as the bf16 value 128+q (0x4300 | q); the offset is folded into the
// bias term.  The nibbles of a word come out as pairs (q_i, q_{i+4}), the activations are
// paired the same way.
//
// 8-bit: a uint4 = 16 codes, the four lanes of a row cover one group of 64, all 16 A rows
// are tokens (TT = 16), codes are converted with v_cvt_f32_ubyte and truncated (exact).
//
// KW waves of a block split K chunk-wise (wave wk takes chunks wk, wk+KW, ...), the other
// 4/KW waves take further row tiles; partial sums meet in LDS and are added in wave order.

#ifndef MI_MOE_RING
#define MI_MOE_RING 4
#endif
#ifndef MI_MOE_RING_DEEP
#define MI_MOE_RING_DEEP 8  // chunks in flight per wave where a CU holds two blocks (registers are plentiful there)
#endif
#ifndef MI_MOE_TG2_AVG
#define MI_MOE_TG2_AVG 6   // rows per active expert from which the 4-bit gate/up kernel takes two token groups per pass
#endif
#ifndef MI_MOE_TG2_AVG_PLAIN
#define MI_MOE_TG2_AVG_PLAIN 8  // the same for plain products (short rows: a second pass costs them less)
#endif
#ifndef MI_MOE_CUS
#define MI_MOE_CUS 256  // compute units of an MI355X
#endif
#ifndef MI_MOE_SLAB_MIN
#define MI_MOE_SLAB_MIN 1024  // smallest slab (K values)
#endif
#ifndef MI_MOE_SHORT_AVG2
#define MI_MOE_SHORT_AVG2 3  // twice the rows per expert on average up to which segments count as short
#endif
#ifndef MI_MOE_SHORT_TT
#define MI_MOE_SHORT_TT 4  // token rows staged per pass at least, when segments are short on average
#endif
#ifndef MI_MOE_PRECISE_BELOW
#define MI_MOE_PRECISE_BELOW 2  // blocks per CU up to which the ring takes the unconditional form
#endif

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

// Buffer resource over [base, base + bytes): loads past the end return 0, addresses are
// a wave-uniform descriptor + a 32-bit lane offset + a scalar offset (no 64-bit VGPR math).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <int BITS, bool TWO>
struct ChunkRegs {
  static constexpr int NM = TWO ? 2 : 1;
  u32x4_t q[NM];    // packed codes of this lane's weight row
};

// LDS layout of one token tile (all offsets 16-byte aligned):
//   [0, tt*xstride + zero_bytes)  tt staged activation rows + zeros (see zero_bytes)
//   then groups x TT fp32         sum of x over each quantisation group, per token slot
//   then per wave, per tensor     the bf16 scales (and biases) of the wave's 16 weight rows: a flat
//                                 copy of 16 * K/64 values (they are contiguous in memory), or with
//                                 slabs the slab's sk/64 values of each of the 16 rows, or with K split
//                                 over the waves the values of the wave's K range (sb_range_k)
// xstride carries 16 bytes of padding so that token slots spread over the LDS banks.
__host__ __device__ constexpr int x_stride_bytes(int K) { return 2 * K + 16; }
// Zeros that lanes without a token read.  Gate/up kernel, paired tiles, 8-bit codes with K split over
// the waves (long rows, LDS decides how many blocks a CU holds): 64 bytes, read with a chunk stride of
// zero.  Plain products otherwise: a whole zero row at the common stride (the per-lane stride costs
// them 6 VGPRs, which would take the down kernel from 6 to 5 waves per SIMD).
__host__ __device__ constexpr int zero_bytes(int sk, bool glu) { return glu ? 64 : 2 * sk + 16; }
__host__ __device__ constexpr int sb_tile_bytes(int K) { return 32 * (K / 64); }  // 16 rows x K/64 bf16
// K values the scale / bias tiles in LDS cover: the whole row (fetched once, ahead of everything
// else) up to K = 4096; beyond, with slabs, the slab (a row of 14336 values has 7 KB of scales and
// biases per wave and tensor: more than the activations of a few tokens)
__host__ __device__ constexpr int sb_tile_k(int K, int sk) { return sk < K && K > 4096 ? sk : K; }
// With K split over kw waves (whole rows staged) a wave parks the scales / biases of its own K range
// only: K / kw values per row, when that range is a whole number of 16-byte pieces (512 values) of
// 16-byte aligned rows of scales and its 16 rows fit the pieces a lane holds (two with 4-bit codes: the range
// <= 4096 values; four with 8-bit codes: <= 8192).
// Returns that range, or 0: the whole row.
__host__ __device__ constexpr int sb_range_k(int K, int kw, int bits) {
  const int ch = bits == 4 ? 128 : 64, nchunks = K / ch, cpw = (nchunks + kw - 1) / kw;
  return kw > 1 && K % 512 == 0 && (cpw * ch) % 512 == 0 && cpw * ch <= (bits == 8 ? 8192 : 4096) ? cpw * ch : 0;
}
// sk: K values of the activation rows staged at a time (a slab; the whole row when sk = K)
// sbk: K values the scale / bias tiles cover when that is a wave's K range (sb_range_k), else 0
// zb: the 64-byte block of zeros, not a zero row (see zero_bytes)
__host__ __device__ constexpr size_t small_lds_bytes(int K, int sk, int tt, int TT, int n_tensors, int sbk, bool zb) {
  return (size_t)tt * x_stride_bytes(sk) + zero_bytes(sk, zb) + (size_t)(sk / 64) * TT * 4 +
         (size_t)4 * n_tensors * sb_tile_bytes(sbk > 0 && sk == K ? sbk : sb_tile_k(K, sk));
}

// The LDS layout of one instantiation, in one place: the kernel takes its offsets from here and the
// launcher asks for lds_bytes() of the very instantiation it launches, with the values it passes.
template <int BITS, bool GLU, int KW, bool SLABS, int TG, bool PAIR>
struct SmallLayout {
  static constexpr bool TWO = GLU || PAIR;                   // two weight tiles per chunk
  static constexpr bool ZB = TWO || (KW > 1 && BITS == 8);   // 64 bytes of zeros, not a zero row (zero_bytes)
  static constexpr int TT = BITS == 4 ? 8 : 16;              // token slots of one MFMA tile
  static constexpr int TTL = TT * TG;                        // token slots of one pass
  static constexpr int NTEN = TWO ? 4 : 2;                   // scale and bias tiles per wave
  // sk: K values of a token row staged at a time (K itself without slabs)
  // K values of a weight row whose scales (biases) a wave parks: its own K range, the slab, or the row
  __host__ __device__ static constexpr int sb_k(int K, int sk) {
    const int rk = SLABS ? 0 : sb_range_k(K, KW, BITS);
    return KW > 1 && rk > 0 ? rk : sb_tile_k(K, SLABS ? sk : K);
  }
  __host__ __device__ static constexpr size_t gs_offset(int sk, int tt) { return (size_t)tt * x_stride_bytes(sk) + zero_bytes(sk, ZB); }
  __host__ __device__ static constexpr size_t sb_offset(int sk, int tt) { return gs_offset(sk, tt) + (size_t)(sk / 64) * TTL * 4; }
  __host__ __device__ static constexpr size_t lds_bytes(int K, int sk, int tt) {
    return sb_offset(sk, tt) + (size_t)4 * NTEN * sb_tile_bytes(sb_k(K, sk));
  }
  // statically allocated beside it: the partial sums of a K split
  static constexpr size_t static_bytes = KW > 1 ? (size_t)KW * (4 / KW) * (TWO ? 2 : 1) * 4 * 64 * 4 + 16 : 16;
};

// PRECISE: the ring's refills are issued without a condition (chunk index clamped), so the compiler
// waits for exactly the chunk it needs and a wave really keeps D chunks in flight.  With the
// conditional refills it waits for every load in flight before each chunk; that is the faster form
// (by 2-3 %) when 16 and more waves share a CU, and several times slower when long rows leave
// room for two blocks per CU only (K = 4096: 8 KB of LDS per staged token).
// SLABS: the activation rows are staged sk K values at a time (rows too long for LDS); without it
// sk = K and the slab loop below is a single pass the compiler folds away.
// TG: token groups per pass.  A 4-bit MFMA tile holds 8 tokens (its other 8 A rows carry the same
// tokens for the chunk's second quantisation group); with TG = 2 a chunk of weights is multiplied
// with two such tiles, tokens 0-7 and 8-15 of the pass, before its ring slot is refilled: segments
// of 9 to 16 rows then take one pass over the expert's weights instead of two.
// D: chunks kept in flight per wave (ring depth).  Where a CU holds two blocks a wave may use 256
// registers, and with 8-bit codes eight chunks in flight instead of four make up for the few waves.
// PAIR (plain products): a wave takes two adjacent row tiles (32 weight rows) against the same
// activation operand, the way the gate/up kernel takes a gate and an up tile: half the blocks, each
// with twice the weights to stream for one record read, one staging and one pair of barriers.
template <int BITS, bool GLU, int KW, bool PRECISE, bool SLABS, int TG, int D, bool PAIR = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D > MI_MOE_RING ? 2 : 3, 8)))
void qmm_small_kernel(GroupedArgs a, int tt, int sk_arg) {
  static_assert(!PAIR || (!GLU && KW == 1 && !SLABS), "two row tiles per wave: plain product, whole rows, K not split");
  using L = SmallLayout<BITS, GLU, KW, SLABS, TG, PAIR>;
  constexpr bool TWO = L::TWO;  // two weight tiles per chunk
  // lanes without a token read a 64-byte block of zeros (see zero_bytes); with 4-bit codes and K split over
  // the waves (a few tokens of a 128-expert layer) the plain kernel keeps its zero row: the block costs it
  // registers and a quarter of a microsecond there
  constexpr bool ZB = L::ZB;
  static_assert(TG == 1 || (TG == 2 && BITS == 4 && KW == 1), "two token groups: 4-bit, K not split over waves");
  constexpr int NW = 4 / KW;                    // row tiles per block
  constexpr int CH = BITS == 4 ? 128 : 64;      // codes per chunk (one 16-byte load per lane)
  constexpr int XV = BITS == 4 ? 4 : 2;         // 16-byte pieces of activations per lane per chunk
  constexpr int NM = TWO ? 2 : 1;
  static_assert(D == MI_MOE_RING || PRECISE, "the deep ring goes with unconditional refills");
  using Regs = ChunkRegs<BITS, TWO>;

  // one 64-byte record says everything about this block's segment (uniform address: scalar loads)
  const uint4 *recp = reinterpret_cast<const uint4 *>(a.work) + (size_t)blockIdx.y * 4;
  const uint4 rec0 = recp[0];
  const int e = (int)rec0.x;
  const int64_t r0 = rec0.y;
  const int cnt = (int)rec0.z;
  if (cnt == 0) return;
  const bool rec_src = a.src_in_work && rec0.w != 0u;
  constexpr int TT = BITS == 4 ? 8 : 16;        // token slots of one MFMA tile
  constexpr int TTL = TT * TG;                  // token slots of one pass
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform by construction
  const int wk = wave % KW, wn = wave / KW;
  const int c = lane & 15, kb = lane >> 4;
  const int N = a.N, K = a.K;
  const int n0 = (blockIdx.x * NW + wn) * (PAIR ? 32 : 16);
  const bool tile_ok = n0 < N;
  const int n = n0 + c;  // weight row of this lane (B operand / D column); rows >= N load zeros

  const int row_bytes = K * BITS / 8;
  const int groups_per_row = K / 64;
  const int nchunks = K / CH;
  const int cpw = (nchunks + KW - 1) / KW;  // contiguous K range per wave
  const int ch0 = wk * cpw;
  const int ch1 = ch0 + cpw < nchunks ? ch0 + cpw : nchunks;

  // one descriptor per tensor of this expert
  const int64_t ebase = (int64_t)e * N;
  __amdgpu_buffer_rsrc_t wr[NM], sr[NM], br[NM];
  wr[0] = make_rsrc(a.w0 + ebase * (row_bytes / 4), (uint32_t)N * row_bytes);
  sr[0] = make_rsrc(a.s0 + ebase * groups_per_row, (uint32_t)N * groups_per_row * 2);
  br[0] = make_rsrc(a.b0 + ebase * groups_per_row, (uint32_t)N * groups_per_row * 2);
  if constexpr (GLU) {
    wr[1] = make_rsrc(a.w1 + ebase * (row_bytes / 4), (uint32_t)N * row_bytes);
    sr[1] = make_rsrc(a.s1 + ebase * groups_per_row, (uint32_t)N * groups_per_row * 2);
    br[1] = make_rsrc(a.b1 + ebase * groups_per_row, (uint32_t)N * groups_per_row * 2);
  } else if constexpr (PAIR) {  // the same tensors, 16 rows further on
    const uint32_t left = N > 16 ? (uint32_t)(N - 16) : 0u;
    wr[1] = make_rsrc(a.w0 + (ebase + 16) * (row_bytes / 4), left * row_bytes);
    sr[1] = make_rsrc(a.s0 + (ebase + 16) * groups_per_row, left * groups_per_row * 2);
    br[1] = make_rsrc(a.b0 + (ebase + 16) * groups_per_row, left * groups_per_row * 2);
  }
  const uint32_t w_voff = (uint32_t)n * row_bytes + kb * 16;  // lane kb: 16 bytes of the 64-byte chunk
  // Long rows are staged a slab of sk K values at a time (sk = K: the whole row); the weight
  // stream, its ring and the accumulators run on across the slabs.
  const int sk = SLABS ? sk_arg : K;
  const int groups_per_slab = sk / 64;
  const int sb_rk = SLABS ? 0 : sb_range_k(K, KW, BITS);  // K split over the waves: the tiles of the wave's range
  const bool sb_range = KW > 1 && sb_rk > 0;
  const bool sb_whole = !sb_range && (!SLABS || sb_tile_k(K, sk) == K);  // scale / bias tiles of the whole row
  const int sbt = sb_tile_bytes(L::sb_k(K, sk));  // bytes of one tensor's scale (bias) tile in LDS
  const int sb_groups = sb_range ? sb_rk / 64 : (sb_whole ? groups_per_row : groups_per_slab);  // per row in LDS

  // issue every global load of chunk ch into R
  auto issue = [&](int ch, Regs &R) {
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      R.q[m] = __builtin_amdgcn_raw_buffer_load_b128(wr[m], w_voff, ch * 64, 0);
    }
  };

  // The first token row this wave stages (row `wave` of the segment): its loads go out ahead of the
  // weight stream.  Loads come back in the order of issue, so behind the ring's first chunks the
  // staging would wait for those too, with nothing further in flight meanwhile.  Whole rows of up
  // to 2048 values (one 16-byte piece per lane and load, four loads).  Not in the gate/up kernel:
  // there it gains half a microsecond when the chip holds all blocks of the launch at once and
  // loses two when it does not (a block then starts while others stream; measured).
  constexpr bool PRE = !SLABS && !GLU;
  const bool pre_on = PRE && K <= 2048 && wave < cnt && wave < tt;
  uint4 pre[4];
  if (PRE && pre_on) {
    int64_t src = r0 + wave;
    if (rec_src) src = a.work[(size_t)blockIdx.y * 16 + 4 + wave];
    else if (a.src_rows) src = a.src_rows[src];
    const uint16_t *xr = a.x + src * K;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int blk = j * 64 + lane;
      pre[j] = make_uint4(0, 0, 0, 0);
      if (blk < K / 8) pre[j] = *reinterpret_cast<const uint4 *>(xr + blk * 8);
    }
  }

  // the weight stream does not depend on the tokens either
  Regs ring[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    if constexpr (PRECISE) issue(ch0 + d < nchunks ? ch0 + d : nchunks - 1, ring[d]);
    else if (ch0 + d < ch1) issue(ch0 + d, ring[d]);
  }

  // scales and biases of the wave's 16 rows: K/2 contiguous bytes per tensor, fetched with
  // fully coalesced 16-byte loads now and parked in LDS (wave-private) before the chunk loop
  constexpr int NTEN = L::NTEN;  // tensors: scales, biases (x gate, up)
  static_assert(NTEN == 2 * NM, "tiles per wave");
  constexpr int SBI = KW > 1 && BITS == 8 ? 4 : 2;  // 16-byte loads per lane per tensor kept in registers
  const uint32_t sb_goff = (uint32_t)n0 * groups_per_row * 2 + lane * 16;
  u32x4_t sbv[NTEN][SBI];
  if (KW > 1 && sb_range) {
    // 16 rows x (range / 32) bytes in 16-byte pieces, piece p = row * ppr + piece of the row
    const int ppr = sb_rk / 512;
#pragma unroll
    for (int t = 0; t < NTEN; ++t)
#pragma unroll
      for (int i = 0; i < SBI; ++i) {
        const int p = i * 64 + lane;
        if (p < 16 * ppr)
          sbv[t][i] = __builtin_amdgcn_raw_buffer_load_b128(
              (t & 1) ? br[t >> 1] : sr[t >> 1],
              (uint32_t)(n0 + p / ppr) * groups_per_row * 2 + (uint32_t)(ch0 * CH / 64) * 2 + (p % ppr) * 16, 0, 0);
      }
  } else if (sb_whole) {
#pragma unroll
    for (int t = 0; t < NTEN; ++t)
#pragma unroll
      for (int i = 0; i < SBI; ++i)
        if (i * 1024 < sbt)
          sbv[t][i] = __builtin_amdgcn_raw_buffer_load_b128((t & 1) ? br[t >> 1] : sr[t >> 1], sb_goff, i * 1024, 0);
  }

  const int xstride = x_stride_bytes(sk);
  const uint32_t nib_mask = opaque_reg(0x000f000fu), nib_magic = opaque_reg(0x43004300u);  // q -> bf16 128 + q

  extern __shared__ __align__(16) unsigned char lds[];
  unsigned char *lds_x = lds;
  float *lds_gs = reinterpret_cast<float *>(lds + L::gs_offset(sk, tt));  // [groups of the slab][TTL] sums of x
  unsigned char *lds_sb = lds + L::sb_offset(sk, tt) + wave * NTEN * sbt;

  // park the scale / bias tiles (wave-private: no barrier needed, only the wave's own wait);
  // long rows in slabs: each slab brings its own piece (see the slab loop)
  auto park_sb = [&]() __attribute__((always_inline)) {
  if (KW > 1 && sb_range) {
#pragma unroll
    for (int t = 0; t < NTEN; ++t)
#pragma unroll
      for (int i = 0; i < SBI; ++i)
        if ((i * 64 + lane) * 16 < sbt)
          *reinterpret_cast<u32x4_t *>(lds_sb + t * sbt + (i * 64 + lane) * 16) = sbv[t][i];
  } else if (sb_whole) {
#pragma unroll
    for (int t = 0; t < NTEN; ++t) {
#pragma unroll
      for (int i = 0; i < SBI; ++i)
        if (i * 1024 + lane * 16 < sbt)
          *reinterpret_cast<u32x4_t *>(lds_sb + t * sbt + i * 1024 + lane * 16) = sbv[t][i];
      for (int off = SBI * 1024 + lane * 16; off < sbt; off += 1024)  // K > 4096: the rest, synchronously
        *reinterpret_cast<u32x4_t *>(lds_sb + t * sbt + off) = __builtin_amdgcn_raw_buffer_load_b128(
            (t & 1) ? br[t >> 1] : sr[t >> 1], (uint32_t)n0 * groups_per_row * 2 + off, 0, 0);
    }
  }
  };
  if constexpr (!PRE) park_sb();
  // the scales / biases of the groups [s0 / 64, (s0 + sk) / 64) of the wave's 16 rows: sk / 32 bytes
  // per row and tensor, in 16-byte pieces (the launcher takes slabs only when rows of scales are
  // 16-byte aligned, K a multiple of 512).  Past a row's end a piece reads the next row's (or, past
  // the tensor, zeros): those values belong to no chunk.
  auto load_sb_slab = [&](int s0) __attribute__((always_inline)) {
    const int ppr = groups_per_slab / 8;  // pieces per row
#pragma unroll
    for (int t = 0; t < NTEN; ++t)
      for (int p = lane; p < 16 * ppr; p += 64) {
        const int row = p / ppr, piece = p % ppr;
        *reinterpret_cast<u32x4_t *>(lds_sb + t * sbt + p * 16) = __builtin_amdgcn_raw_buffer_load_b128(
            (t & 1) ? br[t >> 1] : sr[t >> 1],
            (uint32_t)(n0 + row) * groups_per_row * 2 + (uint32_t)(s0 / 64) * 2 + piece * 16, 0, 0);
      }
  };
  // this lane's scale / bias of the first chunk in LDS: row c, group (4-bit) kb >> 1 of the chunk's two
  const unsigned char *sbl = lds_sb + (c * sb_groups + (BITS == 4 ? (kb >> 1) : 0)) * 2;
  __shared__ float red[KW > 1 ? KW : 1][KW > 1 ? NW : 1][NM][4][KW > 1 ? 64 : 1];

  // zero block and zero group sums (slots that carry no token stay zero for the whole launch)
  for (int i = threadIdx.x; i < zero_bytes(sk, ZB) / 16; i += 256)
    *reinterpret_cast<uint4 *>(lds_x + tt * xstride + i * 16) = make_uint4(0, 0, 0, 0);
  for (int i = threadIdx.x; i < groups_per_slab * TTL / 4; i += 256)
    *reinterpret_cast<uint4 *>(lds_gs + i * 4) = make_uint4(0, 0, 0, 0);

  // the prefetched row into LDS, as stage_rows() below does it for the others
  auto put_row = [&](int ts, int b0, int sl, const uint4 (&v)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int blk = b0 + j * 64 + lane;
      const uint4 w = v[j];
      float sum = ((bf16lo_to_f32(w.x) + bf16hi_to_f32(w.x)) + (bf16lo_to_f32(w.y) + bf16hi_to_f32(w.y))) +
                  ((bf16lo_to_f32(w.z) + bf16hi_to_f32(w.z)) + (bf16lo_to_f32(w.w) + bf16hi_to_f32(w.w)));
      sum += __shfl_xor(sum, 1, kWave);
      sum += __shfl_xor(sum, 2, kWave);
      sum += __shfl_xor(sum, 4, kWave);
      if (blk < sl / 8) {
        uint4 p = w;
        if (BITS == 4 && !a.x_paired) {
          p.x = (w.x & 0xffffu) | (w.z << 16);
          p.y = (w.x >> 16) | (w.z & 0xffff0000u);
          p.z = (w.y & 0xffffu) | (w.w << 16);
          p.w = (w.y >> 16) | (w.w & 0xffff0000u);
        }
        *reinterpret_cast<uint4 *>(lds_x + ts * xstride + blk * 16) = p;
        if ((blk & 7) == 0) lds_gs[(blk >> 3) * TTL + ts] = sum;
      }
    }
  };
  if constexpr (PRE) {
    __syncthreads();  // zero fill done
    if (pre_on) put_row(wave, 0, K, pre);
    park_sb();
  }

  for (int t0 = 0; t0 < cnt; t0 += tt) {
    const int nt = cnt - t0 < tt ? cnt - t0 : tt;  // tokens of this tile

    // set after a slab has been staged (kept out of the staging's way: they cost registers there)
    const unsigned char *xl[TG];  // activation row of this lane (A operand), per token group
    int xcs[TG];                  // bytes from one chunk of it to the next (0: the zero block)
    const float *gsl;             // group sums of x for this lane's 4 D rows (token slots), first group of the slab
    f32x4_t tot[TG][NM];
    int slab_ch0 = 0;  // first chunk of the slab that is in LDS

    // one chunk: MFMAs on raw codes, then scale and bias applied to the fp32 group sums
    auto compute = [&](int ch, const Regs &R) {
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        // the groups one after the other: interleaved, both groups' activations would be live at once
        if (TG > 1 && g > 0) __builtin_amdgcn_sched_barrier(0);
        uint4 xv[XV];
#pragma unroll
        for (int i = 0; i < XV; ++i) xv[i] = *reinterpret_cast<const uint4 *>(xl[g] + (SLABS ? ch - slab_ch0 : ch) * (ZB ? xcs[g] : CH * 2) + i * 16);
        f32x4_t acc[NM];
#pragma unroll
        for (int m = 0; m < NM; ++m) acc[m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if constexpr (BITS == 4) {
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const uint32_t av[4] = {xv[s].x, xv[s].y, xv[s].z, xv[s].w};
#pragma unroll
            for (int m = 0; m < NM; ++m) {
              const uint32_t w = R.q[m][s];
              uint32_t bv[4];
              bv[0] = and_or(w, nib_mask, nib_magic);
              bv[1] = and_or(w >> 4, nib_mask, nib_magic);
              bv[2] = and_or(w >> 8, nib_mask, nib_magic);
              bv[3] = and_or(w >> 12, nib_mask, nib_magic);
              acc[m] = mfma16(av, bv, acc[m]);
            }
          }
        } else {
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const uint32_t av[4] = {xv[s].x, xv[s].y, xv[s].z, xv[s].w};
#pragma unroll
            for (int m = 0; m < NM; ++m) {
              const uint32_t wA = R.q[m][2 * s], wB = R.q[m][2 * s + 1];
              uint32_t bv[4];
              bv[0] = (__float_as_uint((float)(wA & 0xffu)) >> 16) |
                      (__float_as_uint((float)((wA >> 8) & 0xffu)) & 0xffff0000u);
              bv[1] = (__float_as_uint((float)((wA >> 16) & 0xffu)) >> 16) |
                      (__float_as_uint((float)(wA >> 24)) & 0xffff0000u);
              bv[2] = (__float_as_uint((float)(wB & 0xffu)) >> 16) |
                      (__float_as_uint((float)((wB >> 8) & 0xffu)) & 0xffff0000u);
              bv[3] = (__float_as_uint((float)((wB >> 16) & 0xffu)) >> 16) |
                      (__float_as_uint((float)(wB >> 24)) & 0xffff0000u);
              acc[m] = mfma16(av, bv, acc[m]);
            }
          }
        }
        // sum_c x_c (s (128 + q_c - 128) + b) = s * acc + (b - 128 s) * sum_c x_c   (8-bit: no offset)
        const float4 xs = *reinterpret_cast<const float4 *>(gsl + (SLABS ? ch - slab_ch0 : ch) * (BITS == 4 ? 2 : 1) * TTL + TT * g);
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          const int goff = (sb_whole ? ch : (KW > 1 && sb_range ? ch - ch0 : ch - slab_ch0)) * (BITS == 4 ? 4 : 2);
          const float sc = bf16_to_f32(*reinterpret_cast<const uint16_t *>(sbl + (2 * m) * sbt + goff));
          float bi = bf16_to_f32(*reinterpret_cast<const uint16_t *>(sbl + (2 * m + 1) * sbt + goff));
          if constexpr (BITS == 4) bi = __builtin_fmaf(-128.0f, sc, bi);
          tot[g][m][0] = __builtin_fmaf(sc, acc[m][0], __builtin_fmaf(bi, xs.x, tot[g][m][0]));
          tot[g][m][1] = __builtin_fmaf(sc, acc[m][1], __builtin_fmaf(bi, xs.y, tot[g][m][1]));
          tot[g][m][2] = __builtin_fmaf(sc, acc[m][2], __builtin_fmaf(bi, xs.z, tot[g][m][2]));
          tot[g][m][3] = __builtin_fmaf(sc, acc[m][3], __builtin_fmaf(bi, xs.w, tot[g][m][3]));
        }
      }
    };


    // staging of the K values [s0, s0 + sl) of the tile's rows
    auto stage_rows = [&](int s0, int sl) __attribute__((always_inline)) {
      // stage the slab of the tile's activation rows in LDS (4-bit: each 8-block stored as the pairs
      // (x0,x4)(x1,x5)(x2,x6)(x3,x7) the nibble unpacking produces) and the per-group sums of x.
      // Rows past nt are never read (their lanes read the zero row); their group sums are cleared
      // once per tile (nobody writes them afterwards).
      if (s0 == 0 && t0 > 0 && nt < tt)
        for (int i = threadIdx.x; i < (tt - nt) * groups_per_slab; i += 256)
          lds_gs[(i / (tt - nt)) * TTL + nt + i % (tt - nt)] = 0.f;
      // wave w stages token slots w, w+4, ...: the source row is wave-uniform (read from the
      // record through the scalar cache) and every load of a row is issued before the first use
      for (int ts = wave + (PRE && t0 == 0 && pre_on ? 4 : 0); ts < nt; ts += 4) {
        const int64_t r = r0 + t0 + ts;
        int64_t src = r;
        if (rec_src && t0 + ts < 12) src = a.work[(size_t)blockIdx.y * 16 + 4 + t0 + ts];
        else if (a.src_rows) src = a.src_rows[r];
        const uint16_t *xr = a.x + src * K + s0;
        for (int b0 = 0; b0 < sl / 8; b0 += 256) {
          uint4 v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int blk = b0 + j * 64 + lane;
            v[j] = make_uint4(0, 0, 0, 0);
            if (blk < sl / 8) v[j] = *reinterpret_cast<const uint4 *>(xr + blk * 8);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int blk = b0 + j * 64 + lane;
            const uint4 w = v[j];
            float sum = ((bf16lo_to_f32(w.x) + bf16hi_to_f32(w.x)) + (bf16lo_to_f32(w.y) + bf16hi_to_f32(w.y))) +
                        ((bf16lo_to_f32(w.z) + bf16hi_to_f32(w.z)) + (bf16lo_to_f32(w.w) + bf16hi_to_f32(w.w)));
            sum += __shfl_xor(sum, 1, kWave);
            sum += __shfl_xor(sum, 2, kWave);
            sum += __shfl_xor(sum, 4, kWave);
            if (blk < sl / 8) {
              uint4 p = w;
              if (BITS == 4 && !a.x_paired) {
                p.x = (w.x & 0xffffu) | (w.z << 16);
                p.y = (w.x >> 16) | (w.z & 0xffff0000u);
                p.z = (w.y & 0xffffu) | (w.w << 16);
                p.w = (w.y >> 16) | (w.w & 0xffff0000u);
              }
              *reinterpret_cast<uint4 *>(lds_x + ts * xstride + blk * 16) = p;
              if ((blk & 7) == 0) lds_gs[(blk >> 3) * TTL + ts] = sum;
            }
          }
        }
      }
    };
    // after a slab has been staged: where this lane reads, and (first slab) zero accumulators
    auto after_stage = [&](int s0) __attribute__((always_inline)) {
      {
        // lanes without data read zeros (gate/up: the zero block, with a chunk stride of zero)
#pragma unroll
        for (int g = 0; g < TG; ++g) {
          const int ts_l = (BITS == 4 ? (c & 7) : c) + TT * g;
          bool a_on = ts_l < nt;
          if constexpr (BITS == 4) a_on = a_on && ((kb >> 1) == (c >> 3));
          if constexpr (ZB) {
            xl[g] = a_on ? lds_x + ts_l * xstride + kb * (CH / 4) * 2 : lds_x + tt * xstride;
            xcs[g] = a_on ? CH * 2 : 0;
          } else {
            xl[g] = lds_x + (a_on ? ts_l : tt) * xstride + kb * (CH / 4) * 2;
          }
        }
        gsl = lds_gs + (BITS == 4 ? (kb >> 1) * TTL + 4 * (kb & 1) : 4 * kb);
        if (!SLABS || s0 == 0) {
#pragma unroll
          for (int g = 0; g < TG; ++g)
#pragma unroll
            for (int m = 0; m < NM; ++m) tot[g][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
      }

    };
    // the chunks [c_first, c_last) against the slab in LDS
    auto run_chunks = [&](int c_first, int c_last) __attribute__((always_inline)) {
      // D chunks in flight: slot d is refilled as soon as its chunk has been consumed.
      if constexpr (PRECISE) {
        int base = c_first;
        for (; base + D <= c_last; base += D) {
#pragma unroll
          for (int d = 0; d < D; ++d) {
            const int ch = base + d;
            compute(ch, ring[d]);
            issue(ch + D < nchunks ? ch + D : nchunks - 1, ring[d]);  // past the end: repeats of the last chunk
          }
        }
#pragma unroll
        for (int d = 0; d < D; ++d)  // fewer than D chunks left (the end of the wave's range): they sit in their slots
          if (base + d < c_last) compute(base + d, ring[d]);
      } else {
        for (int base = c_first; base < c_last; base += D) {
#pragma unroll
          for (int d = 0; d < D; ++d) {
            const int ch = base + d;
            if (ch < c_last) {
              compute(ch, ring[d]);
              if (ch + D < ch1) issue(ch + D, ring[d]);  // refill the slot just consumed
            }
          }
        }
      }
    };
    auto reprime = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if constexpr (PRECISE) issue(ch0 + d < nchunks ? ch0 + d : nchunks - 1, ring[d]);
        else if (ch0 + d < ch1) issue(ch0 + d, ring[d]);
      }
    };
    if constexpr (!SLABS) {
      if (!PRE || t0 > 0) __syncthreads();  // zero fill done / every wave is done reading the previous tile
      if (t0 > 0) reprime();
      stage_rows(0, K);
      __syncthreads();
      after_stage(0);
      run_chunks(ch0, ch1);
    } else {
      for (int s0 = 0; s0 < K; s0 += sk) {
        const int sl = K - s0 < sk ? K - s0 : sk;  // K values of this slab
        __syncthreads();  // every wave is done reading the previous slab or tile
        slab_ch0 = s0 / CH;
        if (s0 == 0 && t0 > 0) reprime();
        if (!sb_whole) load_sb_slab(s0);
        stage_rows(s0, sl);
        __syncthreads();
        after_stage(s0);
        // this wave's chunks inside the slab.  Slabs and (when K is split over the waves) the waves'
        // ranges start at multiples of D chunks, so a chunk keeps the ring slot (ch - ch0) % D.
        const int slab_ch1 = (s0 + sl) / CH;
        run_chunks(ch0 > slab_ch0 ? ch0 : slab_ch0, ch1 < slab_ch1 ? ch1 : slab_ch1);
      }
    }

    if constexpr (BITS == 4) {  // rows 8-15 (second group of each chunk) onto rows 0-7
#pragma unroll
      for (int g = 0; g < TG; ++g)
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
          for (int r = 0; r < 4; ++r) tot[g][m][r] += __shfl_xor(tot[g][m][r], 32, kWave);
    }

    // cross-wave sum over the K split, in wave order
    constexpr int LR = BITS == 4 ? 32 : 64;  // lanes that hold distinct results
    float res[TG][NM][4];
    if constexpr (KW == 1) {
#pragma unroll
      for (int g = 0; g < TG; ++g)
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
          for (int r = 0; r < 4; ++r) res[g][m][r] = tot[g][m][r];
    } else {
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wk][wn][m][r][lane] = tot[0][m][r];
      __syncthreads();
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < KW; ++w) s += red[w][wn][m][r][lane];
          res[0][m][r] = s;
        }
    }

    // epilogue: one wave per row tile writes nt x 16 outputs
    if (wk == 0 && tile_ok && lane < LR) {
#pragma unroll
      for (int g = 0; g < TG; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int slot = TT * g + (BITS == 4 ? 4 * (kb & 1) + r : 4 * kb + r);
          if (slot < nt) {
            const int64_t rr = r0 + t0 + slot;
            const int64_t dst = a.dst_rows ? (int64_t)a.dst_rows[rr] : rr;
            float v;
            if constexpr (GLU) v = silu_mul(res[g][0][r], res[g][1][r]);
            else v = res[g][0][r];
            int col = n;
            if (a.y_paired) col = (n & ~7) | ((n & 7) < 4 ? 2 * (n & 7) : 2 * ((n & 7) - 4) + 1);
            a.y[dst * N + col] = (uint16_t)(cvt_pk_bf16(v, 0.f) & 0xffffu);
            if constexpr (PAIR) {  // the second tile: the same column 16 rows on (16 keeps the paired order)
              if (n0 + 16 < N) a.y[dst * N + col + 16] = (uint16_t)(cvt_pk_bf16(res[g][1][r], 0.f) & 0xffffu);
            }
          }
        }
    }
  }
}

// A kernel gets 64 KB of dynamic LDS without asking.  More is asked for on every such launch (the
// attribute belongs to the device's copy of the kernel; the call is a table update on the host).
// An error is left for hipGetLastError() of the caller.
static bool allow_lds(const void *fn, size_t lds) {
  if (lds <= 64 * 1024) return true;
  return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess;
}

// what launch_small has chosen, handed to the one instantiation that runs it
struct LaunchChoice {
  const GroupedArgs *a;
  dim3 grid;
  size_t lds;  // the size the choice was made with
  int tt, sk;
  hipStream_t st;
};
template <int BITS, bool GLU, int KW, bool PRECISE, bool SLABS, int TG, int D, bool PAIR>
KernelSlot small_slot("qmm_small_kernel<%d,%d,%d,%d,%d,%d,%d,%d>", BITS, (int)GLU, KW, (int)PRECISE, (int)SLABS, TG, D, (int)PAIR);

template <int BITS, bool GLU, int KW, bool PRECISE, bool SLABS, int TG, int D, bool PAIR>
static hipError_t launch_small_as(const LaunchChoice &c) {
  using L = SmallLayout<BITS, GLU, KW, SLABS, TG, PAIR>;
  const GroupedArgs &a = *c.a;
  const size_t need = L::lds_bytes(a.K, SLABS ? c.sk : a.K, c.tt);
  if (need != c.lds || need + L::static_bytes > (size_t)160 * 1024 || c.tt < 1 || (!SLABS && c.sk != a.K)) return hipErrorInvalidConfiguration;
  const auto kernel = &qmm_small_kernel<BITS, GLU, KW, PRECISE, SLABS, TG, D, PAIR>;
  if (!planning() && !allow_lds(reinterpret_cast<const void *>(kernel), need)) return hipGetLastError();
  launch_kernel(small_slot<BITS, GLU, KW, PRECISE, SLABS, TG, D, PAIR>, kernel, c.grid, dim3(256), need, c.st, a, c.tt, c.sk);
  return planning() ? hipSuccess : hipGetLastError();
}

template <int BITS, bool GLU>
static hipError_t launch_small(const GroupedArgs &a, hipStream_t st) {
  constexpr int TT = BITS == 4 ? 8 : 16;  // token slots of one MFMA tile
  // split K over the 4 waves of a block when there are too few row tiles to fill the chip
  const int64_t tiles = (int64_t)(a.N / 16) * a.max_active;
  const int chunks = a.K / (BITS == 4 ? 128 : 64);
  int kw = 1;  // measured on the 128-expert layer: 2 pays below ~2000 row tiles, 4 only when nearly empty
  if (tiles < 256 && chunks >= 8) kw = 4;
  else if (tiles < (GLU ? 2048 : 1024) && chunks >= 4) kw = 2;  // (plain products: one token of the 128-expert layer is 1024 tiles, -0.5 us unsplit)
  // 4-bit, segments that can be longer than one MFMA tile's 8 tokens, and long enough on average
  // for it to matter: two token groups per pass (a 9- to 16-row segment then reads its expert's
  // weights once, not twice)
  const int64_t longest = a.max_streamed_rows > 0 && a.max_streamed_rows < a.max_rows_per_expert
                              ? a.max_streamed_rows : a.max_rows_per_expert;
  const bool two_groups = BITS == 4 && kw == 1 && longest > TT &&
                          a.total_rows >= (int64_t)(GLU ? MI_MOE_TG2_AVG : MI_MOE_TG2_AVG_PLAIN) * a.max_active;
  const int TTL = two_groups ? 2 * TT : TT;  // token slots of one pass
  // plain products with two token groups per pass: two row tiles per
  // wave (measured: the down product of the 128-expert layer at 80 to 256 tokens -2..-4 us; with
  // fewer rows per expert the same costs up to a microsecond: there more, smaller blocks win)
  bool pair = !GLU && two_groups && a.K <= 2048 && a.N % 32 == 0;
  // (the three below follow `pair`: not const, a launch that ends up with slabs gives the pairing up and sizes again)
  int n_tensors = (GLU || pair) ? 4 : 2;   // scale and bias tiles per wave in LDS
  const int sbk = sb_range_k(a.K, kw, BITS);     // K split over the waves: tiles of a wave's range only
  bool zb = GLU || pair || (kw > 1 && BITS == 8);  // a block of zeros instead of a zero row (see zero_bytes)
  int regs_blocks = (GLU || pair) ? 4 : 6;  // blocks a CU holds by registers
  // tokens staged per tile: bounded by the tile, by the longest possible segment and by LDS
  int want = TTL;
  // short segments on average: stage fewer rows where the LDS saved buys a fourth block per CU (but
  // no fewer than that takes: a segment longer than the tile reads its expert's weights again)
  if (2 * a.total_rows <= MI_MOE_SHORT_AVG2 * (int64_t)a.max_active)
    while (want > MI_MOE_SHORT_TT && 4 * small_lds_bytes(a.K, a.K, want, TTL, n_tensors, sbk, zb) > (size_t)160 * 1024) --want;
  if (longest < want) want = (int)longest;
  // Every token of a segment beyond tt costs another pass over the expert's weights, so LDS is
  // traded for occupancy only down to about twice the average segment; below that the tile keeps
  // its rows even if a CU then holds one block.  Long rows are staged in slabs of 4096, 2048 or
  // 1024 values (activations, their group sums and the scale/bias tiles all shrink with the slab);
  // the weight stream runs on across the slabs.
  const size_t lds_soft = 60 * 1024, lds_hard = 150 * 1024;  // + up to 8 KB of static LDS (K-split reduction) under the 160 KB of a CU
  const int64_t avg2 = (2 * a.total_rows + a.max_active - 1) / a.max_active;
  const int need = (int)(avg2 < 1 ? 1 : (avg2 < want ? avg2 : want));
  auto fit = [&](int slab) {
    int t = want;
    while (t > need && small_lds_bytes(a.K, slab, t, TTL, n_tensors, sbk, zb) > lds_soft) --t;
    while (t > 1 && small_lds_bytes(a.K, slab, t, TTL, n_tensors, sbk, zb) > lds_hard) --t;
    return t;
  };
  // The whole row, or the largest slab that does better, first in tokens per pass, then in blocks
  // per CU.  What counts as better in blocks (measured): nothing beyond one, if the launch has no
  // more blocks than the chip has CUs (Mixtral's down product for one token is 256 blocks: slabs
  // only cost it barriers); a third block only with up to two slabs per row (sixteen 2048-value
  // rows in two slabs of 1024: yes; 4096-value rows in four: no); a second block always.  Slabs
  // need rows of scales that are 16-byte aligned (K a multiple of 512).
  const int64_t launch_blocks = (int64_t)((a.N + 16 * (4 / kw) - 1) / (16 * (4 / kw))) * a.max_active;
  auto blocks_of = [&](int slab, int t) {
    const int b = (int)((size_t)160 * 1024 / small_lds_bytes(a.K, slab, t, TTL, n_tensors, sbk, zb));
    const int cap = launch_blocks <= MI_MOE_CUS ? 1 : (2 * slab >= a.K ? 3 : 2);
    return b < cap ? b : cap;
  };
  int sk = a.K, tt = 0;
  auto choose_slab = [&]() {
    sk = a.K;
    tt = fit(sk);
    if (a.K % 512 == 0) {
      int best_t = tt < need ? tt : need, best_b = blocks_of(sk, tt);
      for (int cand = 4096; cand >= MI_MOE_SLAB_MIN; cand /= 2) {
        if (cand >= a.K) continue;
        const int t = fit(cand), tn = t < need ? t : need, b = blocks_of(cand, t);
        if (tn > best_t || (tn == best_t && b > best_b)) {
          sk = cand;
          tt = t;
          best_t = tn;
          best_b = b;
        }
      }
    }
  };
  choose_slab();
  if (sk < a.K && pair) {
    // The paired kernel stages whole rows only.  Without it the kernel keeps a zero ROW in LDS, not the 64-byte
    // block of zeros, and two tensors' tiles per wave: the sizes are taken again for that kernel (launched with the
    // paired kernel's sizes it would address LDS past what the launch asked for and read zeros for its scales).
    pair = false;
    n_tensors = 2;
    zb = kw > 1 && BITS == 8;
    regs_blocks = 6;
    choose_slab();
  }
  const bool slabs = sk < a.K;
  size_t lds = small_lds_bytes(a.K, sk, tt, TTL, slabs ? (GLU ? 4 : 2) : n_tensors, sbk, zb);
  // with slabs a chunk's ring slot must not depend on the slab: the waves' K ranges have to start
  // at multiples of the ring depth
  const int by_lds0 = (int)((size_t)160 * 1024 / (lds > 0 ? lds : 1));
  // two blocks per CU, 8-bit codes: eight chunks in flight (Mixtral shape -2..-4 %; with 4-bit codes, twice
  // the unpacking and matrix work per byte, the same costs 8 % at 32 tokens of the Qwen3-235B shape)
  const bool deep = BITS == 8 && (by_lds0 < regs_blocks ? by_lds0 : regs_blocks) <= 2;
  // one block per CU (one token of the Mixtral shape's down product: whole rows of 14336 values): sixteen
  const int64_t grid_blocks = (int64_t)((a.N + 16 * (4 / kw) - 1) / (16 * (4 / kw))) * a.max_active;
  const bool deeper = deep && (by_lds0 <= 1 || grid_blocks <= MI_MOE_CUS) && !slabs &&
                      ((chunks + kw - 1) / kw) % (2 * MI_MOE_RING_DEEP) == 0;
  // K goes unsplit after all when slabs and the split do not line up, or when the split's extra LDS (the
  // partial sums of the waves, up to 8 KB) is what does not fit beside rows this long
  const bool split_misfit = kw > 1 && lds + 4096 * (GLU ? 2 : 1) + 16 > (size_t)160 * 1024;
  if ((sk < a.K && kw > 1 && ((chunks + kw - 1) / kw) % (deep ? MI_MOE_RING_DEEP : MI_MOE_RING) != 0) || split_misfit) {
    kw = 1;  // (and with it the zero row instead of the block of zeros)
    lds = small_lds_bytes(a.K, sk, tt, TTL, GLU ? 4 : 2, 0, GLU);
  }
  const int nw = 4 / kw;
  const int wave_rows = pair ? 32 : 16;  // weight rows per wave
  dim3 grid((unsigned)((a.N + wave_rows * nw - 1) / (wave_rows * nw)), (unsigned)a.max_active);
  // blocks a CU holds: by LDS (160 KB) and by registers (4 with the gate/up kernel, 6 otherwise)
  const int by_lds = (int)((size_t)160 * 1024 / (lds > 0 ? lds : 1));
  const bool precise = (by_lds < regs_blocks ? by_lds : regs_blocks) <= MI_MOE_PRECISE_BELOW;
  // The launch asks for the LDS of the very instantiation it starts, from that instantiation's own layout and
  // the values the kernel is given; the size the search above worked with must be that size (a launch
  // whose two sides disagree is refused: it would address LDS it did not ask for).
  const LaunchChoice ch{&a, grid, lds, tt, sk, st};
  hipError_t err = hipSuccess;
#define MI_SMALL_LAUNCH(KWV, PR, SL, TGV, DV, PAIRV) err = launch_small_as<BITS, GLU, KWV, PR, SL, TGV, DV, PAIRV>(ch)
  // Ring depth: only 8-bit codes go deeper than MI_MOE_RING (`deep`, `deeper` are false with 4-bit codes).  With
  // 8-bit codes and whole rows the unconditional ring is always a deep one (what makes it unconditional, two
  // blocks per CU or fewer, is what makes it deep); the gate/up kernel with K unsplit has no use for sixteen chunks
  // (one block per CU means rows that long are in slabs, a launch of at most one block per CU has K split).
#define MI_SMALL(KWV, TGV)                                                                      \
  do {                                                                                          \
    if constexpr (BITS == 8) {                                                                  \
      if (slabs && deep) { MI_SMALL_LAUNCH(KWV, true, true, TGV, MI_MOE_RING_DEEP, false); break; }              \
      if (slabs) { MI_SMALL_LAUNCH(KWV, true, true, TGV, MI_MOE_RING, false); break; }          \
      if (precise) {                                                                            \
        if constexpr (!(GLU && KWV == 1)) {                                                     \
          if (deeper) { MI_SMALL_LAUNCH(KWV, true, false, TGV, 2 * MI_MOE_RING_DEEP, false); break; } \
        }                                                                                       \
        MI_SMALL_LAUNCH(KWV, true, false, TGV, MI_MOE_RING_DEEP, false);                        \
        break;                                                                                  \
      }                                                                                         \
      MI_SMALL_LAUNCH(KWV, false, false, TGV, MI_MOE_RING, false);                              \
    } else {                                                                                    \
      if (slabs) MI_SMALL_LAUNCH(KWV, true, true, TGV, MI_MOE_RING, false); /* long rows: few blocks per CU anyway */ \
      else if (precise) MI_SMALL_LAUNCH(KWV, true, false, TGV, MI_MOE_RING, false);             \
      else MI_SMALL_LAUNCH(KWV, false, false, TGV, MI_MOE_RING, false);                         \
    }                                                                                           \
  } while (0)
  if constexpr (!GLU && BITS == 4) {
    if (pair) {  // (two token groups, kw = 1, whole rows)
      if (precise) MI_SMALL_LAUNCH(1, true, false, 2, MI_MOE_RING, true);
      else MI_SMALL_LAUNCH(1, false, false, 2, MI_MOE_RING, true);
      return err;
    }
  }
  if constexpr (BITS == 4) {
    if (two_groups) {
      MI_SMALL(1, 2);
      return err;
    }
  }
  if (kw == 4) MI_SMALL(4, 1);
  else if (kw == 2) MI_SMALL(2, 1);
  else MI_SMALL(1, 1);
#undef MI_SMALL_LAUNCH
#undef MI_SMALL
  return err;
}

// the streaming kernel on its own: segments the dispatch did not list as M tiles
hipError_t launch_small_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  if (a.max_active <= 0 || a.total_rows <= 0) return hipSuccess;
  if (a.bits == 4) return glu ? launch_small<4, true>(a, st) : launch_small<4, false>(a, st);
  return glu ? launch_small<8, true>(a, st) : launch_small<8, false>(a, st);
}

hipError_t launch_grouped_qmm(const GroupedArgs &a, bool glu, hipStream_t st) {
  if (a.max_active <= 0 || a.total_rows <= 0) return hipSuccess;
  // long segments (listed as M tiles by the dispatch) go to the tiled kernel, the rest below
  if (hipError_t e = launch_large_qmm(a, glu, st); e != hipSuccess) return e;
  return launch_small_qmm(a, glu, st);
}

}  // namespace mi_moe
