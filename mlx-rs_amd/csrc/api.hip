// C ABI of libmi_moe: validation, workspace carving and the launch sequence of the block.
// Declarations and the reference interfaces they replace: include/mi_moe.h.
#include "../../include/mi_moe.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <mutex>
#include <new>

#include "common.hpp"

using namespace mi_moe;

// ------------------------------------------------------------------ errors
namespace {

thread_local char g_last_error[512] = "";

// The registered handler with its data.  A failing thread takes a reference under the lock and calls
// the handler outside it, so a handler swapped meanwhile stays alive (its dtor runs when the last
// reference goes) and a handler may itself register another one.
struct Handler {
  void (*fn)(const char *, void *);
  void *data;
  void (*dtor)(void *);
  ~Handler() {
    if (dtor && data) dtor(data);
  }
};
std::mutex g_handler_lock;
std::shared_ptr<Handler> g_handler;

int fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int fail(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
  va_end(ap);
  std::shared_ptr<Handler> h;
  {
    std::lock_guard<std::mutex> g(g_handler_lock);
    h = g_handler;
  }
  if (h && h->fn) h->fn(g_last_error, h->data);
  return 1;
}

// No exception leaves an entry point: every extern "C" body is a function-try-block that ends in this.
#define MI_CATCH(name)                                                                  \
  catch (const std::exception &ex_) { return fail(name ": %s", ex_.what()); }           \
  catch (...) { return fail(name ": unknown C++ exception"); }

int hip_fail(const char *what, hipError_t e) {
  return fail("%s: %s", what, hipGetErrorString(e));
}

#define MI_HIP(call)                                   \
  do {                                                 \
    hipError_t e_ = (call);                            \
    if (e_ != hipSuccess) return hip_fail(#call, e_);  \
  } while (0)

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// the block runs on the tuned kernels with 4- or 8-bit codes in groups of 64; other group sizes and
// 2-bit codes take the plain products
bool plain_config(const mi_moe_config &c) { return c.group_size != 64 || c.bits == 2; }

int check_config(const mi_moe_config *c) {
  if (!c) return fail("config is NULL");
  if (c->bits != 2 && c->bits != 4 && c->bits != 8) return fail("bits must be 2, 4 or 8, got %d", c->bits);
  if (c->group_size != 32 && c->group_size != 64 && c->group_size != 128)
    return fail("group_size must be 32, 64 or 128, got %d", c->group_size);
  if (c->hidden <= 0 || c->hidden % 64) return fail("hidden must be a positive multiple of 64, got %d", c->hidden);
  if (c->intermediate <= 0 || c->intermediate % 64)
    return fail("intermediate must be a positive multiple of 64, got %d", c->intermediate);
  if (c->hidden % c->group_size || c->intermediate % c->group_size)
    return fail("hidden and intermediate must be multiples of group_size (%d), got %d, %d", c->group_size, c->hidden,
                c->intermediate);
  if (c->n_experts < 1 || c->n_experts > 512) return fail("n_experts must be in [1, 512], got %d", c->n_experts);
  if (c->top_k < 1 || c->top_k > c->n_experts || c->top_k > 32)
    return fail("top_k must be in [1, min(n_experts, 32)], got %d", c->top_k);
  if (c->score_mode < 0 || c->score_mode > 2) return fail("unknown score_mode %d", c->score_mode);
  if (!plain_config(*c) && c->bits == 4 && (c->hidden % 128 || c->intermediate % 128))
    return fail("4-bit weights need hidden and intermediate to be multiples of 128 (got %d, %d)", c->hidden,
                c->intermediate);
  return 0;
}

int check_qmat(const mi_moe_qmat &m, const char *name) {
  if (!m.w || !m.scales || !m.biases) return fail("%s: weight, scales and biases must be non-NULL", name);
  if (!aligned16(m.w) || !aligned16(m.scales) || !aligned16(m.biases))
    return fail("%s: pointers must be 16-byte aligned", name);
  return 0;
}

// carve consecutive 256-byte aligned regions out of a workspace; the first one starts at the next
// 256-byte boundary (every *_workspace_size reserves 256 bytes for that)
struct Carver {
  char *base;
  size_t off = 0;
  explicit Carver(void *p)
      : base(reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(p) + 255u) & ~(uintptr_t)255u)) {}
  template <typename T>
  T *take(size_t n) {
    T *p = reinterpret_cast<T *>(base + off);
    off += align_up(n * sizeof(T));
    return p;
  }
};

struct ForwardWs {
  uint16_t *logits;
  uint32_t *topk_idx;
  uint16_t *topk_w;
  uint32_t *counts, *offsets, *work, *mtiles, *perm, *inv_perm, *src_of;
  int max_mtiles;
  bool tiled;  // tile lists are built
  bool heavy;  // most rows are tiled: see heavy_batch()
  int tmr;     // segments of at least this many rows are tiled
  void *disp_scratch;
  uint16_t *hh, *y, *xperm, *xnorm;
  uint16_t *gu;  // plain products only: the gate and the up product, [P, I] each
  void *router_scratch;  // byte planes of x and of the router matrix (logits on the int8 matrix cores), or nullptr
  size_t bytes_min;      // without the byte planes: a workspace of this size makes the forward take the fp64 logits (same bits)
  size_t bytes;
};

ForwardWs carve_forward(const mi_moe_config &c, int64_t T, void *ws) {
  const int64_t P = T * c.top_k;
  Carver cv(ws);
  ForwardWs f;
  f.logits = cv.take<uint16_t>((size_t)T * c.n_experts);
  f.topk_idx = cv.take<uint32_t>((size_t)P);
  f.topk_w = cv.take<uint16_t>((size_t)P);
  f.counts = cv.take<uint32_t>(c.n_experts);
  f.offsets = cv.take<uint32_t>(c.n_experts + 1);
  f.work = cv.take<uint32_t>((size_t)c.n_experts * 16);
  // M tiles of the tiled kernel: the 256-row list holds at most P / 256 full tiles plus one
  // remainder per tiled segment (a segment is at most T rows long: no token picks an expert twice)
  // (the tiled kernel reads scales in 8-byte pieces: rows of scales must be 4-byte aligned, i.e.
  // an even number of groups per row; other shapes stay on the streaming kernel)
  const bool tiled_ok = (c.hidden / 64) % 2 == 0 && (c.intermediate / 64) % 2 == 0;
  f.tiled = tiled_ok && !plain_config(c) && tiled_batch(P, c.n_experts, c.bits);
  f.heavy = f.tiled && heavy_batch(P, c.n_experts, c.bits);
  const int tmr = f.tmr = tile_min_rows(c.bits, f.heavy);
  f.max_mtiles = f.tiled ? (int)(P / kBigTileM + (P / tmr < c.n_experts ? P / tmr : c.n_experts)) : 0;
  f.mtiles = cv.take<uint32_t>(tile_list_words(f.max_mtiles, c.n_experts));
  f.perm = cv.take<uint32_t>((size_t)P);
  f.inv_perm = cv.take<uint32_t>((size_t)P);
  f.src_of = cv.take<uint32_t>((size_t)P);
  f.disp_scratch = cv.take<char>(dispatch_workspace_bytes(c.n_experts, P));
  f.hh = cv.take<uint16_t>((size_t)P * c.intermediate);
  f.y = cv.take<uint16_t>((size_t)P * c.hidden);
  f.xperm = cv.take<uint16_t>(f.tiled && c.bits == 4 ? (size_t)T * c.hidden : 0);
  f.xnorm = cv.take<uint16_t>((size_t)T * c.hidden);  // rms_norm(x) of the residual variant
  f.gu = cv.take<uint16_t>(plain_config(c) ? 2 * (size_t)P * c.intermediate : 0);
  f.bytes_min = cv.off;
  const bool i8_router = router_logits_i8_applies(T, c.hidden, c.n_experts);  // (the last region: optional, see bytes_min)
  f.router_scratch = cv.take<char>(i8_router ? router_logits_i8_bytes(T, c.hidden, c.n_experts) : 0);
  if (!i8_router) f.router_scratch = nullptr;
  f.bytes = cv.off;
  return f;
}

}  // namespace

// Scratch of mi_moe_forward_static: the workspace a forward needs, as one array that is part of the
// library's code object.  Every GPU that loads the library holds its own copy at its own address until
// the process ends.  In host code the name is only a handle for hipGetSymbolAddress: the address a
// kernel may use is looked up once per handle (mi_moe_create, on the handle's device) and kept there.
static __device__ __align__(256) unsigned char scratch[MI_MOE_STATIC_SCRATCH_BYTES];

// Prefill-sized batches: the tile classes and the streamed segments are independent chains (gate/up then
// down over the same rows); three of the four run on side streams, forked from and joined back into the
// caller's stream by events.  The streams and events belong to the GPU, not to a handle: one set per
// device for the whole process, created by the first mi_moe_create on that device and kept until the
// process ends (a model of 48 to 94 layers would otherwise hold 150 to 280 streams on a device with a
// handful of hardware queues).  The host-side fork ... join sequence of a forward runs under the set's
// lock: an event is recorded and waited for by the same forward, never by two at once.
struct DeviceStreams {
  std::mutex lock;
  bool ready = false;
  hipStream_t side[3] = {nullptr, nullptr, nullptr};
  hipEvent_t fork = nullptr, paired = nullptr, join[3] = {nullptr, nullptr, nullptr};
};
constexpr int kMaxStreamDevices = 64;
static DeviceStreams g_device_streams[kMaxStreamDevices];
static std::atomic<int> g_side_streams_created{0};

// the set of `dev` (the current device), created on first use (default priority)
static hipError_t device_streams(int dev, DeviceStreams **out) {
  if (dev < 0 || dev >= kMaxStreamDevices) return hipErrorInvalidDevice;
  DeviceStreams &d = g_device_streams[dev];
  std::lock_guard<std::mutex> g(d.lock);
  if (!d.ready) {
    hipError_t e = hipSuccess;
    for (int i = 0; i < 3 && e == hipSuccess; ++i) {
      if (!d.side[i]) {
        e = hipStreamCreateWithFlags(&d.side[i], hipStreamNonBlocking);
        if (e == hipSuccess) g_side_streams_created.fetch_add(1);
      }
      if (e == hipSuccess && !d.join[i]) e = hipEventCreateWithFlags(&d.join[i], hipEventDisableTiming);
    }
    if (e == hipSuccess && !d.fork) e = hipEventCreateWithFlags(&d.fork, hipEventDisableTiming);
    if (e == hipSuccess && !d.paired) e = hipEventCreateWithFlags(&d.paired, hipEventDisableTiming);
    if (e != hipSuccess) return e;  // what exists is kept for the next attempt
    d.ready = true;
  }
  *out = &d;
  return hipSuccess;
}

struct mi_moe_s {
  mi_moe_config cfg;
  mi_moe_weights w;
  int device = -1;                       // the GPU that was current in mi_moe_create: counters, streams, scratch live there
  unsigned char *scratch_dev = nullptr;  // device address of `scratch` on the handle's GPU
  uint32_t *counters = nullptr;  // device: arrival counters of the fused decode router, zero at rest
  DeviceStreams *streams = nullptr;      // the device's side streams and events (not owned)
};

void destroy_handle(mi_moe_s *h) {
  if (!h) return;
  if (h->counters) (void)hipFree(h->counters);
  delete h;
}

extern "C" {

const char *mi_moe_last_error(void) { return g_last_error; }

void mi_moe_set_error_handler(void (*handler)(const char *, void *), void *data,
                              void (*dtor)(void *)) try {
  std::shared_ptr<Handler> next, old;
  if (handler || data || dtor) next = std::make_shared<Handler>(Handler{handler, data, dtor});
  {
    std::lock_guard<std::mutex> g(g_handler_lock);
    old = std::move(g_handler);
    g_handler = std::move(next);
  }
  // `old` goes here, outside the lock: its dtor runs once no failing thread still uses it
} catch (...) {
  // out of host memory: the previous handler stays
}

const char *mi_moe_version(void) { return "mi_moe 0.1 gfx950"; }

int mi_moe_create(const mi_moe_config *cfg, const mi_moe_weights *weights, mi_moe_handle *out) try {
  if (!out) return fail("create: out handle is NULL");
  if (check_config(cfg)) return 1;
  if (!weights) return fail("create: weights is NULL");
  if (!weights->router_w || !aligned16(weights->router_w))
    return fail("create: router_w must be non-NULL and 16-byte aligned");
  if (check_qmat(weights->gate, "gate") || check_qmat(weights->up, "up") || check_qmat(weights->down, "down"))
    return 1;
  mi_moe_s *h = new (std::nothrow) mi_moe_s;
  if (!h) return fail("create: out of host memory");
  h->cfg = *cfg;
  h->w = *weights;
  // the only device memory the library owns: 260 bytes of counters per handle
  const size_t cbytes = (size_t)(1 + kFusedRouterMaxTokens) * sizeof(uint32_t);
  hipError_t e = hipGetDevice(&h->device);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&h->counters), cbytes);
  if (e == hipSuccess) e = hipMemset(h->counters, 0, cbytes);
  // the device's streams and events for the independent chains of a prefill-sized forward
  if (e == hipSuccess) e = device_streams(h->device, &h->streams);
  // where the built-in scratch of mi_moe_forward_static lives on this GPU
  if (e == hipSuccess) e = hipGetSymbolAddress(reinterpret_cast<void **>(&h->scratch_dev), HIP_SYMBOL(scratch));
  if (e == hipSuccess && (!h->scratch_dev || (reinterpret_cast<uintptr_t>(h->scratch_dev) & 255u))) e = hipErrorInvalidSymbol;
  if (e != hipSuccess) {
    destroy_handle(h);
    return fail("create: device memory, streams and events of the handle: %s", hipGetErrorString(e));
  }
  *out = h;
  return 0;
} MI_CATCH("create")

int mi_moe_destroy(mi_moe_handle h) try {
  destroy_handle(h);
  return 0;
} MI_CATCH("destroy")

int mi_moe_workspace_size(const mi_moe_config *cfg, int64_t max_tokens, size_t *bytes) try {
  if (!bytes) return fail("workspace_size: bytes is NULL");
  if (check_config(cfg)) return 1;
  if (max_tokens < 0) return fail("workspace_size: negative token count");
  if (max_tokens * cfg->top_k > (int64_t)1 << 30) return fail("workspace_size: too many (token, expert) pairs");
  *bytes = carve_forward(*cfg, max_tokens, nullptr).bytes + 256;
  return 0;
} MI_CATCH("workspace_size")

// The operands of the two grouped products of a forward: gate/up (rows gathered from x by token, written
// in sorted order, SwiGLU fused) and down (rows read in sorted order, written back in (token, slot) order).
static void grouped_args(const mi_moe_config &c, const mi_moe_weights &w, const ForwardWs &f, const uint16_t *x,
                         int64_t T, GroupedArgs &a, GroupedArgs &d) {
  const int64_t P = T * c.top_k;
  const bool paired = c.bits == 4;
  a = GroupedArgs{};
  a.work = f.work;
  a.max_active = (int)(P < c.n_experts ? P : c.n_experts);
  a.mtiles = f.tiled ? f.mtiles : nullptr;
  a.max_mtiles = f.max_mtiles;
  a.tile_cap_e = f.tiled ? c.n_experts : 0;
  a.bits = c.bits;
  a.total_rows = P;
  a.max_rows_per_expert = T;  // a token picks an expert at most once
  a.max_streamed_rows = f.tiled ? f.tmr - 1 : 0;
  a.x = x;
  a.x_perm = paired ? (f.tiled ? f.xperm : nullptr) : x;
  a.x_paired = false;
  a.y_paired = paired;
  a.src_rows = f.src_of;
  a.src_in_work = true;
  a.dst_rows = nullptr;
  a.w0 = w.gate.w; a.s0 = w.gate.scales; a.b0 = w.gate.biases;
  a.w1 = w.up.w;   a.s1 = w.up.scales;   a.b1 = w.up.biases;
  a.y = f.hh;
  a.N = c.intermediate;
  a.K = c.hidden;
  d = a;
  d.x = f.hh;
  d.x_perm = f.hh;
  d.x_paired = paired;
  d.y_paired = false;
  d.src_rows = nullptr;
  d.src_in_work = false;
  d.dst_rows = f.perm;
  d.w0 = w.down.w; d.s0 = w.down.scales; d.b0 = w.down.biases;
  d.w1 = nullptr; d.s1 = d.b1 = nullptr;
  d.y = f.y;
  d.N = c.hidden;
  d.K = c.intermediate;
}

// The launch sequence of one forward.  ev: nullptr, or kStages + 1 events recorded on the
// stream before the first launch and after each stage.
// kt: nullptr, or MI_MOE_N_KERNEL_TIMES timers for the grouped-product kernels (with ev).
static int forward_impl(mi_moe_handle h, const uint16_t *x_in, int64_t T, uint16_t *out, void *workspace,
                        size_t workspace_bytes, const mi_moe_debug_out *dbg, hipStream_t st,
                        hipEvent_t *ev, const uint16_t *norm_weight = nullptr, float eps = 0.f,
                        KernelTimer *kt = nullptr) {
  const uint16_t *x = x_in;
  if (!h) return fail("forward: handle is NULL");
  if (T < 0) return fail("forward: negative token count");
  if (T == 0) return 0;
  if (!x || !out) return fail("forward: x and out must be non-NULL");
  if (!aligned16(x) || !aligned16(out)) return fail("forward: x and out must be 16-byte aligned");
  int dev = -1;
  MI_HIP(hipGetDevice(&dev));
  if (dev != h->device)
    return fail("forward: the handle was created on GPU %d, the calling thread's current GPU is %d", h->device, dev);
  const mi_moe_config &c = h->cfg;
  const int64_t P = T * c.top_k;
  if (P > (int64_t)1 << 30) return fail("forward: too many (token, expert) pairs");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return fail("forward: workspace must be non-NULL and 256-byte aligned");
  ForwardWs f = carve_forward(c, T, workspace);
  if (workspace_bytes < f.bytes_min)
    return fail("forward: workspace too small (%zu bytes, need %zu)", workspace_bytes, f.bytes);
  if (workspace_bytes < f.bytes) f.router_scratch = nullptr;  // room for everything but the byte planes: fp64 logits, same bits
  int stage = 0;
#define MI_STAGE_DONE()                                  \
  do {                                                   \
    if (ev) MI_HIP(hipEventRecord(ev[++stage], st));     \
  } while (0)
  if (ev) MI_HIP(hipEventRecord(ev[0], st));
  const bool fused_router = router_fused_applies(T, c.n_experts, c.top_k);
  if (norm_weight) {  // the block's input is rms_norm(x); x itself is added back in the combine
    if (!fused_router) MI_HIP(launch_rms_norm(x_in, norm_weight, eps, T, c.hidden, f.xnorm, st));
    x = f.xnorm;      // decode: written by the router kernel below
  }

  // 4-bit: the tiled kernel reads activations with paired 8-blocks; h is produced that way, x is copied once
  // per forward (prefill-sized T only): by the router's logits kernel, which holds every piece of x in
  // registers anyway, or by a kernel of its own (light batches pair the rows beside their streamed segments)
  const bool paired = c.bits == 4;
  const bool streamed_first = f.tiled && !f.heavy && !ev;  // light batches start their streamed segments first
  const bool pair_in_router = f.tiled && paired && !streamed_first && !fused_router && !plain_config(c) &&
                              router_logits_pairs_rows(T, c.hidden);
  if (fused_router) {
    // decode: one launch for the three stages (the stage times then all land in the first)
    MI_HIP(launch_router_fused(x_in, h->w.router_w, h->w.router_bias, norm_weight, eps, f.xnorm, T, c.hidden,
                               c.n_experts, c.top_k,
                               c.score_mode, f.logits, f.topk_idx, f.topk_w, h->counters, f.counts, f.offsets,
                               f.perm, f.inv_perm, f.src_of, f.work, f.tiled ? f.mtiles : nullptr, f.max_mtiles,
                               f.tmr, st));
    MI_STAGE_DONE();
    MI_STAGE_DONE();
    MI_STAGE_DONE();
  } else {
    // Which route the logits take (all three give the same bits).  Measured, 128 experts, hidden 2048, logits +
    // selection, us at 1024 / 2048 / 4096 / 8192 tokens: fp64 matrix cores 19.9 / 27.0 / 45.7 / 81.6; byte planes +
    // int8 product, selection apart 22.5 / 26.5 / 39.7 / 64.1; one kernel per 32 tokens (planes in LDS, selection
    // included; a block's phases follow each other, and there are T / 32 blocks) 41.3 / 41.9 / 45.2 / 49.5.
    const int64_t logit_work = T * (int64_t)c.hidden * ((c.n_experts + 127) / 128);
    const bool i8_pays = f.router_scratch && logit_work >= (int64_t)3 << 20;
    if (i8_pays && logit_work >= (int64_t)12 << 20 && router_tile_applies(T, c.hidden, c.n_experts, c.top_k)) {
      // logits and selection in one kernel (the stage times both land in the first)
      MI_HIP(launch_router_tile(x, h->w.router_w, h->w.router_bias, T, c.hidden, c.n_experts, c.top_k, c.score_mode,
                                f.logits, f.topk_idx, f.topk_w, f.router_scratch, st, pair_in_router ? f.xperm : nullptr));
      MI_STAGE_DONE();
      MI_STAGE_DONE();
    } else {
      if (i8_pays)
        MI_HIP(launch_router_logits_i8(x, h->w.router_w, h->w.router_bias, T, c.hidden, c.n_experts, f.logits,
                                       f.router_scratch, st, pair_in_router ? f.xperm : nullptr));
      else
        MI_HIP(launch_router_logits(x, h->w.router_w, h->w.router_bias, T, c.hidden, c.n_experts, f.logits, st,
                                    pair_in_router ? f.xperm : nullptr));
      MI_STAGE_DONE();
      MI_HIP(launch_router_select(f.logits, T, c.n_experts, c.top_k, c.score_mode, f.topk_idx, f.topk_w, st));
      MI_STAGE_DONE();
    }
    MI_HIP(launch_dispatch(f.topk_idx, P, c.n_experts, c.top_k, f.counts, f.offsets, f.perm, f.inv_perm,
                           f.src_of, f.work, f.tiled ? f.mtiles : nullptr, f.max_mtiles, f.tmr,
                           f.disp_scratch, st));
    MI_STAGE_DONE();
  }
  GroupedArgs a{}, d{};
  grouped_args(c, h->w, f, x, T, a, d);
  const int max_active = a.max_active;
  if (f.tiled && paired && !streamed_first && !pair_in_router) MI_HIP(launch_pair_rows(x, T, c.hidden, f.xperm, st));
  if (plain_config(c)) {
    // group sizes 32 / 128 or 2-bit codes: the plain products, one output row per sorted pair.  Row r of
    // the sorted order belongs to pair perm[r], token src_of[r], expert topk_idx[perm[r]].
    const size_t PI = (size_t)P * c.intermediate;
    MI_HIP(launch_qmm_plain(x, h->w.gate.w, h->w.gate.scales, h->w.gate.biases, f.src_of, f.topk_idx, f.perm, nullptr,
                            (uint32_t)T, (uint32_t)c.n_experts, P, 1, c.intermediate, c.hidden, c.group_size, c.bits, true, MI_MOE_DTYPE_BF16, f.gu, st));
    MI_HIP(launch_qmm_plain(x, h->w.up.w, h->w.up.scales, h->w.up.biases, f.src_of, f.topk_idx, f.perm, nullptr,
                            (uint32_t)T, (uint32_t)c.n_experts, P, 1, c.intermediate, c.hidden, c.group_size, c.bits, true, MI_MOE_DTYPE_BF16, f.gu + PI, st));
    MI_HIP(launch_swiglu(f.gu, f.gu + PI, (int64_t)PI, f.hh, st));
    MI_STAGE_DONE();
    MI_HIP(launch_qmm_plain(f.hh, h->w.down.w, h->w.down.scales, h->w.down.biases, nullptr, f.topk_idx, f.perm, f.perm,
                            0u, (uint32_t)c.n_experts, P, 1, c.hidden, c.intermediate, c.group_size, c.bits, true, MI_MOE_DTYPE_BF16, f.y, st));
    MI_STAGE_DONE();
  } else if (large_qmm_applies(a) && !ev) {
    // Four chains that share no rows: the three tile classes and the streamed segments, each
    // gate/up then down.  The short classes leave most of the chip idle when they run alone
    // (a few dozen workgroups of 64 K steps each); side by side they fill it.  The chain that is
    // expected to be the longest stays on the caller's stream and is launched first (the others
    // start a cross-stream wait later, and the join waits for them): the tile class of the average
    // segment in a heavy batch, the streamed segments of a light one (whose tile lists are empty
    // unless the routing is uneven; the copy of x with paired rows, which only the tiles read,
    // then runs on a side stream as well).
    // A segment is at most T rows long: a class that cannot occur gets no stream (a fork and a
    // join cost a few microseconds each).
    const bool exists[4] = {T > 128, T > 64, true, true};
    int n_side = 0;
    DeviceStreams &ds = *h->streams;
    std::lock_guard<std::mutex> streams_guard(ds.lock);  // until the side streams have been joined back
    MI_HIP(hipEventRecord(ds.fork, st));
    // the launches, in a function of their own: whatever happens in it, the side streams it has
    // used are joined back below (a caller must never be left with work of ours running beside
    // its stream, or with a capture that has not been joined)
    auto launch_chains = [&]() -> int {
      if (streamed_first) {
        MI_HIP(launch_small_qmm(a, true, st));
        MI_HIP(launch_small_qmm(d, false, st));
        for (int cls = 0; cls < 3; ++cls) {
          if (!exists[cls]) continue;
          hipStream_t s = ds.side[n_side++];
          if (n_side == 1) {
            MI_HIP(hipStreamWaitEvent(s, ds.fork, 0));
            if (paired) {
              MI_HIP(launch_pair_rows(x, T, c.hidden, f.xperm, s));
              MI_HIP(hipEventRecord(ds.paired, s));
            }
          } else {
            MI_HIP(hipStreamWaitEvent(s, paired ? ds.paired : ds.fork, 0));
          }
          MI_HIP(launch_large_qmm_class(a, true, cls, s));
          MI_HIP(launch_large_qmm_class(d, false, cls, s));
        }
      } else {
        // which class is the longest depends on the routing, which the host does not see; it takes
        // the class of the average segment (even routing: 320 to 2048 tokens of the 128-expert shape
        // -9 % against always leading with the 256-row class; zipf-1.1 routing: +4 to +6 % there)
        const int64_t avg_rows = P / (max_active > 0 ? max_active : 1);
        const int lead = avg_rows <= 64 ? 2 : (avg_rows <= 128 ? 1 : 0);
        // With the 256-row class in the lead (more than 128 rows per expert on average) the other three chains
        // follow each other on ONE side stream: two kernels share the chip at a time instead of four, and the
        // 256-row launches are stretched less (128-expert shape, 2560 to 8192 tokens, Zipf and even routing:
        // -1.3 to -5.5 %; Mixtral shape: no change).  With a shorter class in the lead the side chains hold most
        // of the rows and need a stream each (one stream for them at 320 to 2048 tokens, Zipf routing: +10 to +36 %).
        const bool one_side = lead == 0;
        if (one_side) {
          hipStream_t s = ds.side[n_side++];
          MI_HIP(hipStreamWaitEvent(s, ds.fork, 0));
          MI_HIP(launch_large_qmm_class(a, true, 0, st));
          MI_HIP(launch_large_qmm_class(d, false, 0, st));
          // the side stream: every gate/up launch, then every down launch (against chain after chain: -0.6 %)
          for (int cls = 1; cls <= 2; ++cls) MI_HIP(launch_large_qmm_class(a, true, cls, s));
          MI_HIP(launch_small_qmm(a, true, s));
          for (int cls = 1; cls <= 2; ++cls) MI_HIP(launch_large_qmm_class(d, false, cls, s));
          MI_HIP(launch_small_qmm(d, false, s));
          return 0;
        }
        for (int i = 0; i < 4; ++i) {
          const int chain = i == 0 ? lead : (i <= lead ? i - 1 : i);
          if (!exists[chain]) continue;
          hipStream_t s = st;
          if (i > 0) {
            s = ds.side[n_side++];
            MI_HIP(hipStreamWaitEvent(s, ds.fork, 0));
          }
          if (chain < 3) {
            MI_HIP(launch_large_qmm_class(a, true, chain, s));
            MI_HIP(launch_large_qmm_class(d, false, chain, s));
          } else {
            MI_HIP(launch_small_qmm(a, true, s));
            MI_HIP(launch_small_qmm(d, false, s));
          }
        }
      }
      return 0;
    };
    const int rc = launch_chains();
    hipError_t je = hipSuccess;
    for (int i = 0; i < n_side; ++i) {
      hipError_t e = hipEventRecord(ds.join[i], ds.side[i]);
      if (e == hipSuccess) e = hipStreamWaitEvent(st, ds.join[i], 0);
      if (e != hipSuccess && je == hipSuccess) je = e;
    }
    if (rc) return rc;
    MI_HIP(je);
  } else if (kt) {
    // one kernel after the other, each dispatch with a timer of its own: tile classes 0, 1, 2 (the
    // 256-, 128- and 64-row lists), then the streamed segments; gate/up first, then down
    struct TimerScope {  // the timer never outlives the launch it is meant for
      explicit TimerScope(KernelTimer *t) { g_kernel_timer = t; }
      ~TimerScope() { g_kernel_timer = nullptr; }
    };
    for (int half = 0; half < 2; ++half) {
      const GroupedArgs &g = half == 0 ? a : d;
      for (int cls = 0; cls < 3; ++cls) {
        TimerScope scope(&kt[4 * half + cls]);
        MI_HIP(launch_large_qmm_class(g, half == 0, cls, st));
      }
      {
        TimerScope scope(&kt[4 * half + 3]);
        MI_HIP(launch_small_qmm(g, half == 0, st));
      }
      MI_STAGE_DONE();
    }
  } else {
    MI_HIP(launch_grouped_qmm(a, true, st));
    MI_STAGE_DONE();
    MI_HIP(launch_grouped_qmm(d, false, st));
    MI_STAGE_DONE();
  }
  MI_HIP(launch_combine(f.y, f.topk_w, nullptr, T, c.top_k, c.hidden, norm_weight ? x_in : nullptr, out, st));
  MI_STAGE_DONE();
#undef MI_STAGE_DONE

  if (dbg) {
    if (dbg->topk_idx) MI_HIP(hipMemcpyAsync(dbg->topk_idx, f.topk_idx, P * 4, hipMemcpyDeviceToDevice, st));
    if (dbg->topk_w) MI_HIP(hipMemcpyAsync(dbg->topk_w, f.topk_w, P * 2, hipMemcpyDeviceToDevice, st));
    if (dbg->counts) MI_HIP(hipMemcpyAsync(dbg->counts, f.counts, c.n_experts * 4, hipMemcpyDeviceToDevice, st));
    if (dbg->offsets) MI_HIP(hipMemcpyAsync(dbg->offsets, f.offsets, (c.n_experts + 1) * 4, hipMemcpyDeviceToDevice, st));
    if (dbg->perm) MI_HIP(hipMemcpyAsync(dbg->perm, f.perm, P * 4, hipMemcpyDeviceToDevice, st));
    if (dbg->inv_perm) MI_HIP(hipMemcpyAsync(dbg->inv_perm, f.inv_perm, P * 4, hipMemcpyDeviceToDevice, st));
  }
  return 0;
}

int mi_moe_forward(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out, void *workspace,
                   size_t workspace_bytes, const mi_moe_debug_out *dbg, void *stream) try {
  return forward_impl(h, x, T, out, workspace, workspace_bytes, dbg, static_cast<hipStream_t>(stream), nullptr);
} MI_CATCH("forward")

int mi_moe_forward_static(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out,
                          const mi_moe_debug_out *dbg, void *stream) try {
  if (!h) return fail("forward_static: handle is NULL");
  if (T < 0) return fail("forward_static: negative token count");
  if (T * (int64_t)h->cfg.top_k > (int64_t)1 << 30) return fail("forward_static: too many (token, expert) pairs");
  const size_t need = carve_forward(h->cfg, T, nullptr).bytes_min;
  if (need > (size_t)MI_MOE_STATIC_SCRATCH_BYTES)
    return fail("forward_static: %lld tokens of this layer need %zu bytes of workspace, the built-in scratch holds %zu "
                "(use mi_moe_forward with a workspace of the caller's)",
                (long long)T, need, (size_t)MI_MOE_STATIC_SCRATCH_BYTES);
  // no allocation from here on: the kernels get the address looked up by mi_moe_create
  return forward_impl(h, x, T, out, h->scratch_dev, (size_t)MI_MOE_STATIC_SCRATCH_BYTES, dbg,
                      static_cast<hipStream_t>(stream), nullptr);
} MI_CATCH("forward_static")

int mi_moe_forward_residual(mi_moe_handle h, const uint16_t *x, const uint16_t *norm_weight, float eps,
                            int64_t T, uint16_t *out, void *workspace, size_t workspace_bytes,
                            const mi_moe_debug_out *dbg, void *stream) try {
  if (!norm_weight || !aligned16(norm_weight)) return fail("forward_residual: norm_weight must be non-NULL and 16-byte aligned");
  if (!(eps >= 0.f)) return fail("forward_residual: eps must be non-negative");
  if (x == out) return fail("forward_residual: out must not alias x (x is read again at the end)");
  return forward_impl(h, x, T, out, workspace, workspace_bytes, dbg, static_cast<hipStream_t>(stream), nullptr,
                      norm_weight, eps);
} MI_CATCH("forward_residual")

int mi_moe_rms_norm(const uint16_t *x, const uint16_t *weight, float eps, int64_t T, int32_t hidden,
                    uint16_t *out, void *stream) try {
  if (T < 0) return fail("rms_norm: negative row count");
  if (hidden <= 0 || hidden % 8) return fail("rms_norm: hidden must be a positive multiple of 8, got %d", hidden);
  if (!(eps >= 0.f)) return fail("rms_norm: eps must be non-negative");
  if (T == 0) return 0;
  if (!x || !weight || !out) return fail("rms_norm: x, weight and out must be non-NULL");
  if (!aligned16(x) || !aligned16(weight) || !aligned16(out)) return fail("rms_norm: pointers must be 16-byte aligned");
  MI_HIP(launch_rms_norm(x, weight, eps, T, hidden, out, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("rms_norm")

int mi_moe_forward_timed(mi_moe_handle h, const uint16_t *x, int64_t T, uint16_t *out, void *workspace,
                         size_t workspace_bytes, void *stream, float *stage_ms, float *kernel_ms) try {
  if (!stage_ms) return fail("forward_timed: stage_ms is NULL");
  for (int i = 0; i < MI_MOE_N_STAGES; ++i) stage_ms[i] = 0.f;  // what an empty batch or a failed call leaves
  hipStream_t st = static_cast<hipStream_t>(stream);
  constexpr int kEvents = MI_MOE_N_STAGES + 1 + 2 * MI_MOE_N_KERNEL_TIMES;
  hipEvent_t ev[kEvents];
  for (int i = 0; i < kEvents; ++i) {
    const hipError_t e = hipEventCreate(&ev[i]);
    if (e != hipSuccess) {
      while (--i >= 0) (void)hipEventDestroy(ev[i]);
      return hip_fail("hipEventCreate", e);
    }
  }
  KernelTimer kt[MI_MOE_N_KERNEL_TIMES];
  for (int i = 0; i < MI_MOE_N_KERNEL_TIMES; ++i) {
    kt[i].start = ev[MI_MOE_N_STAGES + 1 + 2 * i];
    kt[i].stop = ev[MI_MOE_N_STAGES + 2 + 2 * i];
  }
  int rc = forward_impl(h, x, T, out, workspace, workspace_bytes, nullptr, st, ev, nullptr, 0.f, kt);
  if (kernel_ms)
    for (int i = 0; i < MI_MOE_N_KERNEL_TIMES; ++i) kernel_ms[i] = 0.f;
  if (rc == 0 && T > 0) {
    hipError_t e = hipEventSynchronize(ev[MI_MOE_N_STAGES]);
    if (e != hipSuccess) rc = hip_fail("hipEventSynchronize", e);
    for (int i = 0; rc == 0 && i < MI_MOE_N_STAGES; ++i) {
      e = hipEventElapsedTime(&stage_ms[i], ev[i], ev[i + 1]);
      if (e != hipSuccess) rc = hip_fail("hipEventElapsedTime", e);
    }
    for (int i = 0; rc == 0 && kernel_ms && i < MI_MOE_N_KERNEL_TIMES; ++i) {
      if (!kt[i].used) continue;
      e = hipEventElapsedTime(&kernel_ms[i], kt[i].start, kt[i].stop);
      if (e != hipSuccess) rc = hip_fail("hipEventElapsedTime (kernel)", e);
    }
  }
  for (int i = 0; i < kEvents; ++i) (void)hipEventDestroy(ev[i]);
  return rc;
} MI_CATCH("forward_timed")

// ------------------------------------------------------------------ stage level

int mi_moe_route_workspace_size(int32_t n_experts, int64_t T, size_t *bytes) try {
  if (!bytes) return fail("route_workspace_size: bytes is NULL");
  if (n_experts < 1 || n_experts > 512 || T < 0) return fail("route_workspace_size: bad arguments");
  *bytes = align_up((size_t)T * n_experts * 2) + 256;
  return 0;
} MI_CATCH("route_workspace_size")

int mi_moe_route(const uint16_t *x, const uint16_t *router_w, const float *router_bias, int64_t T,
                 int32_t hidden, int32_t n_experts, int32_t top_k, int32_t score_mode,
                 uint32_t *topk_idx, uint16_t *topk_w, uint16_t *logits_out, void *workspace,
                 size_t workspace_bytes, void *stream) try {
  if (T < 0) return fail("route: negative token count");
  if (hidden <= 0 || hidden % 64) return fail("route: hidden must be a positive multiple of 64, got %d", hidden);
  if (n_experts < 1 || n_experts > 512) return fail("route: n_experts must be in [1, 512], got %d", n_experts);
  if (top_k < 1 || top_k > n_experts || top_k > 32)
    return fail("route: top_k must be in [1, min(n_experts, 32)], got %d", top_k);
  if (score_mode < 0 || score_mode > 2) return fail("route: unknown score_mode %d", score_mode);
  if (T == 0) return 0;
  if (!x || !router_w || !topk_idx || !topk_w) return fail("route: x, router_w, topk_idx and topk_w must be non-NULL");
  if (!aligned16(x) || !aligned16(router_w)) return fail("route: x and router_w must be 16-byte aligned");
  uint16_t *logits = logits_out;
  if (!logits) {
    if (!workspace || workspace_bytes < (size_t)T * n_experts * 2)
      return fail("route: workspace too small (need %zu bytes)", (size_t)T * n_experts * 2);
    logits = static_cast<uint16_t *>(workspace);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  // with room for them behind the logits, the byte planes of the integer route (same bits, see mi_moe_router_logits)
  const size_t lbytes = logits_out ? 0 : align_up((size_t)T * n_experts * 2);
  void *planes = workspace ? static_cast<char *>(workspace) + lbytes : nullptr;
  const bool roomy = workspace && router_logits_i8_applies(T, hidden, n_experts) &&
                     workspace_bytes >= lbytes + router_logits_i8_bytes(T, hidden, n_experts) + 256;
  if (roomy && router_tile_applies(T, hidden, n_experts, top_k)) {
    MI_HIP(launch_router_tile(x, router_w, router_bias, T, hidden, n_experts, top_k, score_mode, logits, topk_idx, topk_w,
                              planes, st));
    return 0;
  }
  if (roomy) MI_HIP(launch_router_logits_i8(x, router_w, router_bias, T, hidden, n_experts, logits, planes, st));
  else MI_HIP(launch_router_logits(x, router_w, router_bias, T, hidden, n_experts, logits, st));
  MI_HIP(launch_router_select(logits, T, n_experts, top_k, score_mode, topk_idx, topk_w, st));
  return 0;
} MI_CATCH("route")

int mi_moe_router_logits_workspace_size(int64_t T, int32_t hidden, int32_t n_experts, size_t *bytes) try {
  if (!bytes) return fail("router_logits_workspace_size: bytes is NULL");
  if (T < 0 || hidden <= 0 || n_experts < 1 || n_experts > 512) return fail("router_logits_workspace_size: bad arguments");
  *bytes = router_logits_i8_applies(T, hidden, n_experts) ? router_logits_i8_bytes(T, hidden, n_experts) + 256 : 256;
  return 0;
} MI_CATCH("router_logits_workspace_size")

int mi_moe_router_logits(const uint16_t *x, const uint16_t *router_w, const float *router_bias, int64_t T,
                         int32_t hidden, int32_t n_experts, uint16_t *logits, void *workspace,
                         size_t workspace_bytes, void *stream) try {
  if (T < 0) return fail("router_logits: negative token count");
  if (hidden <= 0 || hidden % 64) return fail("router_logits: hidden must be a positive multiple of 64, got %d", hidden);
  if (n_experts < 1 || n_experts > 512) return fail("router_logits: n_experts must be in [1, 512], got %d", n_experts);
  if (T == 0) return 0;
  if (!x || !router_w || !logits) return fail("router_logits: x, router_w and logits must be non-NULL");
  if (!aligned16(x) || !aligned16(router_w)) return fail("router_logits: x and router_w must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (router_logits_i8_applies(T, hidden, n_experts)) {
    const size_t need = router_logits_i8_bytes(T, hidden, n_experts) + 256;
    if (!workspace || workspace_bytes < need) return fail("router_logits: workspace too small (need %zu bytes)", need);
    MI_HIP(launch_router_logits_i8(x, router_w, router_bias, T, hidden, n_experts, logits, workspace, st));
  } else {
    MI_HIP(launch_router_logits(x, router_w, router_bias, T, hidden, n_experts, logits, st));
  }
  return 0;
} MI_CATCH("router_logits")

int mi_moe_dispatch_workspace_size(int32_t n_experts, int64_t P, size_t *bytes) try {
  if (!bytes) return fail("dispatch_workspace_size: bytes is NULL");
  if (n_experts < 1 || n_experts > 512 || P < 0) return fail("dispatch_workspace_size: bad arguments");
  // scratch + counts/offsets/active/n_active stand-ins for outputs the caller leaves NULL
  *bytes = align_up(dispatch_workspace_bytes(n_experts, P)) + 256;
  return 0;
} MI_CATCH("dispatch_workspace_size")

int mi_moe_dispatch(const uint32_t *expert_of_pair, int64_t P, int32_t n_experts, uint32_t *counts,
                    uint32_t *offsets, uint32_t *perm, uint32_t *inv_perm, void *workspace,
                    size_t workspace_bytes, void *stream) try {
  if (P < 0 || P > (int64_t)1 << 30) return fail("dispatch: pair count out of range");
  if (n_experts < 1 || n_experts > 512) return fail("dispatch: n_experts must be in [1, 512], got %d", n_experts);
  if (!perm) return fail("dispatch: perm must be non-NULL");
  if (P > 0 && !expert_of_pair) return fail("dispatch: expert_of_pair is NULL");
  size_t need = 0;
  mi_moe_dispatch_workspace_size(n_experts, P, &need);
  if (!workspace || workspace_bytes < need) return fail("dispatch: workspace too small (need %zu bytes)", need);
  Carver cv(workspace);
  void *scratch = cv.take<char>(dispatch_workspace_bytes(n_experts, P));
  hipStream_t st = static_cast<hipStream_t>(stream);
  MI_HIP(launch_dispatch(expert_of_pair, P, n_experts, 1, counts, offsets, perm, inv_perm, nullptr, nullptr,
                         nullptr, 0, 0, scratch, st));
  return 0;
} MI_CATCH("dispatch")

int mi_moe_gather_qmm_workspace_size(int32_t n_experts, int64_t n_idx, int32_t M, size_t *bytes) try {
  if (!bytes) return fail("gather_qmm_workspace_size: bytes is NULL");
  if (n_experts < 1 || n_experts > 512 || n_idx < 0 || M < 1) return fail("gather_qmm_workspace_size: bad arguments");
  const int64_t rows = n_idx * M;  // perm and the (src, dst) row maps hold one entry per output row
  *bytes = align_up(dispatch_workspace_bytes(n_experts, rows)) + 2 * align_up((size_t)(n_experts + 1) * 4) +
           align_up((size_t)n_experts * 64) + 3 * align_up((size_t)rows * 4) + 256;
  return 0;
} MI_CATCH("gather_qmm_workspace_size")

// which products the tuned kernels take; everything else goes to the plain ones
static bool tuned_shape(int32_t dtype, int32_t transpose, int32_t group_size, int32_t bits, int32_t N, int32_t K) {
  return dtype == MI_MOE_DTYPE_BF16 && transpose && group_size == 64 && (bits == 4 || bits == 8) && K % 64 == 0 &&
         (bits != 4 || K % 128 == 0) && N % 16 == 0;
}

static int check_qmm_shape(const char *who, int32_t dtype, int32_t transpose, int32_t group_size, int32_t bits,
                           int32_t N, int32_t K) {
  if (dtype != MI_MOE_DTYPE_BF16 && dtype != MI_MOE_DTYPE_F16 && dtype != MI_MOE_DTYPE_F32)
    return fail("%s: dtype must be MI_MOE_DTYPE_BF16, _F16 or _F32, got %d", who, dtype);
  if (bits != 2 && bits != 4 && bits != 8) return fail("%s: bits must be 2, 4 or 8, got %d", who, bits);
  if (group_size != 32 && group_size != 64 && group_size != 128)
    return fail("%s: group_size must be 32, 64 or 128, got %d", who, group_size);
  if (K <= 0 || N <= 0) return fail("%s: N and K must be positive, got %d, %d", who, N, K);
  // the quantised axis: K with transpose = true (w [N, K*bits/32]), N otherwise (w [K, N*bits/32])
  const int32_t q_axis = transpose ? K : N;
  if (q_axis % group_size)
    return fail("%s: %s (%d) must be a multiple of group_size (%d)", who, transpose ? "K" : "N", q_axis, group_size);
  return 0;
}

static int gather_qmm_impl(const void *x, const uint32_t *w, const void *scales, const void *biases,
                           const uint32_t *lhs_indices, const uint32_t *rhs_indices, int64_t n_idx, int64_t x_batch,
                           int32_t M, int32_t N, int32_t K, int32_t n_experts, int32_t transpose, int32_t group_size,
                           int32_t bits, int32_t dtype, void *y, void *workspace, size_t workspace_bytes,
                           void *stream) {
  if (check_qmm_shape("gather_qmm", dtype, transpose, group_size, bits, N, K)) return 1;
  if (M < 1) return fail("gather_qmm: M must be positive, got %d", M);
  if (n_experts < 1) return fail("gather_qmm: n_experts must be positive, got %d", n_experts);
  if (n_idx < 0 || n_idx * M > (int64_t)1 << 30) return fail("gather_qmm: index count out of range");
  if (n_idx == 0) return 0;
  if (!x || !w || !scales || !biases || !y) return fail("gather_qmm: x, w, scales, biases and y must be non-NULL");
  if (!rhs_indices) return fail("gather_qmm: rhs_indices is required");
  // x_batch = matrices in x (0 = not told).  Without lhs_indices index j reads x[j], so there must be n_idx of them;
  // with lhs_indices the kernels clamp an index beyond x_batch - 1 (and an expert index beyond n_experts - 1) instead
  // of following it: the rows it belongs to are then meaningless, but no memory outside the operands is read.
  if (x_batch < 0 || x_batch > (int64_t)UINT32_MAX) return fail("gather_qmm: x_batch out of range");
  if (!lhs_indices && x_batch > 0 && n_idx > x_batch)
    return fail("gather_qmm: %lld indices without lhs_indices need as many matrices in x, got %lld", (long long)n_idx,
                (long long)x_batch);
  const uint32_t n_lhs = (uint32_t)x_batch;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!tuned_shape(dtype, transpose, group_size, bits, N, K) || n_experts > 512) {  // the plain kernels, no workspace
    MI_HIP(launch_qmm_plain(x, w, scales, biases, lhs_indices, rhs_indices, nullptr, nullptr, n_lhs, (uint32_t)n_experts,
                            n_idx * M, M, N, K, group_size, bits, transpose != 0, dtype, y, st));
    return 0;
  }
  if (!aligned16(x) || !aligned16(w) || !aligned16(scales) || !aligned16(biases) || !aligned16(y))
    return fail("gather_qmm: pointers must be 16-byte aligned");
  const int64_t rows = n_idx * M;
  size_t need = 0;
  mi_moe_gather_qmm_workspace_size(n_experts, n_idx, M, &need);
  if (!workspace || workspace_bytes < need) return fail("gather_qmm: workspace too small (need %zu bytes)", need);
  Carver cv(workspace);
  void *scratch = cv.take<char>(dispatch_workspace_bytes(n_experts, rows));
  uint32_t *counts = cv.take<uint32_t>(n_experts + 1);
  uint32_t *offsets = cv.take<uint32_t>(n_experts + 1);
  uint32_t *work = cv.take<uint32_t>((size_t)n_experts * 16);
  uint32_t *perm = cv.take<uint32_t>((size_t)rows);
  uint32_t *src_rows = cv.take<uint32_t>((size_t)rows);
  uint32_t *dst_rows = cv.take<uint32_t>((size_t)rows);
  MI_HIP(launch_dispatch(rhs_indices, n_idx, n_experts, 1, counts, offsets, perm, nullptr, nullptr, work,
                         nullptr, 0, 0, scratch, st));
  MI_HIP(launch_row_maps(perm, lhs_indices, n_lhs, offsets, n_idx, M, n_experts, src_rows, dst_rows, work, st));
  GroupedArgs a{};
  a.x = static_cast<const uint16_t *>(x);
  a.src_rows = src_rows;
  a.dst_rows = dst_rows;
  a.work = work;
  a.max_active = (int)(n_idx < n_experts ? n_idx : n_experts);
  a.w0 = w; a.s0 = static_cast<const uint16_t *>(scales); a.b0 = static_cast<const uint16_t *>(biases);
  a.y = static_cast<uint16_t *>(y);
  a.N = N;
  a.K = K;
  a.bits = bits;
  a.total_rows = rows;
  a.max_rows_per_expert = rows;
  MI_HIP(launch_grouped_qmm(a, false, st));
  return 0;
}

int mi_moe_gather_qmm(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                      const uint16_t *biases, const uint32_t *lhs_indices, const uint32_t *rhs_indices,
                      int64_t n_idx, int64_t x_batch, int32_t M, int32_t N, int32_t K, int32_t n_experts,
                      int32_t transpose, int32_t group_size, int32_t bits, int32_t sorted_indices,
                      uint16_t *y, void *workspace, size_t workspace_bytes, void *stream) try {
  (void)sorted_indices;  // a hint in MLX; the segments are rebuilt here either way
  return gather_qmm_impl(x, w, scales, biases, lhs_indices, rhs_indices, n_idx, x_batch, M, N, K, n_experts, transpose,
                         group_size, bits, MI_MOE_DTYPE_BF16, y, workspace, workspace_bytes, stream);
} MI_CATCH("gather_qmm")

int mi_moe_gather_qmm_typed(const void *x, const uint32_t *w, const void *scales, const void *biases,
                            const uint32_t *lhs_indices, const uint32_t *rhs_indices, int64_t n_idx,
                            int64_t x_batch, int32_t M, int32_t N, int32_t K, int32_t n_experts,
                            int32_t transpose, int32_t group_size, int32_t bits, int32_t sorted_indices,
                            int32_t dtype, void *y, void *workspace, size_t workspace_bytes, void *stream) try {
  (void)sorted_indices;
  return gather_qmm_impl(x, w, scales, biases, lhs_indices, rhs_indices, n_idx, x_batch, M, N, K, n_experts, transpose,
                         group_size, bits, dtype, y, workspace, workspace_bytes, stream);
} MI_CATCH("gather_qmm_typed")

static size_t qmm_dense_bytes(int64_t M, int32_t K, int32_t bits, size_t *mt_words) {
  const size_t ntiles = (size_t)((M + kBigTileM - 1) / kBigTileM);
  *mt_words = tile_list_words((int)ntiles, 1);
  size_t b = 256 + 256 + 64 + *mt_words * 4 + 256;  // alignment of the base, the record, the tile lists
  if (bits == 4 && M >= tiled_avg_rows(bits)) b += (size_t)M * K * 2 + 256;
  return b;
}

int mi_moe_quantized_matmul_workspace_size(int64_t M, int32_t K, int32_t bits, size_t *bytes) try {
  if (!bytes) return fail("quantized_matmul_workspace_size: bytes is NULL");
  if (M < 0 || K <= 0 || M * (int64_t)K > (int64_t)1 << 40) return fail("quantized_matmul_workspace_size: bad sizes");
  size_t mt = 0;
  *bytes = qmm_dense_bytes(M, K, bits, &mt);
  return 0;
} MI_CATCH("quantized_matmul_workspace_size")

static int quantized_matmul_impl(const void *x, const uint32_t *w, const void *scales, const void *biases,
                                 int64_t M, int32_t N, int32_t K, int32_t transpose, int32_t group_size,
                                 int32_t bits, int32_t dtype, void *y, void *workspace, size_t workspace_bytes,
                                 void *stream) {
  if (check_qmm_shape("quantized_matmul", dtype, transpose, group_size, bits, N, K)) return 1;
  if (M < 0 || M > (int64_t)1 << 30) return fail("quantized_matmul: row count out of range");
  if (M == 0) return 0;
  if (!x || !w || !scales || !biases || !y) return fail("quantized_matmul: x, w, scales, biases and y must be non-NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!tuned_shape(dtype, transpose, group_size, bits, N, K)) {  // the plain kernels, no workspace
    MI_HIP(launch_qmm_plain(x, w, scales, biases, nullptr, nullptr, nullptr, nullptr, 0u, 1u, M, 1, N, K, group_size, bits,
                            transpose != 0, dtype, y, st));
    return 0;
  }
  if (!aligned16(x) || !aligned16(w) || !aligned16(scales) || !aligned16(biases) || !aligned16(y))
    return fail("quantized_matmul: pointers must be 16-byte aligned");
  size_t mt_words = 0;
  const size_t need = qmm_dense_bytes(M, K, bits, &mt_words);
  if (!workspace || workspace_bytes < need) return fail("quantized_matmul: workspace too small (need %zu bytes)", need);
  Carver cv(workspace);
  uint32_t *work = cv.take<uint32_t>(16);
  uint32_t *mtiles = cv.take<uint32_t>(mt_words);
  // one segment of M rows: the tiled kernel from the batch threshold on (fewer rows: streaming passes)
  const bool big = M >= tiled_avg_rows(bits) && (K / 64) % 2 == 0;
  const uint16_t *xb = static_cast<const uint16_t *>(x);
  uint16_t *xperm = (bits == 4 && big) ? cv.take<uint16_t>((size_t)M * K) : nullptr;
  const int cap256 = (int)((M + kBigTileM - 1) / kBigTileM);
  MI_HIP(launch_dense_records(M, big ? tiled_avg_rows(bits) : 0, work, mtiles, cap256, st));
  if (xperm) MI_HIP(launch_pair_rows(xb, M, K, xperm, st));
  GroupedArgs a{};
  a.x = xb;
  a.x_perm = bits == 4 ? xperm : xb;
  a.work = work;
  a.max_active = 1;
  a.mtiles = big ? mtiles : nullptr;
  a.max_mtiles = big ? cap256 : 0;
  a.tile_cap_e = big ? 1 : 0;
  a.w0 = w; a.s0 = static_cast<const uint16_t *>(scales); a.b0 = static_cast<const uint16_t *>(biases);
  a.y = static_cast<uint16_t *>(y);
  a.N = N;
  a.K = K;
  a.bits = bits;
  a.total_rows = M;
  a.max_rows_per_expert = M;
  MI_HIP(launch_grouped_qmm(a, false, st));
  return 0;
}

int mi_moe_quantized_matmul(const uint16_t *x, const uint32_t *w, const uint16_t *scales,
                            const uint16_t *biases, int64_t M, int32_t N, int32_t K, int32_t transpose,
                            int32_t group_size, int32_t bits, uint16_t *y, void *workspace,
                            size_t workspace_bytes, void *stream) try {
  return quantized_matmul_impl(x, w, scales, biases, M, N, K, transpose, group_size, bits, MI_MOE_DTYPE_BF16, y,
                               workspace, workspace_bytes, stream);
} MI_CATCH("quantized_matmul")

int mi_moe_quantized_matmul_typed(const void *x, const uint32_t *w, const void *scales, const void *biases,
                                  int64_t M, int32_t N, int32_t K, int32_t transpose, int32_t group_size,
                                  int32_t bits, int32_t dtype, void *y, void *workspace, size_t workspace_bytes,
                                  void *stream) try {
  return quantized_matmul_impl(x, w, scales, biases, M, N, K, transpose, group_size, bits, dtype, y, workspace,
                               workspace_bytes, stream);
} MI_CATCH("quantized_matmul_typed")

int mi_moe_quantized_linear_typed(const void *x, const uint32_t *w, const void *scales, const void *biases,
                                  const void *linear_bias, int64_t M, int32_t N, int32_t K, int32_t group_size,
                                  int32_t bits, int32_t dtype, void *y, void *workspace, size_t workspace_bytes,
                                  void *stream) try {
  if (quantized_matmul_impl(x, w, scales, biases, M, N, K, 1, group_size, bits, dtype, y, workspace, workspace_bytes, stream))
    return 1;
  if (linear_bias && M > 0) MI_HIP(launch_add_row_bias(y, linear_bias, M, N, dtype, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("quantized_linear_typed")

int mi_moe_swiglu(const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out, void *stream) try {
  if (n < 0) return fail("swiglu: negative element count");
  if (n == 0) return 0;
  if (!gate || !up || !out) return fail("swiglu: gate, up and out must be non-NULL");
  MI_HIP(launch_swiglu(gate, up, n, out, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("swiglu")

int mi_moe_stream_probe(const void *buf, size_t bytes, uint32_t *sink, void *stream) try {
  if (bytes == 0) return 0;
  if (bytes % 32768) return fail("stream_probe: bytes must be a multiple of 32768, got %zu", bytes);
  if (bytes > ((size_t)1 << 34)) return fail("stream_probe: at most 16 GiB, got %zu", bytes);
  if (!buf || !sink) return fail("stream_probe: buf and sink must be non-NULL");
  if (reinterpret_cast<uintptr_t>(buf) % 16) return fail("stream_probe: buf must be 16-byte aligned");
  MI_HIP(launch_stream_probe(buf, bytes, sink, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("stream_probe")

int mi_moe_combine(const uint16_t *y, const uint16_t *scores, const uint32_t *inv_perm, int64_t T,
                   int32_t top_k, int32_t hidden, uint16_t *out, void *stream) try {
  if (T < 0) return fail("combine: negative token count");
  if (top_k < 1) return fail("combine: top_k must be positive, got %d", top_k);
  if (hidden <= 0 || hidden % 8) return fail("combine: hidden must be a positive multiple of 8, got %d", hidden);
  if (T == 0) return 0;
  if (!y || !scores || !out) return fail("combine: y, scores and out must be non-NULL");
  if (!aligned16(y) || !aligned16(out)) return fail("combine: y and out must be 16-byte aligned");
  MI_HIP(launch_combine(y, scores, inv_perm, T, top_k, hidden, nullptr, out, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("combine")

static int check_quant_args(const char *who, int64_t rows, int64_t cols, int32_t group_size, int32_t bits) {
  if (bits != 2 && bits != 4 && bits != 8) return fail("%s: bits must be 2, 4 or 8, got %d", who, bits);
  if (group_size != 32 && group_size != 64 && group_size != 128)
    return fail("%s: group_size must be 32, 64 or 128, got %d", who, group_size);
  if (rows < 0 || cols < 0) return fail("%s: negative shape", who);
  if (cols % group_size) return fail("%s: columns (%lld) must be divisible by group_size (%d)", who, (long long)cols, group_size);
  return 0;
}

static int check_dtype(const char *who, int32_t dtype) {
  if (dtype != MI_MOE_DTYPE_BF16 && dtype != MI_MOE_DTYPE_F16 && dtype != MI_MOE_DTYPE_F32)
    return fail("%s: dtype must be MI_MOE_DTYPE_BF16, _F16 or _F32, got %d", who, dtype);
  return 0;
}

int mi_moe_quantize_typed(const float *w, int64_t rows, int64_t cols, int32_t group_size, int32_t bits,
                          int32_t dtype, uint32_t *q, void *scales, void *biases, void *stream) try {
  if (check_quant_args("quantize", rows, cols, group_size, bits) || check_dtype("quantize", dtype)) return 1;
  if (rows * cols == 0) return 0;
  if (!w || !q || !scales || !biases) return fail("quantize: w, q, scales and biases must be non-NULL");
  MI_HIP(launch_quantize(w, rows, cols, group_size, bits, q, scales, biases, dtype, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("quantize_typed")

int mi_moe_quantize(const float *w, int64_t rows, int64_t cols, int32_t group_size, int32_t bits,
                    uint32_t *q, uint16_t *scales, uint16_t *biases, void *stream) try {
  return mi_moe_quantize_typed(w, rows, cols, group_size, bits, MI_MOE_DTYPE_BF16, q, scales, biases, stream);
} MI_CATCH("quantize")

int mi_moe_dequantize_typed(const uint32_t *q, const void *scales, const void *biases, int64_t rows,
                            int64_t cols, int32_t group_size, int32_t bits, int32_t dtype, float *w_hat,
                            void *stream) try {
  if (check_quant_args("dequantize", rows, cols, group_size, bits) || check_dtype("dequantize", dtype)) return 1;
  if (rows * cols == 0) return 0;
  if (!q || !scales || !biases || !w_hat) return fail("dequantize: q, scales, biases and w_hat must be non-NULL");
  MI_HIP(launch_dequantize(q, scales, biases, rows, cols, group_size, bits, w_hat, dtype, false, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("dequantize_typed")

int mi_moe_dequantize_native(const uint32_t *q, const void *scales, const void *biases, int64_t rows,
                             int64_t cols, int32_t group_size, int32_t bits, int32_t dtype, void *w_hat,
                             void *stream) try {
  if (check_quant_args("dequantize", rows, cols, group_size, bits) || check_dtype("dequantize", dtype)) return 1;
  if (rows * cols == 0) return 0;
  if (!q || !scales || !biases || !w_hat) return fail("dequantize: q, scales, biases and w_hat must be non-NULL");
  MI_HIP(launch_dequantize(q, scales, biases, rows, cols, group_size, bits, w_hat, dtype, true, static_cast<hipStream_t>(stream)));
  return 0;
} MI_CATCH("dequantize_native")

int mi_moe_dequantize(const uint32_t *q, const uint16_t *scales, const uint16_t *biases, int64_t rows,
                      int64_t cols, int32_t group_size, int32_t bits, float *w_hat, void *stream) try {
  return mi_moe_dequantize_typed(q, scales, biases, rows, cols, group_size, bits, MI_MOE_DTYPE_BF16, w_hat, stream);
} MI_CATCH("dequantize")

// ------------------------------------------------------------------ introspection (no counterpart in the reference)

int32_t mi_moe_debug_kernel_count(void) {
  int32_t n = 0;
  for (const KernelSlot *s = kernel_slots(); s; s = s->next) ++n;
  return n;
}

const char *mi_moe_debug_kernel_name(int32_t index) {
  int32_t i = 0;
  for (KernelSlot *s = kernel_slots(); s; s = s->next, ++i)
    if (i == index) return s->name;
  return nullptr;
}

int64_t mi_moe_debug_kernel_launches(int32_t index) {
  int32_t i = 0;
  for (KernelSlot *s = kernel_slots(); s; s = s->next, ++i)
    if (i == index) return (int64_t)__atomic_load_n(&s->launches, __ATOMIC_RELAXED);
  return -1;
}

namespace {
// nothing is launched while one of these lives on the calling thread: launch_kernel writes to `plan` instead
struct PlanScope {
  LaunchPlan plan;
  PlanScope(char *out, size_t cap) : plan{out, cap} {
    if (out && cap) out[0] = 0;
    g_launch_plan = &plan;
  }
  ~PlanScope() { g_launch_plan = nullptr; }
};
}  // namespace

int mi_moe_debug_plan_grouped(int32_t N, int32_t K, int32_t bits, int32_t glu, int64_t total_rows, int32_t max_active,
                              int64_t max_rows_per_expert, int64_t max_streamed_rows, int32_t tile_lists,
                              int32_t paired_out, char *out, size_t cap) try {
  if (bits != 4 && bits != 8) return fail("debug_plan_grouped: the tuned kernels take 4- or 8-bit codes, got %d", bits);
  if (N <= 0 || K <= 0 || K % 64 || (bits == 4 && K % 128) || N % 16)
    return fail("debug_plan_grouped: N must be a multiple of 16, K of 64 (4-bit: 128), got %d, %d", N, K);
  if (total_rows < 0 || max_active < 0 || max_rows_per_expert < 0 || max_streamed_rows < 0) return fail("debug_plan_grouped: negative count");
  static const uint32_t dummy[4] = {0, 0, 0, 0};  // never read: nothing is launched
  GroupedArgs a{};
  a.x = a.x_perm = reinterpret_cast<const uint16_t *>(dummy);
  a.work = dummy;
  a.w0 = a.w1 = dummy;
  a.N = N; a.K = K; a.bits = bits;
  a.total_rows = total_rows;
  a.max_active = max_active;
  a.max_rows_per_expert = max_rows_per_expert;
  a.max_streamed_rows = max_streamed_rows;
  a.y_paired = paired_out != 0;
  if (tile_lists) {
    a.mtiles = dummy;
    a.max_mtiles = (int)(total_rows / kBigTileM + max_active);
    a.tile_cap_e = max_active;
  }
  PlanScope scope(out, cap);
  MI_HIP(launch_grouped_qmm(a, glu != 0, nullptr));
  return 0;
} MI_CATCH("debug_plan_grouped")

int mi_moe_debug_plan_forward(const mi_moe_config *cfg, int64_t T, char *out, size_t cap) try {
  if (check_config(cfg)) return 1;
  if (T < 1 || T * cfg->top_k > (int64_t)1 << 30) return fail("debug_plan_forward: token count out of range");
  if (plain_config(*cfg)) {
    if (out && cap) out[0] = 0;
    return 0;  // the plain products: none of the listed kernels
  }
  const ForwardWs f = carve_forward(*cfg, T, reinterpret_cast<void *>(uintptr_t{256}));
  mi_moe_weights w{};
  GroupedArgs a{}, d{};
  grouped_args(*cfg, w, f, reinterpret_cast<const uint16_t *>(uintptr_t{256}), T, a, d);
  PlanScope scope(out, cap);
  MI_HIP(launch_grouped_qmm(a, true, nullptr));
  MI_HIP(launch_grouped_qmm(d, false, nullptr));
  return 0;
} MI_CATCH("debug_plan_forward")

int mi_moe_debug_tile_rule(const mi_moe_config *cfg, int64_t T, int32_t *tiled, int32_t *tile_min_rows) try {
  if (check_config(cfg)) return 1;
  if (T < 0 || T * cfg->top_k > (int64_t)1 << 30) return fail("debug_tile_rule: token count out of range");
  const ForwardWs f = carve_forward(*cfg, T, nullptr);
  if (tiled) *tiled = f.tiled ? 1 : 0;
  if (tile_min_rows) *tile_min_rows = f.tmr;
  return 0;
} MI_CATCH("debug_tile_rule")

int32_t mi_moe_debug_side_streams_created(void) { return g_side_streams_created.load(); }

}  // extern "C"
