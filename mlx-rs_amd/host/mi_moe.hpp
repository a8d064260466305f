// mi_moe.hpp -- header-only C++17 host layer over the C ABI of libmi_moe (include/mi_moe.h).
//
// It mirrors, for the quantized mixture-of-experts path only, the surface an mlx-rs user
// programs against:
//   Array                      a typed, shaped device buffer (mlx-rs/src/array/mod.rs:384-403)
//   Exception / Result<T>      every operation returns a value or the library's message,
//                              never throws on its own (mlx-rs/src/error.rs:226-280,
//                              utils/guard.rs:20-49); Result::unwrap() throws for callers
//                              who want exceptions
//   ops::quantize / dequantize / gather_qmm
//                              same argument order, optionals and defaults as
//                              mlx-rs/src/ops/quantization.rs:50-83,124-158,160-230
//   nn::SparseMoeBlock         forward(const Array&) -> Result<Array>, training_mode(bool):
//                              the Module<&Array> contract, mlx-rs/src/module/module.rs:28-50
// All arithmetic happens in libmi_moe.so; this file owns memory, shapes and error plumbing.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <memory>
#include <numeric>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <algorithm>
#include <utility>
#include <variant>
#include <vector>

#include "mi_moe.h"

namespace mi_moe {

class Exception : public std::runtime_error {
 public:
  explicit Exception(const std::string &what) : std::runtime_error(what) {}
  static Exception custom(const std::string &what) { return Exception(what); }
};

template <class T>
class Result {
 public:
  Result(T v) : v_(std::move(v)) {}
  Result(Exception e) : v_(std::move(e)) {}
  bool is_ok() const { return v_.index() == 0; }
  bool is_err() const { return !is_ok(); }
  const Exception &error() const { return std::get<1>(v_); }
  T &value() { return std::get<0>(v_); }
  const T &value() const { return std::get<0>(v_); }
  T unwrap() {
    if (is_err()) throw error();
    return std::move(std::get<0>(v_));
  }

 private:
  std::variant<T, Exception> v_;
};

struct Unit {};

namespace detail {
inline Exception last_error(const char *who) {
  return Exception(std::string(who) + ": " + mi_moe_last_error());
}
inline Exception hip_error(const char *who, hipError_t e) {
  return Exception(std::string(who) + ": " + hipGetErrorString(e));
}
}  // namespace detail

enum class Dtype { Bfloat16, Float16, Float32, Uint32 };
inline size_t size_of(Dtype d) { return d == Dtype::Bfloat16 || d == Dtype::Float16 ? 2 : 4; }

struct Stream {
  hipStream_t handle = nullptr;  // nullptr = the default stream
  void *as_ptr() const { return static_cast<void *>(handle); }
};

// A contiguous row-major device buffer with shape and dtype.  Copies share the allocation.
class Array {
 public:
  Array() = default;
  static Result<Array> empty(std::vector<int64_t> shape, Dtype dtype) {
    Array a;
    a.shape_ = std::move(shape);
    a.dtype_ = dtype;
    const size_t bytes = a.nbytes();
    void *p = nullptr;
    if (bytes) {
      if (hipError_t e = hipMalloc(&p, bytes); e != hipSuccess)
        return detail::hip_error("Array::empty", e);
    }
    a.mem_ = std::shared_ptr<void>(p, [](void *q) { if (q) (void)hipFree(q); });
    return a;
  }
  // a view of memory somebody else owns (e.g. a tensor of the embedding framework)
  static Array from_device_ptr(void *p, std::vector<int64_t> shape, Dtype dtype) {
    Array a;
    a.shape_ = std::move(shape);
    a.dtype_ = dtype;
    a.mem_ = std::shared_ptr<void>(p, [](void *) {});
    return a;
  }
  static Result<Array> from_host(const void *src, std::vector<int64_t> shape, Dtype dtype,
                                 Stream s = {}) {
    auto r = empty(std::move(shape), dtype);
    if (r.is_err()) return r;
    if (size_t n = r.value().nbytes()) {
      if (hipError_t e = hipMemcpyAsync(r.value().data(), src, n, hipMemcpyHostToDevice, s.handle);
          e != hipSuccess)
        return detail::hip_error("Array::from_host", e);
      if (hipError_t e = hipStreamSynchronize(s.handle); e != hipSuccess)
        return detail::hip_error("Array::from_host", e);
    }
    return r;
  }
  // eval + copy out, the counterpart of Array::as_slice
  Result<Unit> to_host(void *dst, Stream s = {}) const {
    if (hipError_t e = hipMemcpyAsync(dst, data(), nbytes(), hipMemcpyDeviceToHost, s.handle);
        e != hipSuccess)
      return detail::hip_error("Array::to_host", e);
    if (hipError_t e = hipStreamSynchronize(s.handle); e != hipSuccess)
      return detail::hip_error("Array::to_host", e);
    return Unit{};
  }
  const std::vector<int64_t> &shape() const { return shape_; }
  int64_t dim(int i) const { return shape_[i < 0 ? shape_.size() + i : i]; }
  size_t ndim() const { return shape_.size(); }
  Dtype dtype() const { return dtype_; }
  int64_t size() const {
    return std::accumulate(shape_.begin(), shape_.end(), (int64_t)1, std::multiplies<int64_t>());
  }
  size_t nbytes() const { return (size_t)size() * size_of(dtype_); }
  void *data() const { return mem_.get(); }
  template <class T> T *ptr() const { return static_cast<T *>(mem_.get()); }
  Array reshape(std::vector<int64_t> shape) const {
    Array a = *this;
    a.shape_ = std::move(shape);
    return a;
  }

 private:
  std::vector<int64_t> shape_;
  Dtype dtype_ = Dtype::Bfloat16;
  std::shared_ptr<void> mem_;
};

namespace detail {
inline std::optional<Exception> want(const Array &a, Dtype d, const char *who, const char *name) {
  if (a.dtype() != d) return Exception(std::string(who) + ": " + name + " has the wrong dtype");
  return std::nullopt;
}
}  // namespace detail

namespace ops {

constexpr int32_t DEFAULT_GROUP_SIZE = 64;  // mlx-rs/src/ops/quantization.rs:13-14
constexpr int32_t DEFAULT_BITS = 4;

// quantize(w, group_size, bits) -> (w_q, scales, biases); w: f32 [rows, cols]
inline Result<std::tuple<Array, Array, Array>> quantize(const Array &w,
                                                         std::optional<int32_t> group_size = {},
                                                         std::optional<int32_t> bits = {},
                                                         Stream s = {}) {
  const int32_t g = group_size.value_or(DEFAULT_GROUP_SIZE), b = bits.value_or(DEFAULT_BITS);
  if (auto e = detail::want(w, Dtype::Float32, "quantize", "w")) return *e;
  if (w.ndim() != 2) return Exception("quantize: w must be a matrix");
  const int64_t rows = w.dim(0), cols = w.dim(1);
  // let the library judge the arguments before anything is allocated
  if (g <= 0 || cols % g || (b != 2 && b != 4 && b != 8) || (g != 32 && g != 64 && g != 128)) {
    if (mi_moe_quantize(nullptr, rows, cols, g, b, nullptr, nullptr, nullptr, nullptr))
      return detail::last_error("quantize");
  }
  auto q = Array::empty({rows, cols * b / 32}, Dtype::Uint32);
  auto sc = Array::empty({rows, cols / g}, Dtype::Bfloat16);
  auto bi = Array::empty({rows, cols / g}, Dtype::Bfloat16);
  if (q.is_err()) return q.error();
  if (sc.is_err()) return sc.error();
  if (bi.is_err()) return bi.error();
  if (mi_moe_quantize(w.ptr<float>(), rows, cols, g, b, q.value().ptr<uint32_t>(),
                      sc.value().ptr<uint16_t>(), bi.value().ptr<uint16_t>(), s.as_ptr()))
    return detail::last_error("quantize");
  return std::make_tuple(q.value(), sc.value(), bi.value());
}

// dequantize(w, scales, biases, group_size, bits) -> f32 [rows, cols]
inline Result<Array> dequantize(const Array &w, const Array &scales, const Array &biases,
                                std::optional<int32_t> group_size = {},
                                std::optional<int32_t> bits = {}, Stream s = {}) {
  const int32_t g = group_size.value_or(DEFAULT_GROUP_SIZE), b = bits.value_or(DEFAULT_BITS);
  if (auto e = detail::want(w, Dtype::Uint32, "dequantize", "w")) return *e;
  if (auto e = detail::want(scales, Dtype::Bfloat16, "dequantize", "scales")) return *e;
  if (auto e = detail::want(biases, Dtype::Bfloat16, "dequantize", "biases")) return *e;
  if (w.ndim() != 2 || (b != 2 && b != 4 && b != 8)) {
    if (mi_moe_dequantize(nullptr, nullptr, nullptr, 1, 64, g, b, nullptr, nullptr))
      return detail::last_error("dequantize");
    return Exception("dequantize: w must be a matrix");
  }
  const int64_t rows = w.dim(0), cols = w.dim(1) * 32 / b;
  auto out = Array::empty({rows, cols}, Dtype::Float32);
  if (out.is_err()) return out;
  if (mi_moe_dequantize(w.ptr<uint32_t>(), scales.ptr<uint16_t>(), biases.ptr<uint16_t>(), rows,
                        cols, g, b, out.value().ptr<float>(), s.as_ptr()))
    return detail::last_error("dequantize");
  return out;
}

// quantized_matmul(x, w, scales, biases, transpose, group_size, bits): x bf16 [M, K]; w u32
// [N, K*bits/32] with transpose = true, [K, N*bits/32] without; scales and biases [N, K/group_size] /
// [K, N/group_size]; returns bf16 [M, N].  transpose defaults to false as in the reference
// (mlx-rs/src/ops/quantization.rs:101); QuantizedLinear passes true (nn/quantized.rs:363-386).
// The operand shapes are checked against each other before anything is launched.
inline Result<Array> quantized_matmul(const Array &x, const Array &w, const Array &scales,
                                      const Array *biases = nullptr, std::optional<bool> transpose = {},
                                      std::optional<int32_t> group_size = {},
                                      std::optional<int32_t> bits = {}, Stream s = {}) {
  const bool tr = transpose.value_or(false);
  const int32_t g = group_size.value_or(DEFAULT_GROUP_SIZE), b = bits.value_or(DEFAULT_BITS);
  if (auto e = detail::want(x, Dtype::Bfloat16, "quantized_matmul", "x")) return *e;
  if (auto e = detail::want(w, Dtype::Uint32, "quantized_matmul", "w")) return *e;
  if (auto e = detail::want(scales, Dtype::Bfloat16, "quantized_matmul", "scales")) return *e;
  if (!biases) return Exception("quantized_matmul: biases are required in affine mode");
  if (x.ndim() != 2 || w.ndim() != 2) return Exception("quantized_matmul: x must be [M, K] and w [N, K*bits/32]");
  if (auto e = detail::want(*biases, Dtype::Bfloat16, "quantized_matmul", "biases")) return *e;
  const int64_t M = x.dim(0);
  if (b != 2 && b != 4 && b != 8) return Exception("quantized_matmul: bits must be 2, 4 or 8");
  if (g != 32 && g != 64 && g != 128) return Exception("quantized_matmul: group_size must be 32, 64 or 128");
  const int32_t K = (int32_t)x.dim(1), N = tr ? (int32_t)w.dim(0) : (int32_t)(w.dim(1) * 32 / b);
  const int64_t w_k = tr ? w.dim(1) * 32 / b : w.dim(0);
  if (w_k != K)
    return Exception("quantized_matmul: x has K = " + std::to_string(K) + ", w has K = " + std::to_string(w_k) +
                     (tr ? " (transpose = true)" : " (transpose = false)"));
  const int64_t q_rows = tr ? N : K, q_axis = tr ? K : N;
  if (q_axis % g == 0 && (scales.ndim() != 2 || biases->ndim() != 2 || scales.dim(0) != q_rows || scales.dim(1) != q_axis / g ||
                          biases->dim(0) != q_rows || biases->dim(1) != q_axis / g))
    return Exception("quantized_matmul: scales and biases must be [" + std::to_string(q_rows) + ", " +
                     std::to_string(q_axis / g) + "]");
  size_t ws_bytes = 0;
  if (mi_moe_quantized_matmul_workspace_size(M, K, b, &ws_bytes)) return detail::last_error("quantized_matmul");
  auto ws = Array::empty({(int64_t)(ws_bytes + 256 + 3) / 4}, Dtype::Uint32);
  auto y = Array::empty({M, (int64_t)N}, Dtype::Bfloat16);
  if (ws.is_err()) return ws;
  if (y.is_err()) return y;
  if (mi_moe_quantized_matmul(x.ptr<uint16_t>(), w.ptr<uint32_t>(), scales.ptr<uint16_t>(),
                              biases->ptr<uint16_t>(), M, N, K, tr ? 1 : 0, g, b, y.value().ptr<uint16_t>(),
                              ws.value().data(), ws.value().nbytes(), s.as_ptr()))
    return detail::last_error("quantized_matmul");
  if (hipError_t e = hipStreamSynchronize(s.handle); e != hipSuccess)
    return detail::hip_error("quantized_matmul", e);
  return y;
}

// the library's code of a floating element type, or -1
inline int32_t float_code(Dtype d) {
  return d == Dtype::Bfloat16 ? MI_MOE_DTYPE_BF16 : d == Dtype::Float16 ? MI_MOE_DTYPE_F16
       : d == Dtype::Float32 ? MI_MOE_DTYPE_F32 : -1;
}

namespace idx {
// index array `a` (or, when absent, 0, 1, ... in the shape `counted`) on the host, with its shape
inline Result<std::pair<std::vector<uint32_t>, std::vector<int64_t>>> host_indices(const Array *a,
                                                                                  const std::vector<int64_t> &counted,
                                                                                  Stream s) {
  std::pair<std::vector<uint32_t>, std::vector<int64_t>> r;
  if (a) {
    if (a->dtype() != Dtype::Uint32) return Exception("gather_qmm: index arrays must be uint32");
    r.first.resize((size_t)a->size());
    r.second = a->shape();
    if (a->size()) {
      auto c = a->to_host(r.first.data(), s);
      if (c.is_err()) return c.error();
    }
  } else {
    int64_t n = 1;
    for (int64_t d : counted) n *= d;
    r.first.resize((size_t)n);
    std::iota(r.first.begin(), r.first.end(), 0u);
    r.second = counted;
  }
  return r;
}
// numpy-style broadcast of two shapes (aligned at the last axis); empty optional: they do not broadcast
inline std::optional<std::vector<int64_t>> broadcast_shape(const std::vector<int64_t> &a, const std::vector<int64_t> &b) {
  const size_t n = std::max(a.size(), b.size());
  std::vector<int64_t> out(n);
  for (size_t i = 0; i < n; ++i) {
    const int64_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
    const int64_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
    if (da != db && da != 1 && db != 1) return std::nullopt;
    out[i] = da == 1 ? db : da;
  }
  return out;
}
// the elements of `v` (shape `from`) as an array of shape `to` (a broadcast of `from`), flattened
inline std::vector<uint32_t> broadcast_to(const std::vector<uint32_t> &v, const std::vector<int64_t> &from,
                                          const std::vector<int64_t> &to) {
  int64_t n = 1;
  for (int64_t d : to) n *= d;
  std::vector<uint32_t> out((size_t)n);
  const size_t off = to.size() - from.size();
  for (int64_t i = 0; i < n; ++i) {
    int64_t rem = i, src = 0, stride = 1;
    for (size_t ax = to.size(); ax-- > 0;) {
      const int64_t c = rem % to[ax];
      rem /= to[ax];
      if (ax >= off) {
        const int64_t d = from[ax - off];
        src += (d == 1 ? 0 : c) * stride;
        stride *= d;
      }
    }
    out[(size_t)i] = v[(size_t)src];
  }
  return out;
}
}  // namespace idx

// gather_qmm(x, w, scales, biases, lhs_indices, rhs_indices, transpose, group_size, bits,
// sorted_indices) with the batch semantics of mlx-rs/src/ops/quantization.rs:160-230: x is
// [..., M, K] in bf16, f16 or f32 (scales and biases in the same type), w u32 [..., N, K*bits/32]
// (transpose = false: [..., K, N*bits/32]); the leading axes are batch axes which the uint32 index
// arrays (any shapes, broadcast against each other; an absent one counts through its batch) index in
// flattened form.  Returns [*broadcast shape, M, N].  The index arrays pass through the host.
inline Result<Array> gather_qmm(const Array &x, const Array &w, const Array &scales,
                                const Array *biases = nullptr, const Array *lhs_indices = nullptr,
                                const Array *rhs_indices = nullptr,
                                std::optional<bool> transpose = {},
                                std::optional<int32_t> group_size = {},
                                std::optional<int32_t> bits = {},
                                std::optional<bool> sorted_indices = {}, Stream s = {}) {
  const bool tr = transpose.value_or(true), sorted = sorted_indices.value_or(false);
  const int32_t g = group_size.value_or(DEFAULT_GROUP_SIZE), b = bits.value_or(DEFAULT_BITS);
  const int32_t dt = float_code(x.dtype());
  if (dt < 0) return Exception("gather_qmm: x has the wrong dtype (bfloat16, float16 or float32)");
  if (auto e = detail::want(w, Dtype::Uint32, "gather_qmm", "w")) return *e;
  if (auto e = detail::want(scales, x.dtype(), "gather_qmm", "scales")) return *e;
  if (!biases) return Exception("gather_qmm: biases are required in affine mode");
  if (auto e = detail::want(*biases, x.dtype(), "gather_qmm", "biases")) return *e;
  if (x.ndim() < 2 || w.ndim() < 2 || b <= 0)
    return Exception("gather_qmm: x must be [..., M, K] and w [..., N, K*bits/32]");
  const std::vector<int64_t> xb_shape(x.shape().begin(), x.shape().end() - 2), wb_shape(w.shape().begin(), w.shape().end() - 2);
  int64_t xb = 1, E = 1;
  for (int64_t d : xb_shape) xb *= d;
  for (int64_t d : wb_shape) E *= d;
  const int32_t M = (int32_t)x.dim(-2), K = (int32_t)x.dim(-1);
  const int32_t N = tr ? (int32_t)w.dim(-2) : (int32_t)(w.dim(-1) * 32 / b);
  // index arrays of one shape need no broadcast: they go to the library as they are, on the device
  if (lhs_indices && rhs_indices && lhs_indices->shape() == rhs_indices->shape()) {
    if (lhs_indices->dtype() != Dtype::Uint32 || rhs_indices->dtype() != Dtype::Uint32)
      return Exception("gather_qmm: index arrays must be uint32");
    const int64_t n_same = rhs_indices->size();
    std::vector<int64_t> shape_same = rhs_indices->shape();
    shape_same.push_back(M);
    shape_same.push_back(N);
    auto y = Array::empty(shape_same, x.dtype());
    if (y.is_err() || n_same == 0) return y;
    size_t wb = 0;
    if (mi_moe_gather_qmm_workspace_size((int32_t)std::min<int64_t>(std::max<int64_t>(E, 1), 512), n_same, M, &wb))
      return detail::last_error("gather_qmm");
    auto ws = Array::empty({(int64_t)(wb + 256 + 3) / 4}, Dtype::Uint32);
    if (ws.is_err()) return ws;
    const int rc = mi_moe_gather_qmm_typed(x.data(), w.ptr<uint32_t>(), scales.data(), biases->data(),
                                           lhs_indices->ptr<uint32_t>(), rhs_indices->ptr<uint32_t>(), n_same, xb, M, N, K,
                                           (int32_t)E, tr ? 1 : 0, g, b, sorted ? 1 : 0, dt, y.value().data(),
                                           ws.value().data(), ws.value().nbytes(), s.as_ptr());
    // the workspace goes when this function returns: the work that uses it must have finished (also after a failure)
    const hipError_t e = hipStreamSynchronize(s.handle);
    if (rc) return detail::last_error("gather_qmm");
    if (e != hipSuccess) return detail::hip_error("gather_qmm", e);
    return y;
  }
  // otherwise the arrays pass through the host, where they are broadcast (this path synchronises the stream)
  auto lh = idx::host_indices(lhs_indices, xb_shape, s);
  if (lh.is_err()) return lh.error();
  auto rh = idx::host_indices(rhs_indices, wb_shape, s);
  if (rh.is_err()) return rh.error();
  const auto bshape = idx::broadcast_shape(lh.value().second, rh.value().second);
  if (!bshape) return Exception("gather_qmm: the shapes of lhs_indices and rhs_indices do not broadcast");
  const std::vector<uint32_t> lf = idx::broadcast_to(lh.value().first, lh.value().second, *bshape);
  const std::vector<uint32_t> rf = idx::broadcast_to(rh.value().first, rh.value().second, *bshape);
  const int64_t n_idx = (int64_t)rf.size();
  std::vector<int64_t> out_shape = *bshape;
  out_shape.push_back(M);
  out_shape.push_back(N);
  auto y = Array::empty(out_shape, x.dtype());
  if (y.is_err() || n_idx == 0) return y;
  auto ld = Array::from_host(lf.data(), {n_idx}, Dtype::Uint32, s);
  auto rd = Array::from_host(rf.data(), {n_idx}, Dtype::Uint32, s);
  // from here on the uploads of the index copies may be in flight: every way out waits for the stream
  // before the copies (and the workspace) are released
  auto leave = [&](Result<Array> r) -> Result<Array> {
    const hipError_t e = hipStreamSynchronize(s.handle);
    if (r.is_err() || e == hipSuccess) return r;
    return detail::hip_error("gather_qmm", e);
  };
  if (ld.is_err()) return leave(ld);
  if (rd.is_err()) return leave(rd);
  size_t ws_bytes = 0;
  if (mi_moe_gather_qmm_workspace_size((int32_t)std::min<int64_t>(std::max<int64_t>(E, 1), 512), n_idx, M, &ws_bytes))
    return leave(detail::last_error("gather_qmm"));
  auto ws = Array::empty({(int64_t)(ws_bytes + 256 + 3) / 4}, Dtype::Uint32);
  if (ws.is_err()) return leave(ws);
  if (mi_moe_gather_qmm_typed(x.data(), w.ptr<uint32_t>(), scales.data(), biases->data(), ld.value().ptr<uint32_t>(),
                              rd.value().ptr<uint32_t>(), n_idx, xb, M, N, K, (int32_t)E, tr ? 1 : 0, g, b,
                              sorted ? 1 : 0, dt, y.value().data(), ws.value().data(), ws.value().nbytes(),
                              s.as_ptr()))
    return leave(detail::last_error("gather_qmm"));
  return leave(y);
}

}  // namespace ops

namespace fast {

// rms_norm(x, weight, eps): weight * x * rsqrt(mean(x^2) + eps) over the last axis
// (mlx-rs/src/fast.rs:190-207).  x: bf16 [..., H]; weight: bf16 [H].
inline Result<Array> rms_norm(const Array &x, const Array &weight, float eps, Stream s = {}) {
  if (auto e = detail::want(x, Dtype::Bfloat16, "rms_norm", "x")) return *e;
  if (auto e = detail::want(weight, Dtype::Bfloat16, "rms_norm", "weight")) return *e;
  if (x.ndim() < 1 || weight.size() != x.dim(-1)) return Exception("rms_norm: weight must match the last axis of x");
  auto out = Array::empty(x.shape(), Dtype::Bfloat16);
  if (out.is_err()) return out;
  const int64_t H = x.dim(-1);
  if (mi_moe_rms_norm(x.ptr<uint16_t>(), weight.ptr<uint16_t>(), eps, x.size() / H, (int32_t)H,
                      out.value().ptr<uint16_t>(), s.as_ptr()))
    return detail::last_error("rms_norm");
  return out;
}

}  // namespace fast

namespace nn {

// E quantized matrices with a leading expert axis: the fields of QuantizedLinear
// (mlx-rs/src/nn/quantized.rs:254-279) per expert
struct QuantizedSwitchLinear {
  Array weight;  // u32 [E, N, K*bits/32]
  Array scales;  // bf16 [E, N, K/group_size]
  Array biases;  // bf16 [E, N, K/group_size]
  mi_moe_qmat c_struct() const {
    return {weight.ptr<uint32_t>(), scales.ptr<uint16_t>(), biases.ptr<uint16_t>()};
  }
};

class SparseMoeBlock {
 public:
  SparseMoeBlock(const SparseMoeBlock &) = delete;
  SparseMoeBlock &operator=(const SparseMoeBlock &) = delete;
  SparseMoeBlock(SparseMoeBlock &&o) noexcept { *this = std::move(o); }
  SparseMoeBlock &operator=(SparseMoeBlock &&o) noexcept {
    if (this != &o) {
      release();
      cfg_ = o.cfg_;
      gate_weight_ = std::move(o.gate_weight_);
      router_bias_ = std::move(o.router_bias_);
      gate_proj_ = std::move(o.gate_proj_);
      up_proj_ = std::move(o.up_proj_);
      down_proj_ = std::move(o.down_proj_);
      workspace_ = std::move(o.workspace_);
      workspace_tokens_ = o.workspace_tokens_;
      handle_ = o.handle_;
      training_ = o.training_;
      o.handle_ = nullptr;
    }
    return *this;
  }
  ~SparseMoeBlock() { release(); }

  // gate_weight: bf16 [E, H] (the router, a bias-free Linear); router_bias: f32 [E] or none
  static Result<SparseMoeBlock> create(const mi_moe_config &cfg, Array gate_weight,
                                       QuantizedSwitchLinear gate_proj,
                                       QuantizedSwitchLinear up_proj,
                                       QuantizedSwitchLinear down_proj,
                                       std::optional<Array> router_bias = {}) {
    SparseMoeBlock b;
    b.cfg_ = cfg;
    b.gate_weight_ = std::move(gate_weight);
    b.router_bias_ = std::move(router_bias);
    b.gate_proj_ = std::move(gate_proj);
    b.up_proj_ = std::move(up_proj);
    b.down_proj_ = std::move(down_proj);
    mi_moe_weights w{b.gate_weight_.ptr<uint16_t>(),
                     b.router_bias_ ? b.router_bias_->ptr<float>() : nullptr,
                     b.gate_proj_.c_struct(), b.up_proj_.c_struct(), b.down_proj_.c_struct()};
    if (mi_moe_create(&b.cfg_, &w, &b.handle_)) return detail::last_error("SparseMoeBlock");
    return b;
  }

  // x: bf16 [..., H] -> bf16 [..., H]; asynchronous on the stream
  Result<Array> forward(const Array &x, Stream s = {}, const mi_moe_debug_out *dbg = nullptr) {
    if (auto e = detail::want(x, Dtype::Bfloat16, "forward", "x")) return *e;
    if (x.ndim() < 1 || x.dim(-1) != cfg_.hidden)
      return Exception("forward: last dimension must be " + std::to_string(cfg_.hidden));
    const int64_t T = x.size() / cfg_.hidden;
    if (auto r = reserve(T > 0 ? T : 1); r.is_err()) return r.error();
    auto out = Array::empty(x.shape(), Dtype::Bfloat16);
    if (out.is_err()) return out;
    if (mi_moe_forward(handle_, x.ptr<uint16_t>(), T, out.value().ptr<uint16_t>(),
                       workspace_.data(), workspace_.nbytes(), dbg, s.as_ptr()))
      return detail::last_error("forward");
    return out;
  }

  // x + forward(rms_norm(x, norm_weight, eps)): the block between its neighbours in a decoder layer
  // (mlx-lm/src/models/qwen3.rs:310-325), one call
  Result<Array> forward_residual(const Array &x, const Array &norm_weight, float eps, Stream s = {}) {
    if (auto e = detail::want(x, Dtype::Bfloat16, "forward_residual", "x")) return *e;
    if (auto e = detail::want(norm_weight, Dtype::Bfloat16, "forward_residual", "norm_weight")) return *e;
    if (x.ndim() < 1 || x.dim(-1) != cfg_.hidden || norm_weight.size() != cfg_.hidden)
      return Exception("forward_residual: last dimension must be " + std::to_string(cfg_.hidden));
    const int64_t T = x.size() / cfg_.hidden;
    if (auto r = reserve(T > 0 ? T : 1); r.is_err()) return r.error();
    auto out = Array::empty(x.shape(), Dtype::Bfloat16);
    if (out.is_err()) return out;
    if (mi_moe_forward_residual(handle_, x.ptr<uint16_t>(), norm_weight.ptr<uint16_t>(), eps, T,
                                out.value().ptr<uint16_t>(), workspace_.data(), workspace_.nbytes(), nullptr,
                                s.as_ptr()))
      return detail::last_error("forward_residual");
    return out;
  }

  void training_mode(bool mode) { training_ = mode; }  // no layer here depends on it
  const mi_moe_config &config() const { return cfg_; }

  Result<size_t> workspace_bytes(int64_t tokens) const {
    size_t n = 0;
    if (mi_moe_workspace_size(&cfg_, tokens, &n)) return detail::last_error("workspace_size");
    return n;
  }
  Result<Unit> reserve(int64_t tokens) {
    if (tokens <= workspace_tokens_) return Unit{};
    auto n = workspace_bytes(tokens);
    if (n.is_err()) return n.error();
    auto ws = Array::empty({(int64_t)(n.value() + 256 + 3) / 4}, Dtype::Uint32);
    if (ws.is_err()) return ws.error();
    workspace_ = ws.value();
    workspace_tokens_ = tokens;
    return Unit{};
  }

 private:
  SparseMoeBlock() = default;
  void release() {
    if (handle_) mi_moe_destroy(handle_);
    handle_ = nullptr;
  }
  mi_moe_config cfg_{};
  Array gate_weight_;
  std::optional<Array> router_bias_;
  QuantizedSwitchLinear gate_proj_, up_proj_, down_proj_;
  Array workspace_;
  int64_t workspace_tokens_ = -1;
  mi_moe_handle handle_ = nullptr;
  bool training_ = false;
};

}  // namespace nn
}  // namespace mi_moe
