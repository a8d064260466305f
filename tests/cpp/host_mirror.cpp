// Test driver of the C++ host layer (mlx-rs_amd/host/mi_moe.hpp).
//   host_mirror errors          host-only: argument errors come back as Exception values with
//                               the library's message (no GPU is touched)
//   host_mirror forward <dir>   reads a layer and tokens written by the Python test as raw
//                               arrays, runs SparseMoeBlock::forward, ops::gather_qmm,
//                               ops::quantize and ops::dequantize on the GPU and writes the
//                               results back as raw arrays for the test to compare
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "../../mlx-rs_amd/host/mi_moe.hpp"

using namespace mi_moe;

static int fails = 0;
#define EXPECT(cond)                                                     \
  do {                                                                   \
    if (!(cond)) {                                                       \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
      ++fails;                                                           \
    }                                                                    \
  } while (0)

static bool contains(const Exception &e, const char *needle) {
  return std::string(e.what()).find(needle) != std::string::npos;
}

static int run_errors() {
  // a configuration the library refuses: the text names the field
  mi_moe_config bad{256, 8, 2, 512, 3, 64, 0};
  nn::QuantizedSwitchLinear none;
  auto b = nn::SparseMoeBlock::create(bad, Array(), none, none, none);
  EXPECT(b.is_err());
  EXPECT(b.is_err() && contains(b.error(), "bits"));
  bool thrown = false;
  try {
    (void)nn::SparseMoeBlock::create(bad, Array(), none, none, none).unwrap();
  } catch (const Exception &e) {
    thrown = contains(e, "bits");
  }
  EXPECT(thrown);
  // gather_qmm: dtype, rank and missing-operand checks happen before any device work
  Array x = Array::from_device_ptr(nullptr, {4, 1, 128}, Dtype::Bfloat16);
  Array w = Array::from_device_ptr(nullptr, {2, 16, 16}, Dtype::Uint32);
  Array s = Array::from_device_ptr(nullptr, {2, 16, 2}, Dtype::Bfloat16);
  Array idx = Array::from_device_ptr(nullptr, {4}, Dtype::Uint32);
  Array bad_idx = Array::from_device_ptr(nullptr, {4}, Dtype::Float32);
  auto r1 = ops::gather_qmm(x, w, s, &s, nullptr, &bad_idx);
  EXPECT(r1.is_err() && contains(r1.error(), "uint32"));
  auto r2 = ops::gather_qmm(x, w, s, nullptr, nullptr, &idx);
  EXPECT(r2.is_err() && contains(r2.error(), "biases"));
  auto r3 = ops::gather_qmm(w, w, s, &s, nullptr, &idx);
  EXPECT(r3.is_err() && contains(r3.error(), "dtype"));
  // quantize: the library's own message for a group size that does not divide the columns
  Array wf = Array::from_device_ptr(nullptr, {4, 100}, Dtype::Float32);
  auto q = ops::quantize(wf, 64, 4);
  EXPECT(q.is_err() && contains(q.error(), "divisible"));
  auto q2 = ops::quantize(Array::from_device_ptr(nullptr, {4, 128}, Dtype::Float32), 64, 3);
  EXPECT(q2.is_err() && contains(q2.error(), "bits"));
  std::printf(fails ? "errors: %d failed\n" : "errors: ok\n", fails);
  return fails ? 1 : 0;
}

static std::vector<char> slurp(const std::string &p) {
  std::ifstream f(p, std::ios::binary);
  if (!f) {
    std::printf("cannot read %s\n", p.c_str());
    std::exit(2);
  }
  return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}
static void dump(const std::string &p, const Array &a) {
  std::vector<char> h(a.nbytes());
  a.to_host(h.data()).unwrap();
  std::ofstream f(p, std::ios::binary);
  f.write(h.data(), (std::streamsize)h.size());
}
static Array load(const std::string &dir, const char *name, std::vector<int64_t> shape, Dtype d) {
  auto bytes = slurp(dir + "/" + name);
  Array probe = Array::from_device_ptr(nullptr, shape, d);
  if (bytes.size() != probe.nbytes()) {
    std::printf("%s: %zu bytes, expected %zu\n", name, bytes.size(), probe.nbytes());
    std::exit(2);
  }
  return Array::from_host(bytes.data(), std::move(shape), d).unwrap();
}

static int run_forward(const std::string &dir) {
  long H, E, k, I, bits, mode, T, qrows, qcols;
  {
    std::ifstream f(dir + "/cfg.txt");
    if (!(f >> H >> E >> k >> I >> bits >> mode >> T >> qrows >> qcols)) {
      std::printf("bad cfg.txt\n");
      return 2;
    }
  }
  const int64_t wpw = 32 / bits;
  auto bank = [&](const char *n, int64_t N, int64_t K) {
    std::string b(n);
    return nn::QuantizedSwitchLinear{load(dir, (b + "_w.bin").c_str(), {E, N, K / wpw}, Dtype::Uint32),
                                     load(dir, (b + "_s.bin").c_str(), {E, N, K / 64}, Dtype::Bfloat16),
                                     load(dir, (b + "_b.bin").c_str(), {E, N, K / 64}, Dtype::Bfloat16)};
  };
  auto gate = bank("gate", I, H), up = bank("up", I, H), down = bank("down", H, I);
  Array router = load(dir, "router_w.bin", {E, H}, Dtype::Bfloat16);
  Array x = load(dir, "x.bin", {T, H}, Dtype::Bfloat16);
  mi_moe_config cfg{(int32_t)H, (int32_t)E, (int32_t)k, (int32_t)I, (int32_t)bits, 64, (int32_t)mode};
  std::printf("forward: H%ld E%ld k%ld I%ld bits%ld T%ld\n", H, E, k, I, bits, T);
  std::fflush(stdout);

  auto blk = nn::SparseMoeBlock::create(cfg, router, gate, up, down).unwrap();
  blk.training_mode(false);
  // a 3-d input [2, T/2, H] keeps its shape (the layer flattens the leading axes)
  Array out = blk.forward(x.reshape({2, T / 2, H})).unwrap();
  EXPECT(out.ndim() == 3 && out.dim(0) == 2 && out.dim(-1) == H);
  dump(dir + "/out.bin", out);
  // a second, shorter call through the same handle and workspace
  Array out2 = blk.forward(Array::from_device_ptr(x.data(), {T / 2, H}, Dtype::Bfloat16)).unwrap();
  dump(dir + "/out2.bin", out2);
  // a wrong last dimension is an error value, not a crash
  auto bad = blk.forward(x.reshape({T * 2, H / 2}));
  EXPECT(bad.is_err() && contains(bad.error(), "last dimension"));

  // ops::gather_qmm with the indices the test supplies (the gate projection of every pair)
  Array lhs = load(dir, "lhs.bin", {T * k}, Dtype::Uint32);
  Array rhs = load(dir, "rhs.bin", {T * k}, Dtype::Uint32);
  Array g = ops::gather_qmm(x.reshape({T, 1, H}), gate.weight, gate.scales, &gate.biases, &lhs, &rhs,
                            true, 64, (int32_t)bits, false).unwrap();
  EXPECT(g.dim(0) == T * k && g.dim(1) == 1 && g.dim(2) == I);
  dump(dir + "/gq.bin", g);
  // library-side refusal surfaces as an error value with its text
  auto bad2 = ops::gather_qmm(x.reshape({T, 1, H}), gate.weight, gate.scales, &gate.biases, &lhs, &rhs,
                              true, 48, (int32_t)bits, false);
  EXPECT(bad2.is_err() && contains(bad2.error(), "group_size"));
  // index arrays of shapes [2, 1] and [1, 3] broadcast to [2, 3]: the same bytes as the six pairs spelt out
  {
    const uint32_t l21[2] = {5, 1}, r13[3] = {3, 0, 2}, l6[6] = {5, 5, 5, 1, 1, 1}, r6[6] = {3, 0, 2, 3, 0, 2};
    Array a21 = Array::from_host(l21, {2, 1}, Dtype::Uint32).unwrap(), a13 = Array::from_host(r13, {1, 3}, Dtype::Uint32).unwrap();
    Array a6 = Array::from_host(l6, {6}, Dtype::Uint32).unwrap(), b6 = Array::from_host(r6, {6}, Dtype::Uint32).unwrap();
    Array yb = ops::gather_qmm(x.reshape({T, 1, H}), gate.weight, gate.scales, &gate.biases, &a21, &a13, true, 64,
                               (int32_t)bits, false).unwrap();
    Array yf = ops::gather_qmm(x.reshape({T, 1, H}), gate.weight, gate.scales, &gate.biases, &a6, &b6, true, 64,
                               (int32_t)bits, false).unwrap();
    EXPECT(yb.ndim() == 4 && yb.dim(0) == 2 && yb.dim(1) == 3 && yb.dim(2) == 1 && yb.dim(3) == I);
    std::vector<uint16_t> hb((size_t)yb.size()), hf((size_t)yf.size());
    yb.to_host(hb.data()).unwrap();
    yf.to_host(hf.data()).unwrap();
    EXPECT(hb.size() == hf.size() && hb == hf);
    auto bad3 = ops::gather_qmm(x.reshape({T, 1, H}), gate.weight, gate.scales, &gate.biases, &a6, &a13, true, 64,
                                (int32_t)bits, false);
    EXPECT(bad3.is_err() && contains(bad3.error(), "broadcast"));
  }

  // ops::quantize / ops::dequantize with the defaults (group 64, 4 bits)
  Array wf = load(dir, "wf.bin", {qrows, qcols}, Dtype::Float32);
  auto [q, s, b] = ops::quantize(wf).unwrap();
  dump(dir + "/q.bin", q);
  dump(dir + "/s.bin", s);
  dump(dir + "/b.bin", b);
  dump(dir + "/dq.bin", ops::dequantize(q, s, b).unwrap());
  std::printf(fails ? "forward: %d failed\n" : "forward: ok\n", fails);
  return fails ? 1 : 0;
}

int main(int argc, char **argv) {
  if (argc >= 2 && std::string(argv[1]) == "errors") return run_errors();
  if (argc >= 3 && std::string(argv[1]) == "forward") return run_forward(argv[2]);
  std::printf("usage: host_mirror errors | forward <dir>\n");
  return 2;
}
