// Exercises include/rmlx_ops.hpp, the C++ mirror of the reference's operator interface.
//
//   ops_mirror_check validate          no GPU: constructor validation and error variants
//   ops_mirror_check run <dir>         GPU: reads the case a test wrote into <dir>, runs it through the
//                                      mirror and writes the results back for the test to compare
//
// <dir>/meta.txt holds "N K group_size bits M E I T top_k" (group_size and bits of the dense weight; the
// expert weights are Q4 with groups of 64); the arrays are raw little-endian files.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <sstream>

#include "rmlx_ops.hpp"

using rmlx::Array;
using rmlx::Buffer;
using rmlx::DType;
using rmlx::KernelError;
using rmlx::ops::quantized::QuantizedWeight;

static int failures = 0;

#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

template <typename F>
static bool raises(F&& f, KernelError::Kind kind, const char* needle) {
  try {
    f();
  } catch (const KernelError& e) {
    const bool ok = e.kind() == kind && std::string(e.what()).find(needle) != std::string::npos;
    if (!ok) std::printf("  got kind %d message \"%s\"\n", static_cast<int>(e.kind()), e.what());
    return ok;
  }
  std::printf("  no error raised\n");
  return false;
}

static int validate() {
  // Host memory stands in for device memory: the constructor only looks at lengths.
  static uint32_t words[64 * 512 / 8];
  static uint16_t halves[64 * 512 / 64];
  auto w = Buffer::borrow(words, sizeof(words));
  auto s = Buffer::borrow(halves, sizeof(halves));
  auto b = Buffer::borrow(halves, sizeof(halves));
  const auto inv = KernelError::Kind::InvalidShape;

  {
    QuantizedWeight ok(w, s, b, 64, 4, 64, 512);
    EXPECT(ok.handle() != nullptr && ok.out_features == 64 && ok.in_features == 512 && ok.n_experts == 1);
    QuantizedWeight stacked(w, s, b, 64, 4, 16, 512, 4);
    EXPECT(stacked.n_experts == 4);
  }
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 64, 5, 64, 512); }, inv, "unsupported bit width 5"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 48, 4, 64, 512); }, inv, "unsupported group_size 48"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 64, 4, 64, 500); }, inv, "in_features (500) must be a multiple of group_size (64)"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 64, 8, 64, 512); }, inv, "weights_buf too small"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 32, 4, 64, 512); }, inv, "scales_buf too small"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, Buffer::borrow(halves, 8), 64, 4, 64, 512); }, inv, "biases_buf too small"));
  EXPECT(raises([&] { QuantizedWeight q(w, s, b, 64, 4, 64, 512, 0); }, inv, "n_experts"));

  // Nothing runs or allocates before init(): the call fails, it does not fall back to the host.
  {
    QuantizedWeight qw(w, s, b, 64, 4, 64, 512);
    Array x(Buffer::borrow(halves, 1024), {512}, DType::Float16);
    EXPECT(raises([&] { rmlx::ops::quantized::affine_quantized_matmul(qw, x); }, KernelError::Kind::Runtime,
                  "rmlx_hip_init() has not been called"));
    EXPECT(raises([&] { Array::uninit({4}, DType::Float16); }, KernelError::Kind::Runtime, "rmlx_hip_init"));
  }
  Array a(Buffer::borrow(halves, 64), {2, 4, 4}, DType::Float16);
  EXPECT(a.numel() == 32 && a.nbytes() == 64 && a.view().ndim == 3 && a.view().shape[3] == 1);
  EXPECT(rmlx::size_of(DType::Float32) == 4 && rmlx::size_of(DType::Bfloat16) == 2 && rmlx::size_of(DType::UInt8) == 1);
  std::printf(failures == 0 ? "validate ok\n" : "validate FAILED\n");
  return failures == 0 ? 0 : 1;
}

static std::vector<char> slurp(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) throw std::runtime_error("cannot open " + path);
  return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static Array load(const std::string& path, const std::vector<size_t>& shape, DType t) {
  const std::vector<char> bytes = slurp(path);
  Array a = Array::uninit(shape, t);
  if (a.nbytes() != bytes.size()) throw std::runtime_error(path + ": unexpected length");
  rmlx::detail::check(rmlx_hip_memcpy_h2d(a.data(), bytes.data(), bytes.size(), nullptr));
  return a;
}

static std::shared_ptr<QuantizedWeight> load_weight(const std::string& stem, size_t e, size_t n, size_t k, uint32_t gs,
                                                    uint32_t bits) {
  Array w = load(stem + "_w.bin", {e, n, k * bits / 32}, DType::UInt32);
  Array s = load(stem + "_s.bin", {e, n, k / gs}, DType::Float16);
  Array b = load(stem + "_b.bin", {e, n, k / gs}, DType::Float16);
  return std::make_shared<QuantizedWeight>(w.buffer(), s.buffer(), b.buffer(), gs, bits, n, k, e);
}

static void store(const std::string& path, const Array& a) {
  std::vector<char> bytes(a.nbytes());
  a.to_host(bytes.data());
  std::ofstream f(path, std::ios::binary);
  f.write(bytes.data(), static_cast<std::streamsize>(bytes.size()));
}

static int run(const std::string& dir) {
  size_t n, k, gs, bits, m, e, inter, t, top_k;
  {
    const std::vector<char> meta = slurp(dir + "/meta.txt");
    std::istringstream in(std::string(meta.begin(), meta.end()));
    in >> n >> k >> gs >> bits >> m >> e >> inter >> t >> top_k;
    if (!in) throw std::runtime_error("meta.txt: expected nine integers");
  }
  rmlx::init(0);
  namespace q = rmlx::ops::quantized;

  // dense: qmv, qmm, the two fused epilogues and QuantizedLinear with a bias
  auto qw = load_weight(dir + "/dense", 1, n, k, gs, bits);
  Array x = load(dir + "/x.bin", {m, k}, DType::Float16);
  Array side = load(dir + "/side.bin", {m, n}, DType::Float32);
  Array vec(x.buffer(), {k}, DType::Float16);  // row 0
  store(dir + "/out_qmv.bin", q::affine_quantized_matmul(*qw, vec));
  store(dir + "/out_qmm.bin", q::affine_quantized_matmul_batched(x, *qw));
  store(dir + "/out_residual.bin", q::qmm_add_residual(x, *qw, side));
  store(dir + "/out_swiglu.bin", q::qmm_swiglu(x, *qw, side));
  {
    Array norm_weight = load(dir + "/norm_weight.bin", {k}, DType::Float16);
    Array inv_rms = load(dir + "/inv_rms.bin", {m}, DType::Float32);
    store(dir + "/out_norm.bin", q::qmm_norm(x, *qw, norm_weight, inv_rms));
  }
  {
    rmlx::Stream stream;  // the enqueue-only twin, then one synchronisation
    Array bias = load(dir + "/bias.bin", {n}, DType::Float16);
    rmlx::nn::QuantizedLinear lin(qw, bias.buffer());
    Array y = lin.forward(x, &stream);
    stream.synchronize();
    store(dir + "/out_linear.bin", y);
  }
  EXPECT(raises([&] { q::affine_quantized_matmul(*qw, x); }, KernelError::Kind::InvalidShape, "in_features"));

  // experts: gather_qmm, routing, ExpertGroup and the routed block
  auto gate = load_weight(dir + "/gate", e, inter, k, 64, 4);
  auto up = load_weight(dir + "/up", e, inter, k, 64, 4);
  auto down = load_weight(dir + "/down", e, k, inter, 64, 4);
  Array xt = load(dir + "/xt.bin", {t, k}, DType::Float16);
  Array logits = load(dir + "/logits.bin", {t, e}, DType::Float32);
  Array pick = load(dir + "/pick.bin", {t}, DType::UInt32);
  Array x3(xt.buffer(), {t, 1, k}, DType::Float16);
  store(dir + "/out_gather.bin", q::gather_qmm(x3, *gate, pick, t, 1));
  auto route = rmlx::ops::topk_route::gpu_topk_route(logits, top_k);
  store(dir + "/out_route_idx.bin", route.expert_indices);
  store(dir + "/out_route_w.bin", route.expert_weights);
  store(dir + "/out_route_counts.bin", route.expert_counts);
  store(dir + "/out_route_offsets.bin", route.dispatch_offsets);
  rmlx::nn::MoeExperts experts(gate, up, down);
  store(dir + "/out_moe_grouped.bin", experts.forward_grouped(xt, route.expert_indices, route.expert_weights, top_k));
  store(dir + "/out_moe.bin", experts.forward(xt, logits, top_k));
  {
    // two items: the first two tokens through expert 1, the rest through expert 0
    rmlx::nn::ExpertGroup group(gate, up, down);
    Array head(xt.buffer(), {2, k}, DType::Float16);
    Array tail(xt.buffer(), {t - 2, k}, DType::Float16, 2 * k * 2);
    std::vector<Array> ys = group.grouped_forward({{1, head}, {0, tail}});
    EXPECT(ys.size() == 2 && ys[0].shape()[0] == 2 && ys[1].shape()[0] == t - 2);
    store(dir + "/out_group0.bin", ys[0]);
    store(dir + "/out_group1.bin", ys[1]);
    EXPECT(raises([&] { group.grouped_forward({{e, head}}); }, KernelError::Kind::InvalidShape, ""));
  }
  std::printf(failures == 0 ? "run ok\n" : "run FAILED\n");
  return failures == 0 ? 0 : 1;
}

int main(int argc, char** argv) {
  try {
    if (argc == 2 && std::string(argv[1]) == "validate") return validate();
    if (argc == 3 && std::string(argv[1]) == "run") return run(argv[2]);
  } catch (const std::exception& e) {
    std::printf("error: %s\n", e.what());
    return 2;
  }
  std::printf("usage: ops_mirror_check validate | run <dir>\n");
  return 64;
}
