// rmlx_ops.hpp -- C++ host-side mirror of the reference's operator interface for the quantized-matmul
// path, written over the C ABI of rmlx_hip.h (header only; link with -lrmlx_hip).
//
// The reference's host code is Rust; where no Rust toolchain exists this header plays the role its
// `rmlx-core` / `rmlx-nn` wrappers play: same type and function names, the same argument order and
// meaning, and errors that carry the reference's variants and messages:
//   rmlx::KernelError                       crates/rmlx-core/src/kernels/mod.rs:29-42
//   rmlx::DType, rmlx::Array                crates/rmlx-core/src/dtype.rs:34-52, src/array.rs:137-260
//   rmlx::ops::quantized::QuantizedWeight   crates/rmlx-core/src/ops/quantized.rs:78-177
//   ...::affine_quantized_matmul            :1309-1411       ...::affine_quantized_matmul_batched  :7149-7782
//   ...::qmm_add_residual / qmm_swiglu      :8227-8452       ...::gather_qmm                       :9404-9599
//   ...::awq_dequant / gptq_dequant         :2269-2590
//   rmlx::ops::topk_route::gpu_topk_route   crates/rmlx-core/src/ops/topk_route.rs:396-650
//   rmlx::nn::QuantizedLinear               crates/rmlx-nn/src/quantized_linear.rs:77-201
//   rmlx::nn::MoeExperts::forward_grouped   crates/rmlx-nn/src/moe.rs:1391-1508 (routed block of MoeLayer)
// Where the reference takes `(&KernelRegistry, ..., &MTLCommandQueue)` these functions take an optional
// `Stream*`: null = synchronous (`ExecMode::Sync`), a stream = enqueue only (the `_into_cb` twins).
#ifndef RMLX_OPS_HPP
#define RMLX_OPS_HPP

#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "rmlx_hip.h"

namespace rmlx {

// `KernelError` (kernels/mod.rs:29-42): the two variants this path raises, plus a failing runtime call.
class KernelError : public std::runtime_error {
 public:
  enum class Kind { InvalidShape, NotFound, Runtime };
  KernelError(Kind kind, const std::string& msg) : std::runtime_error(msg), kind_(kind) {}
  Kind kind() const { return kind_; }

 private:
  Kind kind_;
};

namespace detail {
inline void check(int32_t status) {
  if (status == RMLX_OK) return;
  const std::string msg = rmlx_hip_last_error();
  throw KernelError(status == RMLX_INVALID_SHAPE ? KernelError::Kind::InvalidShape
                    : status == RMLX_NOT_FOUND   ? KernelError::Kind::NotFound
                                                 : KernelError::Kind::Runtime,
                    msg);
}
}  // namespace detail

// Selects the device and loads the kernels (the role of `KernelRegistry::new` + `register_*` on this path).
inline void init(int device = 0) { detail::check(rmlx_hip_init(device)); }

enum class DType { Float32 = RMLX_DTYPE_F32, Float16 = RMLX_DTYPE_F16, Bfloat16 = RMLX_DTYPE_BF16,
                   UInt32 = RMLX_DTYPE_U32, UInt8 = RMLX_DTYPE_U8 };
inline size_t size_of(DType t) {
  switch (t) {
    case DType::Float32: case DType::UInt32: return 4;
    case DType::Float16: case DType::Bfloat16: return 2;
    default: return 1;
  }
}

// A HIP stream (the reference's command queue / command buffer pair).
class Stream {
 public:
  Stream() { detail::check(rmlx_hip_stream_create(&s_)); }
  ~Stream() { if (s_ != nullptr) rmlx_hip_stream_destroy(s_); }
  Stream(const Stream&) = delete;
  Stream& operator=(const Stream&) = delete;
  void synchronize() { detail::check(rmlx_hip_stream_sync(s_)); }
  rmlx_stream raw() const { return s_; }

 private:
  rmlx_stream s_ = nullptr;
};
inline rmlx_stream raw(const Stream* s) { return s == nullptr ? nullptr : s->raw(); }

// Device memory owned by the host side (an `MTLBuffer` in the reference).
class Buffer {
 public:
  explicit Buffer(size_t bytes) : bytes_(bytes) {
    if (bytes != 0) detail::check(rmlx_hip_malloc(&ptr_, bytes));
  }
  // Wraps device memory somebody else owns (a tensor of the caller's framework); never freed here.
  static std::shared_ptr<Buffer> borrow(void* dev_ptr, size_t bytes) {
    std::shared_ptr<Buffer> b(new Buffer());
    b->ptr_ = dev_ptr;
    b->bytes_ = bytes;
    b->owned_ = false;
    return b;
  }
  ~Buffer() { if (owned_ && ptr_ != nullptr) rmlx_hip_free(ptr_); }
  Buffer(const Buffer&) = delete;
  Buffer& operator=(const Buffer&) = delete;
  void* ptr() const { return ptr_; }
  size_t length() const { return bytes_; }

 private:
  Buffer() : bytes_(0) {}
  void* ptr_ = nullptr;
  size_t bytes_;
  bool owned_ = true;
};

// `Array` (array.rs:137-260): shape, dtype and a shared device buffer; row-contiguous.
class Array {
 public:
  Array() = default;
  Array(std::shared_ptr<Buffer> buf, std::vector<size_t> shape, DType dtype, size_t offset = 0)
      : buf_(std::move(buf)), shape_(std::move(shape)), dtype_(dtype), offset_(offset) {}
  // `Array::uninit` (array.rs:238)
  static Array uninit(const std::vector<size_t>& shape, DType dtype) {
    size_t n = 1;
    for (size_t d : shape) n *= d;
    return Array(std::make_shared<Buffer>(n * size_of(dtype)), shape, dtype);
  }
  static Array from_host(const void* data, const std::vector<size_t>& shape, DType dtype) {
    Array a = uninit(shape, dtype);
    if (a.nbytes() != 0) detail::check(rmlx_hip_memcpy_h2d(a.data(), data, a.nbytes(), nullptr));
    return a;
  }
  void to_host(void* dst) const {
    if (nbytes() != 0) detail::check(rmlx_hip_memcpy_d2h(dst, data(), nbytes(), nullptr));
  }
  const std::vector<size_t>& shape() const { return shape_; }
  size_t ndim() const { return shape_.size(); }
  DType dtype() const { return dtype_; }
  size_t numel() const { size_t n = 1; for (size_t d : shape_) n *= d; return n; }
  size_t nbytes() const { return numel() * size_of(dtype_); }
  void* data() const { return buf_ ? static_cast<char*>(buf_->ptr()) + offset_ : nullptr; }
  const std::shared_ptr<Buffer>& buffer() const { return buf_; }
  rmlx_array view() const {
    if (shape_.size() > 4) throw KernelError(KernelError::Kind::InvalidShape, "arrays of more than 4 dimensions are not supported");
    rmlx_array a;
    a.data = data();
    a.dtype = static_cast<int32_t>(dtype_);
    a.ndim = static_cast<int32_t>(shape_.size());
    for (size_t i = 0; i < 4; ++i) a.shape[i] = i < shape_.size() ? shape_[i] : 1;
    return a;
  }

 private:
  std::shared_ptr<Buffer> buf_;
  std::vector<size_t> shape_;
  DType dtype_ = DType::Float16;
  size_t offset_ = 0;
};

namespace ops {
namespace quantized {

// `QuantizedWeight` (quantized.rs:78-177): three device buffers in MLX affine layout plus metadata.
// `n_experts` > 1 declares the stacked [n_experts, out_features, ...] layout of gather_qmm.
class QuantizedWeight {
 public:
  QuantizedWeight(std::shared_ptr<Buffer> weights_buf, std::shared_ptr<Buffer> scales_buf,
                  std::shared_ptr<Buffer> biases_buf, uint32_t group_size, uint32_t bits, size_t out_features,
                  size_t in_features, size_t n_experts = 1)
      : weights_buf(std::move(weights_buf)), scales_buf(std::move(scales_buf)), biases_buf(std::move(biases_buf)),
        group_size(group_size), bits(bits), out_features(out_features), in_features(in_features), n_experts(n_experts) {
    detail::check(rmlx_hip_qweight_create(
        this->weights_buf ? this->weights_buf->ptr() : nullptr, this->weights_buf ? this->weights_buf->length() : 0,
        this->scales_buf ? this->scales_buf->ptr() : nullptr, this->scales_buf ? this->scales_buf->length() : 0,
        this->biases_buf ? this->biases_buf->ptr() : nullptr, this->biases_buf ? this->biases_buf->length() : 0,
        group_size, bits, out_features, in_features, n_experts, &handle_));
  }
  ~QuantizedWeight() { if (handle_ != nullptr) rmlx_hip_qweight_destroy(handle_); }
  QuantizedWeight(const QuantizedWeight&) = delete;
  QuantizedWeight& operator=(const QuantizedWeight&) = delete;
  const rmlx_qweight* handle() const { return handle_; }
  uint32_t set_expert_gemm_min_rows(uint32_t min_rows) const { return rmlx_hip_qweight_set_expert_gemm_min_rows(handle_, min_rows); }
  uint32_t set_expert_stream_kernel(uint32_t kind) const { return rmlx_hip_qweight_set_expert_stream_kernel(handle_, kind); }
  // Give the K-split GEMMs a tile-contiguous copy of the weights in `dst` (gemm_layout_bytes() bytes, kept alive by the
  // caller via the shared pointer stored here); an empty pointer drops it.
  size_t gemm_layout_bytes() const { return rmlx_hip_qweight_gemm_layout_bytes(handle_); }
  void set_gemm_layout(std::shared_ptr<Buffer> dst, const Stream* stream = nullptr) {
    detail::check(rmlx_hip_qweight_set_gemm_layout(handle_, dst ? dst->ptr() : nullptr, dst ? dst->length() : 0, raw(stream)));
    gemm_layout_buf = std::move(dst);
  }
  std::shared_ptr<Buffer> gemm_layout_buf;

  std::shared_ptr<Buffer> weights_buf, scales_buf, biases_buf;
  uint32_t group_size, bits;
  size_t out_features, in_features, n_experts;

 private:
  rmlx_qweight* handle_ = nullptr;
};

// qmv: vec [in_features] -> f16 [out_features]
inline Array affine_quantized_matmul(const QuantizedWeight& qw, const Array& vec, const Stream* stream = nullptr) {
  Array out = Array::uninit({qw.out_features}, DType::Float16);
  const rmlx_array v = vec.view();
  detail::check(rmlx_hip_affine_quantized_matmul(qw.handle(), &v, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// qmm: x [M, in_features] -> f16 [M, out_features]
inline Array affine_quantized_matmul_batched(const Array& x, const QuantizedWeight& qw, const Stream* stream = nullptr) {
  const size_t m = x.ndim() == 2 ? x.shape()[0] : 0;
  Array out = Array::uninit({m, qw.out_features}, DType::Float16);
  const rmlx_array v = x.view();
  detail::check(rmlx_hip_affine_quantized_matmul_batched(qw.handle(), &v, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// out = x @ dequant(W)^T + residual
inline Array qmm_add_residual(const Array& x, const QuantizedWeight& qw, const Array& residual, const Stream* stream = nullptr) {
  const size_t m = x.ndim() == 2 ? x.shape()[0] : 0;
  Array out = Array::uninit({m, qw.out_features}, DType::Float16);
  const rmlx_array v = x.view(), r = residual.view();
  detail::check(rmlx_hip_qmm_add_residual(qw.handle(), &v, &r, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// out = silu(gate_result) * (x @ dequant(W)^T)
inline Array qmm_swiglu(const Array& x, const QuantizedWeight& qw, const Array& gate_result, const Stream* stream = nullptr) {
  const size_t m = x.ndim() == 2 ? x.shape()[0] : 0;
  Array out = Array::uninit({m, qw.out_features}, DType::Float16);
  const rmlx_array v = x.view(), g = gate_result.view();
  detail::check(rmlx_hip_qmm_swiglu(qw.handle(), &v, &g, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// out = ((x * half(inv_rms[m])) * norm_weight[k]) @ dequant(W)^T: the RMSNorm prologue (`has_norm`) of the
// reference's MMA kernel (quantized.rs:2955-2992, 3070-3095); norm_weight f16 [K], inv_rms f32 [M]
inline Array qmm_norm(const Array& x, const QuantizedWeight& qw, const Array& norm_weight, const Array& inv_rms,
                      const Stream* stream = nullptr) {
  const size_t m = x.ndim() == 2 ? x.shape()[0] : 0;
  Array out = Array::uninit({m, qw.out_features}, DType::Float16);
  const rmlx_array v = x.view(), w = norm_weight.view(), r = inv_rms.view();
  detail::check(rmlx_hip_qmm_norm(qw.handle(), &v, &w, &r, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// out[b] = x[b] @ dequant(W[indices[b]])^T over stacked expert weights
inline Array gather_qmm(const Array& x, const QuantizedWeight& stacked, const Array& indices, size_t batch,
                        size_t m_per_batch, const Stream* stream = nullptr) {
  Array out = Array::uninit({batch, m_per_batch, stacked.out_features}, DType::Float16);
  const rmlx_array v = x.view(), i = indices.view();
  detail::check(rmlx_hip_gather_qmm(&v, stacked.weights_buf->ptr(), stacked.weights_buf->length(),
                                    stacked.scales_buf->ptr(), stacked.scales_buf->length(), stacked.biases_buf->ptr(),
                                    stacked.biases_buf->length(), &i, batch, m_per_batch, stacked.out_features,
                                    stacked.in_features, stacked.n_experts, stacked.group_size, out.data(), out.nbytes(),
                                    raw(stream)));
  return out;
}

// AWQ INT4 -> f32 [rows, cols] (quantized.rs:2269-2383)
inline Array awq_dequant(const Array& qweight, const Array& qzeros, const Array& scales, size_t rows, size_t cols,
                         size_t group_size, const Stream* stream = nullptr) {
  Array out = Array::uninit({rows, cols}, DType::Float32);
  detail::check(rmlx_hip_awq_dequant(qweight.data(), qweight.nbytes(), qzeros.data(), qzeros.nbytes(), scales.data(),
                                     scales.nbytes(), rows, cols, group_size, out.data(), out.nbytes(), raw(stream)));
  return out;
}

// GPTQ INT4 -> f32 [in_features, out_features] (quantized.rs:2407-2590); g_idx: null or i32 [in_features]
// carried in a UInt32 array.
inline Array gptq_dequant(const Array& qweight, const Array& qzeros, const Array& scales, const Array* g_idx,
                          size_t in_features, size_t out_features, size_t group_size, const Stream* stream = nullptr) {
  Array out = Array::uninit({in_features, out_features}, DType::Float32);
  detail::check(rmlx_hip_gptq_dequant(qweight.data(), qweight.nbytes(), qzeros.data(), qzeros.nbytes(), scales.data(),
                                      scales.nbytes(), g_idx != nullptr ? static_cast<const int32_t*>(g_idx->data()) : nullptr,
                                      g_idx != nullptr ? g_idx->nbytes() : 0, in_features, out_features, group_size,
                                      out.data(), out.nbytes(), raw(stream)));
  return out;
}

}  // namespace quantized

namespace topk_route {

// `TopkRouteResult` (topk_route.rs:396-407)
struct TopkRouteResult {
  Array expert_indices;    // u32 [T*K]
  Array expert_weights;    // f32 [T*K]
  Array expert_counts;     // u32 [E]
  Array dispatch_offsets;  // u32 [E+1]
};

inline TopkRouteResult gpu_topk_route(const Array& gate_logits, size_t top_k, const Array* expert_bias = nullptr,
                                      const Stream* stream = nullptr, bool renormalize = true) {
  const size_t t = gate_logits.ndim() == 2 ? gate_logits.shape()[0] : 0, e = gate_logits.ndim() == 2 ? gate_logits.shape()[1] : 0;
  const size_t k = top_k > 8 ? 8 : top_k;
  TopkRouteResult r{Array::uninit({t * k}, DType::UInt32), Array::uninit({t * k}, DType::Float32),
                    Array::uninit({e}, DType::UInt32), Array::uninit({e + 1}, DType::UInt32)};
  const rmlx_array g = gate_logits.view();
  rmlx_array b{};
  if (expert_bias != nullptr) b = expert_bias->view();
  detail::check(rmlx_hip_topk_route(&g, top_k, expert_bias != nullptr ? &b : nullptr, renormalize ? 1 : 0,
                                    static_cast<uint32_t*>(r.expert_indices.data()),
                                    static_cast<float*>(r.expert_weights.data()),
                                    static_cast<uint32_t*>(r.expert_counts.data()),
                                    static_cast<uint32_t*>(r.dispatch_offsets.data()), raw(stream)));
  return r;
}

}  // namespace topk_route
}  // namespace ops

namespace nn {

// `QuantizedLinear` (quantized_linear.rs:77-201) with weights resident on the device (the reference
// uploads them on every forward, :189).
class QuantizedLinear {
 public:
  QuantizedLinear(std::shared_ptr<ops::quantized::QuantizedWeight> weight, std::shared_ptr<Buffer> bias_f16 = nullptr)
      : weight_(std::move(weight)), bias_(std::move(bias_f16)) {}
  // x [in] or [batch, in] -> f16 [out] or [batch, out]
  Array forward(const Array& x, const Stream* stream = nullptr) const {
    const bool one_d = x.ndim() == 1;
    const size_t batch = one_d ? 1 : (x.ndim() == 2 ? x.shape()[0] : 0);
    Array out = one_d ? Array::uninit({weight_->out_features}, DType::Float16)
                      : Array::uninit({batch, weight_->out_features}, DType::Float16);
    const rmlx_array v = x.view();
    detail::check(rmlx_hip_quantized_linear_forward(weight_->handle(), &v, bias_ ? bias_->ptr() : nullptr, out.data(),
                                                    out.nbytes(), raw(stream)));
    return out;
  }
  const ops::quantized::QuantizedWeight& weight() const { return *weight_; }

 private:
  std::shared_ptr<ops::quantized::QuantizedWeight> weight_;
  std::shared_ptr<Buffer> bias_;
};

// `ExpertGroup::grouped_forward` (crates/rmlx-nn/src/expert_group.rs:308-533): (expert_idx, input) pairs
// in, one output per pair out.  Inputs are f16 [batch_i, D].
class ExpertGroup {
 public:
  ExpertGroup(std::shared_ptr<ops::quantized::QuantizedWeight> gate, std::shared_ptr<ops::quantized::QuantizedWeight> up,
              std::shared_ptr<ops::quantized::QuantizedWeight> down)
      : gate_(std::move(gate)), up_(std::move(up)), down_(std::move(down)) {}
  std::vector<Array> grouped_forward(const std::vector<std::pair<size_t, Array>>& batches,
                                     const Stream* stream = nullptr) const {
    std::vector<Array> outs;
    if (batches.empty()) return outs;
    const size_t d = gate_->in_features;
    std::vector<uint32_t> idx, rows;
    size_t total = 0;
    for (const auto& b : batches) {
      if (b.second.ndim() != 2 || b.second.shape()[1] != d || b.second.dtype() != DType::Float16)
        throw KernelError(KernelError::Kind::InvalidShape, "grouped_forward: every input must be Float16 [batch, " +
                                                               std::to_string(d) + "]");
      idx.push_back(static_cast<uint32_t>(b.first));
      rows.push_back(static_cast<uint32_t>(b.second.shape()[0]));
      total += b.second.shape()[0];
    }
    // pack the inputs one after another, run one grouped launch sequence, hand out views of the result
    Array x = Array::uninit({total, d}, DType::Float16);
    size_t at = 0;
    for (const auto& b : batches) {
      if (b.second.nbytes() != 0)
        detail::check(rmlx_hip_memcpy_d2d(static_cast<char*>(x.data()) + at, b.second.data(), b.second.nbytes(), raw(stream)));
      at += b.second.nbytes();
    }
    Array out = Array::uninit({total, down_->out_features}, DType::Float16);
    const rmlx_array v = x.view();
    detail::check(rmlx_hip_expert_group_grouped_forward(gate_->handle(), up_ ? up_->handle() : nullptr, down_->handle(),
                                                        batches.size(), idx.data(), rows.data(), &v, out.data(),
                                                        out.nbytes(), raw(stream)));
    at = 0;
    for (size_t i = 0; i < batches.size(); ++i) {
      outs.emplace_back(out.buffer(), std::vector<size_t>{rows[i], down_->out_features}, DType::Float16, at);
      at += size_t(rows[i]) * down_->out_features * 2;
    }
    return outs;
  }

 private:
  std::shared_ptr<ops::quantized::QuantizedWeight> gate_, up_, down_;
};

// The routed-expert block of `MoeLayer` (moe.rs:1391-1508) over stacked Q4 expert weights: gate / up
// [E, I, D] (or one fused [E, 2I, D] weight with `up` null) and down [E, D, I].
class MoeExperts {
 public:
  MoeExperts(std::shared_ptr<ops::quantized::QuantizedWeight> gate, std::shared_ptr<ops::quantized::QuantizedWeight> up,
             std::shared_ptr<ops::quantized::QuantizedWeight> down)
      : gate_(std::move(gate)), up_(std::move(up)), down_(std::move(down)) {}
  // x [T, D], expert_indices u32 [T*K], expert_weights f32 [T*K] (device) -> f16 [T, D]
  Array forward_grouped(const Array& x, const Array& expert_indices, const Array& expert_weights, size_t top_k,
                        const Stream* stream = nullptr) const {
    const size_t t = x.ndim() == 2 ? x.shape()[0] : 0, d = x.ndim() == 2 ? x.shape()[1] : 0;
    Array out = Array::uninit({t, d}, DType::Float16);
    const rmlx_array v = x.view();
    detail::check(rmlx_hip_moe_forward_grouped(gate_->handle(), up_ ? up_->handle() : nullptr, down_->handle(), &v,
                                               static_cast<const uint32_t*>(expert_indices.data()),
                                               static_cast<const float*>(expert_weights.data()), top_k, out.data(),
                                               out.nbytes(), raw(stream)));
    return out;
  }
  // Average rows per expert from which the expert projections of this layer run on the grouped MFMA GEMM instead
  // of the streaming GEMV; 0 = never.  Kept in the gate weight's handle (so an ExpertGroup over the same weights
  // follows it); returns the previous value.
  uint32_t set_expert_gemm_min_rows(uint32_t min_rows) { return gate_->set_expert_gemm_min_rows(min_rows); }
  // Streaming kernel of decode-sized batches (0 = the library's choice; see rmlx_hip_qweight_set_expert_stream_kernel);
  // returns the previous value.
  uint32_t set_expert_stream_kernel(uint32_t kind) { return gate_->set_expert_stream_kernel(kind); }
  // routing included: gate_logits [T, E]
  Array forward(const Array& x, const Array& gate_logits, size_t top_k, const Array* expert_bias = nullptr,
                const Stream* stream = nullptr) const {
    const size_t t = x.ndim() == 2 ? x.shape()[0] : 0, d = x.ndim() == 2 ? x.shape()[1] : 0;
    Array out = Array::uninit({t, d}, DType::Float16);
    const rmlx_array v = x.view(), g = gate_logits.view();
    rmlx_array b{};
    if (expert_bias != nullptr) b = expert_bias->view();
    detail::check(rmlx_hip_moe_forward(gate_->handle(), up_ ? up_->handle() : nullptr, down_->handle(), &v, &g, top_k,
                                       expert_bias != nullptr ? &b : nullptr, out.data(), out.nbytes(), raw(stream)));
    return out;
  }

 private:
  std::shared_ptr<ops::quantized::QuantizedWeight> gate_, up_, down_;
};

}  // namespace nn
}  // namespace rmlx

#endif  // RMLX_OPS_HPP
