// Portable kernels: the scalar quantized matmul that accepts every bit width / group size the
// QuantizedWeight type admits (the role of the reference's generic `affine_qmv`,
// crates/rmlx-core/src/ops/quantized.rs:210-291, and scalar `affine_qmm`, :2871-2937, and
// `gather_qmm_f32`, :9300-9368), dtype casts, bias add and index validation.
#include "common.hpp"

namespace rmlx {
namespace {

__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }

__global__ void cast_to_f16_kernel(const void* src, int src_dtype, __half* dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = src_dtype == RMLX_DTYPE_F32 ? reinterpret_cast<const float*>(src)[i]
                                          : bf16_to_f32(reinterpret_cast<const uint16_t*>(src)[i]);
    dst[i] = __float2half(v);
  }
}

// RMSNorm prologue as a pass of its own (the kernels without a fused prologue): the reference's A loader
// computes half(x) * half(inv_rms[row]) * norm_weight[k] in half precision (quantized.rs:3070-3095)
__global__ void norm_rows_kernel(const void* src, int src_dtype, const __half* __restrict__ norm_w,
                                 const float* __restrict__ inv_rms, uint32_t K, __half* dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const _Float16 xh = src_dtype == RMLX_DTYPE_F16 ? reinterpret_cast<const _Float16*>(src)[i]
                        : src_dtype == RMLX_DTYPE_F32 ? (_Float16)reinterpret_cast<const float*>(src)[i]
                                                      : (_Float16)bf16_to_f32(reinterpret_cast<const uint16_t*>(src)[i]);
    const _Float16 rs = (_Float16)inv_rms[i / K];
    const _Float16 scaled = xh * rs;
    reinterpret_cast<_Float16*>(dst)[i] = scaled * reinterpret_cast<const _Float16*>(norm_w)[i % K];
  }
}

__global__ void cast_f16_to_f32_kernel(const __half* src, float* dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = __half2float(src[i]);
}

// One wave per weight row; lanes stride over the packed words of the row; up to 4 activation
// rows per pass share each unpacked word.  f32 accumulation of scale*q*x + bias*x per value.
constexpr int kGenRows = 4;
__global__ __launch_bounds__(64) void generic_qmm_kernel(GenericArgs a) {
  // blockIdx.y enumerates (batch, pass): a pass covers up to kGenRows rows of one batch, so all
  // rows of a pass use the same expert.  Without indices there is a single batch of M rows.
  const uint32_t nrow = blockIdx.x;
  const uint32_t rpi = a.rows_per_index;
  const uint32_t passes = (rpi + kGenRows - 1) / kGenRows;
  const uint32_t batch = blockIdx.y / passes;
  const uint32_t m0 = batch * rpi + (blockIdx.y % passes) * kGenRows;
  const uint32_t mend = (batch + 1) * rpi < a.M ? (batch + 1) * rpi : a.M;
  const uint32_t lane = threadIdx.x;
  // Layout of the reference's affine_qmv (quantized.rs:210-291): 32 / bits values per word, group_size / (32 / bits)
  // words per group, a row is its groups' words one after another.  At 2, 4 and 8 bits that is the flat packing; at
  // 3 and 6 bits a word holds 10 / 5 values (2 bits unused) and the values of a group past its last whole word
  // (2 of 32, 4 of 64, 8 of 128) have no word: they count for nothing, in the product and in the bias term alike.
  const uint32_t per = 32 / a.bits;
  const uint32_t wpg = a.group_size / per;
  const uint32_t gpr = a.K / a.group_size;
  const uint32_t words = gpr * wpg;
  const uint32_t mask = (1u << a.bits) - 1u;

  float acc[kGenRows] = {0.f, 0.f, 0.f, 0.f};
  uint32_t expert = 0;
  bool valid = true;
  if (a.indices != nullptr) {
    expert = a.indices[batch];
    valid = expert < a.n_experts;
  }
  if (valid) {
    const uint32_t* wrow = a.w + ((uint64_t)expert * a.N + nrow) * words;
    const __half* srow = a.s + ((uint64_t)expert * a.N + nrow) * gpr;
    const __half* brow = a.b + ((uint64_t)expert * a.N + nrow) * gpr;
    for (uint32_t wi = lane; wi < words; wi += 64) {
      const uint32_t word = wrow[wi];
      const uint32_t grp = wi / wpg, kbase = grp * a.group_size + (wi % wpg) * per;
      for (uint32_t i = 0; i < per; ++i) {
        const uint32_t k = kbase + i;
        const float q = (float)((word >> (i * a.bits)) & mask);
        const float wv = __half2float(srow[grp]) * q + __half2float(brow[grp]);
#pragma unroll
        for (int r = 0; r < kGenRows; ++r)
          if (m0 + r < mend) acc[r] += wv * __half2float(a.x[(uint64_t)(m0 + r) * a.K + k]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kGenRows; ++r) {
    float v = acc[r];
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0 && m0 + r < mend) a.out[(uint64_t)(m0 + r) * a.N + nrow] = __float2half(v);
  }
}

__global__ void add_bias_rows_kernel(__half* out, const __half* bias, uint32_t M, uint32_t N) {
  const size_t total = (size_t)M * N;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride)
    out[i] = __float2half(__half2float(out[i]) + __half2float(bias[i % N]));
}

__global__ void check_indices_kernel(const uint32_t* idx, uint32_t n, uint32_t limit, uint32_t* flag) {
  uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && idx[i] >= limit) atomicMin(flag, i);  // first offending position
}

}  // namespace

int32_t launch_cast_to_f16(const void* src, int32_t src_dtype, __half* dst, size_t n, hipStream_t s) {
  if (n == 0) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(cast_to_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, s, src, src_dtype, dst, n);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_norm_rows(const void* x, int32_t x_dtype, const __half* norm_w, const float* inv_rms, uint32_t M,
                         uint32_t K, __half* dst, hipStream_t s) {
  const size_t n = (size_t)M * K;
  if (n == 0) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(norm_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, x_dtype, norm_w, inv_rms, K, dst, n);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_cast_f16_to_f32(const __half* src, float* dst, size_t n, hipStream_t s) {
  if (n == 0) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(cast_f16_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, src, dst, n);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_generic(const GenericArgs& a, hipStream_t s) {
  if (a.M == 0 || a.N == 0) return RMLX_OK;
  if (a.bits != 2 && a.bits != 3 && a.bits != 4 && a.bits != 6 && a.bits != 8)
    return fail(RMLX_NOT_FOUND, "no kernel for %u-bit weights", a.bits);
  GenericArgs k = a;
  if (k.indices == nullptr) k.rows_per_index = a.M;
  const uint32_t batches = (a.M + k.rows_per_index - 1) / k.rows_per_index;
  const uint32_t passes = (k.rows_per_index + kGenRows - 1) / kGenRows;
  hipLaunchKernelGGL(generic_qmm_kernel, dim3(a.N, batches * passes), dim3(64), 0, s, k);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_add_bias_rows(__half* out, const __half* bias, uint32_t M, uint32_t N, hipStream_t s) {
  size_t total = (size_t)M * N;
  if (total == 0) return RMLX_OK;
  size_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(add_bias_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, out, bias, M, N);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_check_indices(const uint32_t* idx, uint32_t n, uint32_t limit, uint32_t* flag, hipStream_t s) {
  if (n == 0) return RMLX_OK;
  hipLaunchKernelGGL(check_indices_kernel, dim3((n + 255) / 256), dim3(256), 0, s, idx, n, limit, flag);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

namespace {
__global__ void epilogue_kernel(__half* __restrict__ out, int kind, const void* __restrict__ e, int32_t e_dtype, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float ev = e_dtype == RMLX_DTYPE_F32 ? static_cast<const float*>(e)[i] : __half2float(static_cast<const __half*>(e)[i]);
    const float v = __half2float(out[i]);
    out[i] = __float2half(kind == EPI_RESIDUAL ? v + ev : ev / (1.0f + __expf(-ev)) * v);
  }
}
}  // namespace

int32_t launch_epilogue(__half* out, int kind, const void* e, int32_t e_dtype, size_t n, hipStream_t s) {
  if (n == 0 || kind == EPI_NONE) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(epilogue_kernel, dim3((unsigned)blocks), dim3(256), 0, s, out, kind, e, e_dtype, n);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
