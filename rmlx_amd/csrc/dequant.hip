// AWQ / GPTQ INT4 -> f32 dequantisation (crates/rmlx-core/src/ops/quantized.rs:707-783; hosts :2269-2383
// and :2407-2590).  Pure streaming: every output element is written once (4 bytes) and costs half a byte of
// packed weight plus a share of one zero-point word and one scale, so the kernels are bound by the f32
// store stream.  Both move 16 bytes per lane per access:
//   awq_dequant_kernel   lane = 4 adjacent columns of 8 consecutive rows   (packing runs along columns)
//   gptq_dequant_kernel  lane = 4 adjacent columns of the 8 rows one packed word row holds (packing runs
//                        along rows), so one 16-byte load feeds eight 16-byte stores
// and a one-element-per-thread kernel takes the cases whose pointers are not 16-byte aligned.
#include "common.hpp"

namespace rmlx {
namespace {

constexpr int kThreads = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void store4(float* dst, float4 o) {
  f32x4 v = {o.x, o.y, o.z, o.w};
  __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dst));
}

__device__ __forceinline__ float4 dequant4(uint32_t q, uint32_t z, int zero_plus, float4 s) {
  // q, z: four nibbles in the low 16 bits
  float4 o;
  o.x = s.x * ((float)(q & 0xF) - (float)((z & 0xF) + zero_plus));
  o.y = s.y * ((float)((q >> 4) & 0xF) - (float)(((z >> 4) & 0xF) + zero_plus));
  o.z = s.z * ((float)((q >> 8) & 0xF) - (float)(((z >> 8) & 0xF) + zero_plus));
  o.w = s.w * ((float)((q >> 12) & 0xF) - (float)(((z >> 12) & 0xF) + zero_plus));
  return o;
}

constexpr int kAwqRows = 8;  // rows per lane: 128 bytes of output per lane, as in the GPTQ kernel

// grid = row blocks of kAwqRows x column blocks of 4*kThreads, the column block varying fastest so that
// the workgroups in flight together cover contiguous memory
__global__ __launch_bounds__(kThreads) void awq_dequant_kernel(const uint32_t* __restrict__ qweight,
                                                               const uint32_t* __restrict__ qzeros,
                                                               const float* __restrict__ scales,
                                                               float* __restrict__ out, uint32_t rows, uint32_t cols,
                                                               uint32_t group_size, uint32_t col_blocks) {
  const uint32_t quad = (blockIdx.x % col_blocks) * kThreads + threadIdx.x;  // columns 4*quad .. 4*quad+3
  if (quad * 4 >= cols) return;
  const uint32_t r0 = (blockIdx.x / col_blocks) * kAwqRows;
  const uint32_t words = cols / 8;
  const uint32_t shift = (quad & 1) * 16;
  // Lanes 2j and 2j+1 share the packed words of columns 8j..8j+7: the even lane fetches those of the even
  // rows, the odd lane those of the odd rows, and one lane swap hands each the other's word.
  uint32_t q[kAwqRows], g[kAwqRows];
#pragma unroll
  for (int i = 0; i < kAwqRows; i += 2) {
    const uint32_t mine = r0 + i + (quad & 1);
    const uint32_t r = mine < rows ? mine : rows - 1;
    const uint32_t w = qweight[(size_t)r * words + quad / 2];
    const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xB1, 0xF, 0xF, true);  // lane ^ 1
    q[i] = (quad & 1) ? other : w;
    q[i + 1] = (quad & 1) ? w : other;
  }
#pragma unroll
  for (int i = 0; i < kAwqRows; ++i) g[i] = (r0 + i < rows ? r0 + i : rows - 1) / group_size;
  uint32_t z[kAwqRows];
  float4 s[kAwqRows];
#pragma unroll
  for (int i = 0; i < kAwqRows; ++i) {
    z[i] = qzeros[(size_t)g[i] * words + quad / 2];
    s[i] = *reinterpret_cast<const float4*>(scales + (size_t)g[i] * cols + quad * 4);
  }
#pragma unroll
  for (int i = 0; i < kAwqRows; ++i) {
    if (r0 + i < rows) {
      const float4 o = dequant4(q[i] >> shift, z[i] >> shift, 0, s[i]);
      store4(out + (size_t)(r0 + i) * cols + quad * 4, o);
    }
  }
}

// grid = packed rows x column blocks of 4*kThreads, the column block varying fastest.  Rows whose group index is outside
// [0, num_groups) -- only possible through g_idx -- are written as zeros.
__global__ __launch_bounds__(kThreads) void gptq_dequant_kernel(const uint32_t* __restrict__ qweight,
                                                                const uint32_t* __restrict__ qzeros,
                                                                const float* __restrict__ scales,
                                                                const int32_t* __restrict__ g_idx,
                                                                float* __restrict__ out, uint32_t out_features,
                                                                uint32_t group_size, uint32_t num_groups,
                                                                uint32_t col_blocks) {
  const uint32_t quad = (blockIdx.x % col_blocks) * kThreads + threadIdx.x;
  if (quad * 4 >= out_features) return;
  const uint32_t pr = blockIdx.x / col_blocks;
  const uint32_t zwords = out_features / 8;
  const uint32_t shift = (quad & 1) * 16;
  const uint4 w = *reinterpret_cast<const uint4*>(qweight + (size_t)pr * out_features + quad * 4);
  uint32_t g[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) g[r] = g_idx != nullptr ? (uint32_t)g_idx[pr * 8 + r] : (pr * 8 + r) / group_size;
  uint32_t z[8];
  float4 s[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const uint32_t gc = g[r] < num_groups ? g[r] : 0;
    z[r] = qzeros[(size_t)gc * zwords + quad / 2] >> shift;
    s[r] = *reinterpret_cast<const float4*>(scales + (size_t)gc * out_features + quad * 4);
    if (g[r] >= num_groups) s[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    // nibble r of each of the four words
    const uint32_t q = ((w.x >> (4 * r)) & 0xF) | (((w.y >> (4 * r)) & 0xF) << 4) | (((w.z >> (4 * r)) & 0xF) << 8) |
                       (((w.w >> (4 * r)) & 0xF) << 12);
    const float4 o = dequant4(q, z[r], 1, s[r]);
    store4(out + (size_t)(pr * 8 + r) * out_features + quad * 4, o);
  }
}

// One element per thread, any alignment.  GPTQ = true: qweight is [rows/8, cols], zero point + 1.
template <bool GPTQ>
__global__ __launch_bounds__(kThreads) void dequant_elem_kernel(const uint32_t* __restrict__ qweight,
                                                                const uint32_t* __restrict__ qzeros,
                                                                const float* __restrict__ scales,
                                                                const int32_t* __restrict__ g_idx,
                                                                float* __restrict__ out, uint32_t rows, uint32_t cols,
                                                                uint32_t group_size, uint32_t num_groups) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= (size_t)rows * cols) return;
  const uint32_t row = (uint32_t)(i / cols), col = (uint32_t)(i % cols);
  const uint32_t g = (GPTQ && g_idx != nullptr) ? (uint32_t)g_idx[row] : row / group_size;
  if (g >= num_groups) {
    out[i] = 0.f;
    return;
  }
  const uint32_t qw = GPTQ ? qweight[(size_t)(row / 8) * cols + col] : qweight[(size_t)row * (cols / 8) + col / 8];
  const uint32_t nib = (qw >> (4 * ((GPTQ ? row : col) % 8))) & 0xF;
  const uint32_t zero = ((qzeros[(size_t)g * (cols / 8) + col / 8] >> (4 * (col % 8))) & 0xF) + (GPTQ ? 1 : 0);
  out[i] = scales[(size_t)g * cols + col] * ((float)nib - (float)zero);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

int32_t launch_awq_dequant(const uint32_t* qweight, const uint32_t* qzeros, const float* scales, float* out,
                           uint32_t rows, uint32_t cols, uint32_t group_size, hipStream_t s) {
  if (rows == 0 || cols == 0) return RMLX_OK;
  const uint32_t num_groups = rows / group_size;
  if (aligned16(scales) && aligned16(out)) {
    const uint32_t col_blocks = (cols / 4 + kThreads - 1) / kThreads;
    const size_t blocks = (size_t)((rows + kAwqRows - 1) / kAwqRows) * col_blocks;
    if (blocks > 0x7fffffffull) return fail(RMLX_INVALID_SHAPE, "awq_dequant: matrix too large");
    hipLaunchKernelGGL(awq_dequant_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, s, qweight, qzeros, scales, out,
                       rows, cols, group_size, col_blocks);
  } else {
    const size_t blocks = ((size_t)rows * cols + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffull) return fail(RMLX_INVALID_SHAPE, "awq_dequant: matrix too large");
    hipLaunchKernelGGL(dequant_elem_kernel<false>, dim3((unsigned)blocks), dim3(kThreads), 0, s, qweight, qzeros,
                       scales, (const int32_t*)nullptr, out, rows, cols, group_size, num_groups);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_gptq_dequant(const uint32_t* qweight, const uint32_t* qzeros, const float* scales,
                            const int32_t* g_idx, float* out, uint32_t in_features, uint32_t out_features,
                            uint32_t group_size, uint32_t num_groups, hipStream_t s) {
  if (in_features == 0 || out_features == 0) return RMLX_OK;
  if (aligned16(qweight) && aligned16(scales) && aligned16(out)) {
    const uint32_t col_blocks = (out_features / 4 + kThreads - 1) / kThreads;
    const size_t blocks = (size_t)(in_features / 8) * col_blocks;
    if (blocks > 0x7fffffffull) return fail(RMLX_INVALID_SHAPE, "gptq_dequant: matrix too large");
    hipLaunchKernelGGL(gptq_dequant_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, s, qweight, qzeros, scales,
                       g_idx, out, out_features, group_size, num_groups, col_blocks);
  } else {
    const size_t blocks = ((size_t)in_features * out_features + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffull) return fail(RMLX_INVALID_SHAPE, "gptq_dequant: matrix too large");
    hipLaunchKernelGGL(dequant_elem_kernel<true>, dim3((unsigned)blocks), dim3(kThreads), 0, s, qweight, qzeros,
                       scales, g_idx, out, in_features, out_features, group_size, num_groups);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
