// Machine floors the throughput figures are read against: an empty launch, a plain streaming read, a loop of
// matrix instructions.  They are launched through the same C ABI, on the same stream and timed by the same events
// as the matmul kernels, so a benchmark can put "what this GPU does with nothing but the loads / nothing but the
// MFMAs" beside every measured kernel.  No counterpart in the reference.
#include "common.hpp"

namespace rmlx {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ void floor_empty_kernel() {}

// Every lane issues U 16-byte non-temporal loads (a wave-wide load covers 1 KB contiguous) before it consumes the
// first; a workgroup of 512 threads reads U * 8 KB.  Nothing is written unless the xor of all words hits a magic
// value, which keeps the loads alive without a store stream.
template <int U>
__global__ __launch_bounds__(512) void floor_read_kernel(const u32x4* __restrict__ src, size_t n_vec, uint32_t* __restrict__ sink) {
  const size_t base = (size_t)blockIdx.x * (512 * U) + threadIdx.x;
  u32x4 v[U];
#pragma unroll
  for (int i = 0; i < U; ++i) {
    const size_t j = base + (size_t)i * 512;
    v[i] = j < n_vec ? __builtin_nontemporal_load(src + j) : u32x4{0, 0, 0, 0};
  }
  u32x4 acc = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < U; ++i) acc ^= v[i];
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u) sink[0] = 1;
}

// `iters` rounds of 16 independent 16x16x32 f16 MFMAs per wave (four accumulators, four products each): nothing
// but matrix instructions and the loop counter.  8 waves per workgroup.
__global__ __launch_bounds__(512) void floor_mfma_kernel(uint32_t iters, float* __restrict__ sink) {
  f16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (_Float16)(float)((threadIdx.x + i) & 3);
    b[i] = (_Float16)(float)((threadIdx.x * 3 + i) & 1);
  }
  f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c3, 0, 0, 0);
    }
  }
  const f32x4 s = c0 + c1 + c2 + c3;
  if (s[0] + s[1] + s[2] + s[3] == -1.0f) sink[0] = s[0];
}

}  // namespace
}  // namespace rmlx

using namespace rmlx;

extern "C" int32_t rmlx_hip_measure_floor(int32_t kind, const void* src_dev, size_t bytes, size_t n_src, uint32_t iters,
                                          void* sink_dev, size_t count, rmlx_stream stream) {
  RMLX_TRY(require_init());
  hipStream_t s = (hipStream_t)stream;
  if (kind == RMLX_FLOOR_EMPTY) {
    for (size_t i = 0; i < count; ++i) hipLaunchKernelGGL(floor_empty_kernel, dim3(1), dim3(64), 0, s);
  } else if (kind == RMLX_FLOOR_READ4 || kind == RMLX_FLOOR_READ8 || kind == RMLX_FLOOR_READ2) {
    if (src_dev == nullptr || sink_dev == nullptr || bytes == 0 || bytes % 16 != 0 || n_src == 0 ||
        (reinterpret_cast<uintptr_t>(src_dev) & 15u) != 0)
      return fail(RMLX_INVALID_SHAPE, "measure_floor: the read needs a 16-byte aligned source of n_src * bytes bytes, bytes %% 16 == 0");
    const size_t n_vec = bytes / 16;
    const int u = kind == RMLX_FLOOR_READ2 ? 2 : (kind == RMLX_FLOOR_READ4 ? 4 : 8);
    const size_t blocks = (n_vec + 512 * (size_t)u - 1) / (512 * (size_t)u);
    if (blocks > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "measure_floor: %zu bytes is too large for one launch", bytes);
    for (size_t i = 0; i < count; ++i) {  // the n_src consecutive copies are read in turn
      const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const char*>(src_dev) + (i % n_src) * bytes);
      if (u == 2) hipLaunchKernelGGL(floor_read_kernel<2>, dim3((unsigned)blocks), dim3(512), 0, s, p, n_vec, static_cast<uint32_t*>(sink_dev));
      else if (u == 4) hipLaunchKernelGGL(floor_read_kernel<4>, dim3((unsigned)blocks), dim3(512), 0, s, p, n_vec, static_cast<uint32_t*>(sink_dev));
      else hipLaunchKernelGGL(floor_read_kernel<8>, dim3((unsigned)blocks), dim3(512), 0, s, p, n_vec, static_cast<uint32_t*>(sink_dev));
    }
  } else if (kind == RMLX_FLOOR_MFMA) {
    if (sink_dev == nullptr || iters == 0) return fail(RMLX_INVALID_SHAPE, "measure_floor: the MFMA loop needs a sink and iters > 0");
    const unsigned blocks = (unsigned)(bytes == 0 ? 2 * (size_t)ctx().num_cus : bytes);  // `bytes` doubles as the workgroup count
    for (size_t i = 0; i < count; ++i)
      hipLaunchKernelGGL(floor_mfma_kernel, dim3(blocks), dim3(512), 0, s, iters, static_cast<float*>(sink_dev));
  } else {
    return fail(RMLX_NOT_FOUND, "measure_floor: unknown kind %d", kind);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return finish(s);
}
