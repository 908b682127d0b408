// Machine floors the throughput figures are read against: an empty launch, a plain streaming read, a loop of
// matrix instructions (alone and with vector-ALU work beside it), a loop of LDS reads.  They are launched through the same C ABI, on the same stream and timed by the same events
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

// one v_and_or_b32 the compiler neither merges nor drops
__device__ __forceinline__ void and_or(uint32_t& d, uint32_t a, uint32_t m, uint32_t k) {
  asm volatile("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(m), "v"(k));
}

// The same loop with V cheap vector-ALU instructions (and-or on registers of their own, the unpacking instruction
// of the 4-bit kernels) behind every MFMA: what the matrix unit still delivers while the vector ALU of the same
// SIMD runs a dequantisation beside it.
template <int V>
__global__ __launch_bounds__(512) void floor_mfma_valu_kernel(uint32_t iters, float* __restrict__ sink) {
  f16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (_Float16)(float)((threadIdx.x + i) & 3);
    b[i] = (_Float16)(float)((threadIdx.x * 3 + i) & 1);
  }
  uint32_t w[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) w[i] = threadIdx.x * 2654435761u + i;
  uint32_t m = 0x000F000Fu, k = 0x64006400u;
  asm volatile("" : "+s"(m), "+v"(k));
  f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c0, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < V; ++v) and_or(w[v % 8], w[(v + 1) % 8], m, k);
      c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c1, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < V; ++v) and_or(w[(v + 2) % 8], w[(v + 3) % 8], m, k);
      c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c2, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < V; ++v) and_or(w[(v + 4) % 8], w[(v + 5) % 8], m, k);
      c3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c3, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < V; ++v) and_or(w[(v + 6) % 8], w[(v + 7) % 8], m, k);
    }
  }
  const f32x4 s = c0 + c1 + c2 + c3;
  uint32_t x = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) x ^= w[i];
  if (s[0] + s[1] + s[2] + s[3] == -1.0f || x == 0x9E3779B9u) sink[0] = s[0];
}

// `iters` rounds of four 16-byte loads per lane from a small source that every workgroup walks in full (starting at
// its own offset): after the first pass the loads hit the L2 of the workgroup's XCD, so the rate is what L2 hits
// deliver to the CUs.  n_vec is a power of two.
__global__ __launch_bounds__(512) void floor_l2_read_kernel(const u32x4* __restrict__ src, uint32_t n_vec, uint32_t iters,
                                                           uint32_t* __restrict__ sink) {
  u32x4 acc = {0, 0, 0, 0};
  uint32_t at = blockIdx.x * 2048 + threadIdx.x;
  for (uint32_t it = 0; it < iters; ++it) {
    u32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = src[(at + i * 512) & (n_vec - 1)];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc ^= v[i];
    at += 2048;
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u) sink[0] = 1;
}

// `iters` rounds of eight 16-byte LDS reads per lane (consecutive lanes read consecutive 16 bytes: no bank
// conflicts), WAVES waves per workgroup, one workgroup per CU and launch slot: the rate at which a CU's LDS feeds
// operands.  64 KB of LDS per workgroup.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void floor_lds_kernel(uint32_t iters, uint32_t* __restrict__ sink) {
  __shared__ u32x4 buf[4096];
  for (int i = threadIdx.x; i < 4096; i += WAVES * 64) buf[i] = u32x4{(uint32_t)i, 1u, 2u, 3u};
  __syncthreads();
  u32x4 acc = {0, 0, 0, 0};
  uint32_t at = threadIdx.x;
  for (uint32_t it = 0; it < iters; ++it) {
    u32x4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = buf[(at + i * 512) & 4095];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc ^= v[i];
    at += 64;
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u) sink[0] = 1;
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
  } else if (kind == RMLX_FLOOR_MFMA_VALU) {
    if (sink_dev == nullptr || iters == 0) return fail(RMLX_INVALID_SHAPE, "measure_floor: the MFMA loop needs a sink and iters > 0");
    const unsigned blocks = (unsigned)(bytes == 0 ? 2 * (size_t)ctx().num_cus : bytes);
    for (size_t i = 0; i < count; ++i) {  // `n_src` doubles as the vector instructions per MFMA
      float* sk = static_cast<float*>(sink_dev);
      switch (n_src) {
        case 2: hipLaunchKernelGGL(floor_mfma_valu_kernel<2>, dim3(blocks), dim3(512), 0, s, iters, sk); break;
        case 4: hipLaunchKernelGGL(floor_mfma_valu_kernel<4>, dim3(blocks), dim3(512), 0, s, iters, sk); break;
        case 6: hipLaunchKernelGGL(floor_mfma_valu_kernel<6>, dim3(blocks), dim3(512), 0, s, iters, sk); break;
        case 8: hipLaunchKernelGGL(floor_mfma_valu_kernel<8>, dim3(blocks), dim3(512), 0, s, iters, sk); break;
        default: return fail(RMLX_INVALID_SHAPE, "measure_floor: 2, 4, 6 or 8 vector instructions per MFMA (n_src=%zu)", n_src);
      }
    }
  } else if (kind == RMLX_FLOOR_L2_READ) {
    if (src_dev == nullptr || sink_dev == nullptr || iters == 0 || bytes < 32768 || (bytes & (bytes - 1)) != 0 || bytes > (1u << 30))
      return fail(RMLX_INVALID_SHAPE, "measure_floor: the L2 read needs a source of 2^n bytes (32 KB .. 1 GB) and iters > 0");
    const unsigned blocks = (unsigned)(n_src == 0 ? 2 * (size_t)ctx().num_cus : n_src);  // `n_src` doubles as the workgroup count
    for (size_t i = 0; i < count; ++i)
      hipLaunchKernelGGL(floor_l2_read_kernel, dim3(blocks), dim3(512), 0, s, static_cast<const u32x4*>(src_dev),
                         (uint32_t)(bytes / 16), iters, static_cast<uint32_t*>(sink_dev));
  } else if (kind == RMLX_FLOOR_LDS) {
    if (sink_dev == nullptr || iters == 0) return fail(RMLX_INVALID_SHAPE, "measure_floor: the LDS loop needs a sink and iters > 0");
    const unsigned blocks = (unsigned)(bytes == 0 ? (size_t)ctx().num_cus : bytes);
    for (size_t i = 0; i < count; ++i) {  // `n_src` doubles as the waves per workgroup (8 or 16)
      if (n_src == 16) hipLaunchKernelGGL(floor_lds_kernel<16>, dim3(blocks), dim3(1024), 0, s, iters, static_cast<uint32_t*>(sink_dev));
      else hipLaunchKernelGGL(floor_lds_kernel<8>, dim3(blocks), dim3(512), 0, s, iters, static_cast<uint32_t*>(sink_dev));
    }
  } else {
    return fail(RMLX_NOT_FOUND, "measure_floor: unknown kind %d", kind);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return finish(s);
}
