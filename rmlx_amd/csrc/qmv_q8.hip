// Streaming 8-bit quantized GEMV for gfx950 (M <= 16 rows per pass over the weights).
//
// Replaces the reference's affine_qmv_fast_q8 (crates/rmlx-core/src/ops/quantized.rs:620-695) and the
// small-M end of its Q8 ladder (:7718-7775), where the weights are streamed once per row.
//
// Same skeleton as the 4-bit kernel (qmv.hip): a workgroup is 8 independent waves that split K,
// every lane issues all 128-bit weight loads of a pass up front, the waves meet only in the final
// reduction.  What differs:
//   * A slab is 16 rows x 64 k = exactly one quantisation group (group size 64), so no row-splitting
//     trick is needed and all 16 accumulator rows carry activation rows: up to 16 rows per pass.
//   * Lane (n = lane%16, g = lane/16) holds the 16 bytes k = 16g..16g+15 of weight row n: two MFMA
//     operands of 8 values in natural order.  Bytes become f16 with one v_perm each pair
//     (0x6400 | q = 1024 + q); the offset is removed per (row, slab) as -1024 * sum(x).
//   * The activation operand needs no permutation, so it is loaded straight from global memory in
//     operand layout (lane (m, g) reads x[m][slab*64 + 16g .. +15]); sum(x) per (row, slab) comes
//     from one extra MFMA against a ones operand, which lands in the accumulator layout directly.
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kSpw = 4;  // slabs (64 k) per wave and pass

struct Q8Params {
  const uint32_t* w; const __half* s; const __half* b;
  const __half* x;
  __half* out;
  uint32_t K, ld_out, M, N;
};

// 8 bytes (two words) -> 8 f16 values 1024 + q, natural order.
__device__ __forceinline__ h8 bytes_to_f16_plus_1024(uint32_t w0, uint32_t w1) {
  u4 o;
  o.x = __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u);
  o.y = __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u);
  o.z = __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u);
  o.w = __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u);
  return __builtin_bit_cast(h8, o);
}

__global__ __launch_bounds__(kThreads) void qmv_q8_kernel(Q8Params p) {
  __shared__ float red[kWaves * 256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;  // weight row of the tile / k sub-block; also activation row n
  const uint32_t K = p.K, slabs_total = K >> 6, groups_per_row = K >> 6;
  const uint32_t row0 = blockIdx.y * 16;
  const uint32_t rows = p.M - row0 < 16u ? p.M - row0 : 16u;
  const uint32_t tile_row = blockIdx.x * 16;

  const u4* wrow = reinterpret_cast<const u4*>(p.w + (uint64_t)(tile_row + n) * (K >> 2)) + g;
  const __half* srow = p.s + (uint64_t)(tile_row + n) * groups_per_row;
  const __half* brow = p.b + (uint64_t)(tile_row + n) * groups_per_row;
  // activation operand: lane (m = n, g); rows past the chunk read the last valid row (never stored)
  const uint32_t xm = (uint32_t)n < rows ? (uint32_t)n : rows - 1;
  const u4* xrow = reinterpret_cast<const u4*>(p.x + (uint64_t)(row0 + xm) * K) + 2 * g;

  const h8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
  f4 F = {0.f, 0.f, 0.f, 0.f};

  for (uint32_t slab0 = 0; slab0 < slabs_total; slab0 += kWaves * kSpw) {
    const uint32_t sl = slab0 + wave * kSpw;  // first slab of this wave (K % 2048 == 0: always in range)
    // ---- every load of the pass, small ones first (the memory counter retires in order) -----
    u4 xa[kSpw][2];
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      xa[it][0] = xrow[(uint64_t)(sl + it) * 8];
      xa[it][1] = xrow[(uint64_t)(sl + it) * 8 + 1];
    }
    const uint2 sv = *reinterpret_cast<const uint2*>(srow + sl);  // scales of the 4 slabs (8-byte aligned: sl % 4 == 0)
    const uint2 bv = *reinterpret_cast<const uint2*>(brow + sl);
    u4 wreg[kSpw];
#pragma unroll
    for (int it = 0; it < kSpw; ++it) wreg[it] = wrow[(uint64_t)(sl + it) * 4];

    // ---- sum(x) per (row, slab) on the matrix unit while the weights are in flight ---------------
    f4 xs[kSpw], c[kSpw];
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      xs[it] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        xs[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][jj]), ones, xs[it], 0, 0, 0);
    }
    // ---- integer dot per slab, then acc += scale * (dot - 1024 * sum(x)) + bias * sum(x) -------------
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      c[it] = (f4){0.f, 0.f, 0.f, 0.f};
      c[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][0]),
                                                     bytes_to_f16_plus_1024(wreg[it].x, wreg[it].y), c[it], 0, 0, 0);
      c[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][1]),
                                                     bytes_to_f16_plus_1024(wreg[it].z, wreg[it].w), c[it], 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      const uint32_t sw = it < 2 ? sv.x : sv.y, bw = it < 2 ? bv.x : bv.y;
      const float sc = __half2float(__ushort_as_half((unsigned short)((it & 1) ? sw >> 16 : sw & 0xFFFFu)));
      const float bi = __half2float(__ushort_as_half((unsigned short)((it & 1) ? bw >> 16 : bw & 0xFFFFu)));
#pragma unroll
      for (int i = 0; i < 4; ++i) F[i] += sc * (c[it][i] - 1024.0f * xs[it][i]) + bi * xs[it][i];
    }
  }

  // ---- reduce over the 8 k-parts, write out: accumulator lane (n, g) holds rows 4g..4g+3 of column n ----
#pragma unroll
  for (int i = 0; i < 4; ++i) red[(wave * 16 + g * 4 + i) * 16 + n] = F[i];
  __syncthreads();
  if (tid < 256) {
    const uint32_t m = tid >> 4, nn = tid & 15;
    if (m < rows) {
      float acc = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) acc += red[(w * 16 + m) * 16 + nn];
      p.out[(uint64_t)(row0 + m) * p.ld_out + tile_row + nn] = __float2half(acc);
    }
  }
}

}  // namespace

bool qmv_q8_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  return group_size == 64 && N > 0 && K > 0 && N % 16 == 0 && K % (64 * kWaves * kSpw) == 0;
}

int32_t launch_qmv_q8(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, hipStream_t stream) {
  if (!qmv_q8_supported(N, K, 64))
    return fail(RMLX_INVALID_SHAPE, "qmv_q8: N %% 16 and K %% 2048 required (N=%u K=%u)", N, K);
  if (M == 0) return RMLX_OK;
  Q8Params p{w, s, b, x, out, K, N, M, N};
  hipLaunchKernelGGL(qmv_q8_kernel, dim3(N / 16, (M + 15) / 16), dim3(kThreads), 0, stream, p);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
