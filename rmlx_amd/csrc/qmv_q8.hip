// Streaming 8-bit quantized GEMV for gfx950 (M <= 16 rows per pass over the weights), also over a chunk
// table of (expert, rows) for the expert projections of the MoE block.
//
// Replaces the reference's affine_qmv_fast_q8 (crates/rmlx-core/src/ops/quantized.rs:620-695) and the
// small-M end of its Q8 ladder (:7718-7775), where the weights are streamed once per row.
//
// Same skeleton as the 4-bit kernel (qmv.hip): a workgroup is 8 independent waves that split K,
// every lane issues all 128-bit weight loads of a pass up front, the waves meet only in the final
// reduction.  What differs:
//   * A slab is 16 rows x 64 k = exactly one quantisation group (group size 64; at group size 128 two
//     neighbouring slabs share one), so no row-splitting trick is needed and all 16 accumulator rows
//     carry activation rows: up to 16 rows per pass.
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
  const uint32_t* w; const __half* s; const __half* b;      // tile set 0
  const uint32_t* w1; const __half* s1; const __half* b1;   // tile set 1 (fused gate / up)
  const __half* x;
  void* out;               // f16 (f32 when out_f32)
  uint32_t K, ld_out, M, out_f32;
  // chunk-table mode (expert projections): (expert, first row position, rows <= 16) per blockIdx.y
  const uint32_t* row_map;    // nullable: source row of position p
  const uint32_t* chunk_tab;
  const uint32_t* n_chunks;   // nullable: live chunks (device)
  uint64_t estride_w, estride_s;
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

// TAB: rows come from a device chunk table and the weights from the chunk's expert.  TILES == 2: the
// workgroup multiplies the same activations with a gate tile and an up tile and writes silu(gate) * up.
// A pass covers 32 slabs (2048 k); waves whose slabs lie past K sit it out, so K % 256 == 0 is enough.
// XBF: the activations are bf16 bits, converted to f16 in registers (through f32, rounded to nearest even: what the cast
// kernel does) once the pass's loads are issued.
__device__ __forceinline__ u4 bf16x8_to_f16x8(u4 v) {
  typedef _Float16 h2c __attribute__((ext_vector_type(2)));
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
    const h2c pair = {(_Float16)lo, (_Float16)hi};
    w[e] = __builtin_bit_cast(uint32_t, pair);
  }
  return (u4){w[0], w[1], w[2], w[3]};
}

template <bool TAB, int TILES, bool GS128, bool XBF = false>
__global__ __launch_bounds__(kThreads) void qmv_q8_kernel(Q8Params p) {
  __shared__ float red[kWaves * TILES * 256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;  // weight row of the tile / k sub-block; also activation row n
  const uint32_t K = p.K, slabs_total = K >> 6, groups_per_row = GS128 ? K >> 7 : K >> 6;
  uint32_t expert = 0, row0 = blockIdx.y * 16, rows;
  bool write_zeros = false;
  if (TAB) {
    if (p.n_chunks != nullptr && blockIdx.y >= *p.n_chunks) return;
    expert = p.chunk_tab[3 * blockIdx.y + 0];
    row0 = p.chunk_tab[3 * blockIdx.y + 1];
    rows = p.chunk_tab[3 * blockIdx.y + 2];
    write_zeros = (rows >> 31) != 0;
    rows &= 0x7FFFFFFFu;
    if (rows > 16u) rows = 16u;  // (the host builds chunks of at most 16 rows)
    if (rows == 0) return;
  } else {
    rows = p.M - row0 < 16u ? p.M - row0 : 16u;
  }
  const uint32_t tile_row = blockIdx.x * 16;

  const u4* wrow[TILES];
  const __half* srow[TILES];
  const __half* brow[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const uint64_t e_w = TAB ? expert * p.estride_w : 0, e_s = TAB ? expert * p.estride_s : 0;
    wrow[t] = reinterpret_cast<const u4*>((t == 0 ? p.w : p.w1) + e_w + (uint64_t)(tile_row + n) * (K >> 2)) + g;
    srow[t] = (t == 0 ? p.s : p.s1) + e_s + (uint64_t)(tile_row + n) * groups_per_row;
    brow[t] = (t == 0 ? p.b : p.b1) + e_s + (uint64_t)(tile_row + n) * groups_per_row;
  }
  // activation operand: lane (m = n, g); rows past the chunk read the last valid row (never stored)
  const uint32_t xm = (uint32_t)n < rows ? (uint32_t)n : rows - 1;
  uint32_t xsrc = row0 + xm;
  if (TAB && p.row_map != nullptr) xsrc = p.row_map[xsrc];
  const u4* xrow = reinterpret_cast<const u4*>(p.x + (uint64_t)xsrc * K) + 2 * g;

  const h8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
  f4 F[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};

  for (uint32_t slab0 = 0; slab0 < slabs_total && !write_zeros; slab0 += kWaves * kSpw) {
    const uint32_t sl = slab0 + wave * kSpw;  // first slab of this wave
    if (sl >= slabs_total) break;             // (whole waves: slabs_total is a multiple of kSpw)
    // ---- every load of the pass, small ones first (the memory counter retires in order) -----
    u4 xa[kSpw][2];
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      xa[it][0] = xrow[(uint64_t)(sl + it) * 8];
      xa[it][1] = xrow[(uint64_t)(sl + it) * 8 + 1];
    }
    uint2 sv[TILES], bv[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      if (GS128) {  // two groups for the four slabs: every value twice
        const uint32_t s2 = *reinterpret_cast<const uint32_t*>(srow[t] + (sl >> 1)), b2 = *reinterpret_cast<const uint32_t*>(brow[t] + (sl >> 1));
        sv[t] = make_uint2(__builtin_amdgcn_perm(s2, s2, 0x01000100u), __builtin_amdgcn_perm(s2, s2, 0x03020302u));
        bv[t] = make_uint2(__builtin_amdgcn_perm(b2, b2, 0x01000100u), __builtin_amdgcn_perm(b2, b2, 0x03020302u));
      } else {
        sv[t] = *reinterpret_cast<const uint2*>(srow[t] + sl);  // scales of the 4 slabs (8-byte aligned: sl % 4 == 0)
        bv[t] = *reinterpret_cast<const uint2*>(brow[t] + sl);
      }
    }
    u4 wreg[TILES][kSpw];
#pragma unroll
    for (int it = 0; it < kSpw; ++it)
#pragma unroll
      for (int t = 0; t < TILES; ++t) wreg[t][it] = wrow[t][(uint64_t)(sl + it) * 4];

    if constexpr (XBF) {
#pragma unroll
      for (int it = 0; it < kSpw; ++it) { xa[it][0] = bf16x8_to_f16x8(xa[it][0]); xa[it][1] = bf16x8_to_f16x8(xa[it][1]); }
    }
    // ---- sum(x) per (row, slab) on the matrix unit while the weights are in flight ---------------
    f4 xs[kSpw];
#pragma unroll
    for (int it = 0; it < kSpw; ++it) {
      xs[it] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        xs[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][jj]), ones, xs[it], 0, 0, 0);
    }
    // ---- integer dot per slab, then acc += scale * (dot - 1024 * sum(x)) + bias * sum(x) -------------
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      f4 c[kSpw];
#pragma unroll
      for (int it = 0; it < kSpw; ++it) {
        c[it] = (f4){0.f, 0.f, 0.f, 0.f};
        c[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][0]),
                                                       bytes_to_f16_plus_1024(wreg[t][it].x, wreg[t][it].y), c[it], 0, 0, 0);
        c[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa[it][1]),
                                                       bytes_to_f16_plus_1024(wreg[t][it].z, wreg[t][it].w), c[it], 0, 0, 0);
      }
#pragma unroll
      for (int it = 0; it < kSpw; ++it) {
        const uint32_t sw = it < 2 ? sv[t].x : sv[t].y, bw = it < 2 ? bv[t].x : bv[t].y;
        const float sc = __half2float(__ushort_as_half((unsigned short)((it & 1) ? sw >> 16 : sw & 0xFFFFu)));
        const float bi = __half2float(__ushort_as_half((unsigned short)((it & 1) ? bw >> 16 : bw & 0xFFFFu)));
#pragma unroll
        for (int i = 0; i < 4; ++i) F[t][i] += sc * (c[it][i] - 1024.0f * xs[it][i]) + bi * xs[it][i];
      }
    }
  }

  // ---- reduce over the 8 k-parts, write out: accumulator lane (n, g) holds rows 4g..4g+3 of column n ----
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wave * TILES + t) * 16 + g * 4 + i) * 16 + n] = F[t][i];
  __syncthreads();
  if (tid < 256) {
    const uint32_t m = tid >> 4, nn = tid & 15;
    if (m < rows) {
      float v[TILES];
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) acc += red[((w * TILES + t) * 16 + m) * 16 + nn];
        v[t] = acc;
      }
      float r = v[0];
      if (TILES == 2) r = v[0] / (1.0f + __expf(-v[0])) * v[1];  // silu(gate) * up
      const uint64_t o = (uint64_t)(row0 + m) * p.ld_out + tile_row + nn;
      if (p.out_f32) static_cast<float*>(p.out)[o] = r;
      else static_cast<__half*>(p.out)[o] = __float2half(r);
    }
  }
}

}  // namespace

bool qmv_q8_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  return (group_size == 64 || group_size == 128) && N > 0 && K > 0 && N % 16 == 0 && K % (64 * kSpw) == 0;
}

int32_t launch_qmv_q8(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream, int32_t x_bf16) {
  if (!qmv_q8_supported(N, K, group_size))
    return fail(RMLX_INVALID_SHAPE, "qmv_q8: N %% 16 and K %% 256 required (N=%u K=%u)", N, K);
  if (M == 0) return RMLX_OK;
  Q8Params p{};
  p.w = w; p.s = s; p.b = b; p.x = x; p.out = out; p.K = K; p.ld_out = N; p.M = M;
  // (the group size is a template parameter: as a run-time flag inside the pass loop it cost the 64-wide kernel
  // 13 % on decode-sized expert batches)
  const dim3 grid(N / 16, (M + 15) / 16);
  if (x_bf16) {
    if (group_size == 128) hipLaunchKernelGGL((qmv_q8_kernel<false, 1, true, true>), grid, dim3(kThreads), 0, stream, p);
    else hipLaunchKernelGGL((qmv_q8_kernel<false, 1, false, true>), grid, dim3(kThreads), 0, stream, p);
  } else if (group_size == 128) hipLaunchKernelGGL((qmv_q8_kernel<false, 1, true>), grid, dim3(kThreads), 0, stream, p);
  else hipLaunchKernelGGL((qmv_q8_kernel<false, 1, false>), grid, dim3(kThreads), 0, stream, p);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

// Chunk-table launch (expert projections): a.N weight rows per expert, chunks of at most 16 rows.
int32_t launch_qmv_q8_tab(const QmvArgs& a, hipStream_t stream) {
  if (!qmv_q8_supported(a.N, a.K, a.group_size == 0 ? 64 : a.group_size))
    return fail(RMLX_INVALID_SHAPE, "qmv_q8: N %% 16, K %% 256 and group size 64 or 128 required (N=%u K=%u)", a.N, a.K);
  if (a.chunk_tab == nullptr || a.max_chunks == 0) return a.chunk_tab == nullptr ? fail(RMLX_RUNTIME_ERROR, "qmv_q8: no chunk table") : RMLX_OK;
  if (a.max_chunks > 65535) return fail(RMLX_INVALID_SHAPE, "qmv_q8: too many row chunks (%u)", a.max_chunks);
  Q8Params p{};
  p.w = a.w0; p.s = a.s0; p.b = a.b0;
  p.w1 = a.dual ? a.w1 : a.w0; p.s1 = a.dual ? a.s1 : a.s0; p.b1 = a.dual ? a.b1 : a.b0;
  p.x = a.x; p.out = a.out; p.K = a.K; p.ld_out = a.ld_out; p.M = 0; p.out_f32 = a.out_f32;
  p.row_map = a.row_map; p.chunk_tab = a.chunk_tab; p.n_chunks = a.n_chunks_dev;
  p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  const dim3 grid(a.N / 16, a.max_chunks);
  const bool gs128 = a.group_size == 128;
  if (a.dual && gs128) hipLaunchKernelGGL((qmv_q8_kernel<true, 2, true>), grid, dim3(kThreads), 0, stream, p);
  else if (a.dual) hipLaunchKernelGGL((qmv_q8_kernel<true, 2, false>), grid, dim3(kThreads), 0, stream, p);
  else if (gs128) hipLaunchKernelGGL((qmv_q8_kernel<true, 1, true>), grid, dim3(kThreads), 0, stream, p);
  else hipLaunchKernelGGL((qmv_q8_kernel<true, 1, false>), grid, dim3(kThreads), 0, stream, p);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
