// Single-row GEMV for 2-bit weights on gfx950 (decode: one activation row per pass over the weights).
//
// Replaces the 2-bit case of the reference's affine_qmv (crates/rmlx-core/src/ops/quantized.rs:211-290), the only
// kernel of the reference that takes 2-bit weights; 16 values per u32 word, value i at bits 2 * (i % 16).
//
// Same organisation as the 4- / 8-bit single-row kernel (qmv_m1.hip): a wave owns one weight row over the whole K, a
// wave-wide 16-byte load covers 1 KB of that row (4096 values: a chunk), the workgroup stages the activation row once
// into LDS in the order the unpacking produces, dot products run on v_dot2_f32_f16, one wave-wide sum at the end.
//   * Fields become f16 without conversion instructions: the four 2-bit fields of a byte sit in mantissa bits 0-1,
//     2-3, 4-5, 6-7 of a half, and or-ing the exponent of 1024 / 256 / 64 / 16 makes the half 1024 + q, 256 + q,
//     64 + q, 16 + q exactly.  One mask-or per pair of values ((w & 0x00030003) | 0x64006400 = (1024 + q0, 1024 + q8),
//     ...), the upper byte of each half after one shift by 8.  The offsets are removed with sum(off * x) per lane.
//   * A word therefore pairs value f with value 8 + f (lower bytes) and 4 + f with 12 + f (upper bytes): the
//     activation image holds the matching pairs, built while staging from the two 8-value units of a word, which sit
//     in neighbouring threads.
//   * A lane's 64 values are one group (group size 64), half of one (128) or two (32): scale and bias are applied per
//     half lane, so all three group sizes run the same code.
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kChunkK = 4096;   // values of one wave-wide 16-byte load
constexpr uint32_t kMaxK = 28672;

struct Q2Params {
  const uint32_t* w; const __half* s; const __half* b;
  const __half* x;
  __half* out;
  uint32_t N, K, M;
  // a weight matrix per output row m (null: one matrix): expert gather_idx[m] of stacked weights (strides in u32 words /
  // halves; an index outside [0, n_experts) writes zeros), multiplied with activation row m / x_div
  const uint32_t* gather_idx;
  uint64_t estride_w, estride_s;
  uint32_t n_experts, x_div;
};

__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // lane ^ 1
  v = dpp_add<0x4E>(v);   // lane ^ 2
  v = dpp_add<0x141>(v);  // the other quad of each 8
  v = dpp_add<0x140>(v);  // the other 8 of each 16
  v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
}

// LDS per activation row: image [chunk][word j][byte half h][lane] of 16-byte pair blocks, then sums
// [chunk][lane][half lane] = (sum(off * x), sum(x)) of the half lane's 32 values
__host__ __device__ inline size_t q2_lds_bytes(uint32_t K) {
  const size_t chunks = (K + kChunkK - 1) / kChunkK;
  return chunks * (kChunkK * 2 + 64 * 2 * sizeof(float2));
}

// GATHER: a weight matrix per output row and workgroups that walk several row blocks (see Q2Params and below)
template <int GS, bool GATHER>
__global__ __launch_bounds__(kThreads) void qmv_q2_kernel(Q2Params p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const uint32_t K = p.K, KH = (K + kChunkK - 1) / kChunkK, G = K / GS, nunits = K / 8;
  const uint32_t row_u4 = K / 64;  // 16-byte pieces of a weight row
  u4* const img = reinterpret_cast<u4*>(lds);
  float2* const cs = reinterpret_cast<float2*>(lds + (size_t)KH * kChunkK * 2);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t m = blockIdx.y;
  // Row blocks (kWaves weight rows) of this workgroup: blockIdx.x, blockIdx.x + gridDim.x, ... -- one per workgroup in the
  // plain launch; a gather over many rows sizes the grid to what the chip keeps resident, so the activations are staged
  // once per workgroup and the next block's weights are in flight while the current block is multiplied.
  const uint32_t nblk = p.N / kWaves;
  const uint32_t my_blocks = !GATHER ? 1u : (blockIdx.x < nblk ? (nblk - 1 - blockIdx.x) / gridDim.x + 1 : 0u);
  auto block_row = [&](uint32_t i) { return (blockIdx.x + i * gridDim.x) * kWaves + wave; };
  uint64_t e_w = 0, e_s = 0;
  bool zeros = false;
  uint32_t xrow = m;
  if constexpr (GATHER) {
    const uint32_t e = p.gather_idx[m];
    zeros = e >= p.n_experts;
    e_w = zeros ? 0 : e * p.estride_w;
    e_s = zeros ? 0 : e * p.estride_s;
    xrow = m / p.x_div;
  }

  // ---- 1. loads, the activations first (the memory counter retires in order), then the row's first two chunks --------
  const u4* xg = reinterpret_cast<const u4*>(p.x + (uint64_t)xrow * K);
  u4 xv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t u = tid + i * kThreads;
    xv[i] = (u4){0u, 0u, 0u, 0u};
    if (u < nunits) xv[i] = xg[u];
  }
  struct Chunk { u4 w; uint32_t s[2], b[2]; };
  // the chunks of all blocks of the workgroup form one sequence (block 0: chunks 0 .. KH - 1, block 1: ...), loaded two
  // ahead of their use
  const uint32_t n_items = my_blocks * KH;
  uint32_t ld_item = 0;
  auto load_chunk = [&](Chunk& t) {
    const uint32_t row = block_row(ld_item / KH), c = ld_item % KH;
    ++ld_item;
    const u4* wrow = reinterpret_cast<const u4*>(p.w + e_w + (uint64_t)row * (K / 16));
    const unsigned short* srow = reinterpret_cast<const unsigned short*>(p.s + e_s) + (uint64_t)row * G;
    const unsigned short* brow = reinterpret_cast<const unsigned short*>(p.b + e_s) + (uint64_t)row * G;
    uint32_t wi = c * 64 + lane;
    wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K meet zeros in the image
#pragma unroll
    for (int hl = 0; hl < 2; ++hl) {
      uint32_t gi = (c * kChunkK + lane * 64 + hl * 32) / GS;
      gi = gi < G ? gi : G - 1;
      t.s[hl] = srow[gi];
      t.b[hl] = brow[gi];
    }
    t.w = __builtin_nontemporal_load(wrow + wi);
  };
  Chunk ca, cb;
  if (n_items > 0) load_chunk(ca);
  if (n_items > 1) load_chunk(cb);

  // ---- 2. stage x: unit u = 8 consecutive k = (chunk, lane, word j, byte half h); the two units of a word sit in
  //         neighbouring threads and exchange their values to build the pair blocks ------------------------------------
  auto stage_unit = [&](uint32_t u, const u4& own) {
    const u4 other = (u4){dpp_mov<0xB1>(own.x), dpp_mov<0xB1>(own.y), dpp_mov<0xB1>(own.z), dpp_mov<0xB1>(own.w)};
    if (u >= KH * 512) return;
    const uint32_t c = u / 512, rem = u % 512, l = rem / 8, q = rem % 8, j = q >> 1, h = q & 1;
    const u4 A = h ? other : own, B = h ? own : other;  // the word's values 0-7 and 8-15
    const uint32_t a_lo = h ? A.z : A.x, a_hi = h ? A.w : A.y, b_lo = h ? B.z : B.x, b_hi = h ? B.w : B.y;
    u4 P;  // pairs (value 4h + f, value 8 + 4h + f), f = 0..3
    P.x = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u);
    P.y = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
    P.z = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u);
    P.w = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
    img[((c * 4 + j) * 2 + h) * 64 + l] = P;
    const h8 hv = __builtin_bit_cast(h8, own);
    float xs = 0.f, xo = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = (float)hv[e];
      xs += v;
      xo += (e % 4 == 0 ? 1024.0f : (e % 4 == 1 ? 256.0f : (e % 4 == 2 ? 64.0f : 16.0f))) * v;
    }
    // the four units of a half lane sit in one quad of threads
    xs = dpp_add<0xB1>(xs); xo = dpp_add<0xB1>(xo);
    xs = dpp_add<0x4E>(xs); xo = dpp_add<0x4E>(xo);
    if ((q & 3) == 0) cs[(c * 64 + l) * 2 + (q >> 2)] = make_float2(xo, xs);
  };
#pragma unroll
  for (int i = 0; i < 4; ++i) stage_unit(tid + i * kThreads, xv[i]);
  for (uint32_t u = tid + 4 * kThreads; u < KH * 512; u += kThreads) {  // K > 16384
    u4 v = (u4){0u, 0u, 0u, 0u};
    if (u < nunits) v = xg[u];
    stage_unit(u, v);
  }
  __syncthreads();

  // ---- 3. chunk by chunk ---------------------------------------------------------------------------------------
  uint32_t mk[4] = {0x00030003u, 0x000C000Cu, 0x00300030u, 0x00C000C0u};
  uint32_t mg[4] = {0x64006400u, 0x5C005C00u, 0x54005400u, 0x4C004C00u};
  float racc = 0.f;
  uint32_t pr_item = 0;
  auto dot_chunk = [&](const Chunk& t) {
    const uint32_t c = pr_item % KH;
    if (c == 0) racc = 0.f;
    const uint32_t wd[4] = {t.w.x, t.w.y, t.w.z, t.w.w};
    const float2 k0 = cs[(c * 64 + lane) * 2], k1 = cs[(c * 64 + lane) * 2 + 1];
    float acc[2] = {0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u4 P0 = img[((c * 4 + j) * 2 + 0) * 64 + lane], P1 = img[((c * 4 + j) * 2 + 1) * 64 + lane];
      const uint32_t p0[4] = {P0.x, P0.y, P0.z, P0.w}, p1[4] = {P1.x, P1.y, P1.z, P1.w};
      const uint32_t lo = wd[j], hi = wd[j] >> 8;
      float a0 = 0.f, a1 = 0.f;
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        a0 = __builtin_amdgcn_fdot2(as_h2((lo & mk[f]) | mg[f]), as_h2(p0[f]), a0, false);
        a1 = __builtin_amdgcn_fdot2(as_h2((hi & mk[f]) | mg[f]), as_h2(p1[f]), a1, false);
      }
      acc[j >> 1] += a0 + a1;
    }
#pragma unroll
    for (int hl = 0; hl < 2; ++hl) {
      const float sc = __half2float(__ushort_as_half((unsigned short)t.s[hl]));
      const float bi = __half2float(__ushort_as_half((unsigned short)t.b[hl]));
      const float2 k = hl ? k1 : k0;
      racc += sc * (acc[hl] - k.x) + bi * k.y;
    }
    if (c == KH - 1) {  // the block's row is complete
      const float total = wave_sum(racc);
      if (lane == 0) p.out[(uint64_t)m * p.N + block_row(pr_item / KH)] = __float2half(zeros ? 0.f : total);
    }
    ++pr_item;
  };
  for (uint32_t i = 0; i < n_items; i += 2) {
    dot_chunk(ca);
    if (i + 2 < n_items) load_chunk(ca);
    if (i + 1 < n_items) {
      dot_chunk(cb);
      if (i + 3 < n_items) load_chunk(cb);
    }
  }
}

}  // namespace

bool qmv_q2_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  if (group_size != 32 && group_size != 64 && group_size != 128) return false;
  // a lane's 16 bytes of a row must be whole (64 values) and the image must fit the default dynamic LDS limit
  return N > 0 && K > 0 && N % kWaves == 0 && K % 64 == 0 && K % group_size == 0 && K <= kMaxK && q2_lds_bytes(K) <= 65536;
}

int32_t launch_qmv_q2(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream) {
  if (!qmv_q2_supported(N, K, group_size))
    return fail(RMLX_INVALID_SHAPE, "qmv_q2: unsupported shape N=%u K=%u group_size=%u", N, K, group_size);
  if (M == 0) return RMLX_OK;
  if (M > 65535) return fail(RMLX_INVALID_SHAPE, "qmv_q2: at most 65535 rows per launch (M=%u)", M);
  Q2Params p{w, s, b, x, out, N, K, M, nullptr, 0, 0, 0, 1};
  const dim3 grid(N / kWaves, M);
  const size_t lds = q2_lds_bytes(K);
  switch (group_size) {
    case 32: hipLaunchKernelGGL((qmv_q2_kernel<32, false>), grid, dim3(kThreads), lds, stream, p); break;
    case 64: hipLaunchKernelGGL((qmv_q2_kernel<64, false>), grid, dim3(kThreads), lds, stream, p); break;
    default: hipLaunchKernelGGL((qmv_q2_kernel<128, false>), grid, dim3(kThreads), lds, stream, p); break;
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

// One activation row per index through stacked 2-bit weights: output row m = activation row m / x_div of x through
// expert idx[m] (outside [0, n_experts): zeros), out [batch, N] f16; strides in u32 words / halves.
int32_t launch_qmv_q2_gather(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                             uint32_t n_experts, const __half* x, uint32_t x_div, const uint32_t* idx, uint32_t batch, __half* out,
                             uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream) {
  if (!qmv_q2_supported(N, K, group_size))
    return fail(RMLX_INVALID_SHAPE, "qmv_q2 gather: unsupported shape N=%u K=%u group_size=%u", N, K, group_size);
  if (idx == nullptr || x_div == 0) return fail(RMLX_RUNTIME_ERROR, "qmv_q2 gather: needs an expert per row");
  const size_t lds = q2_lds_bytes(K);
  for (uint32_t first = 0; first < batch; first += 65535 / x_div * x_div) {  // the row is the second grid dimension
    const uint32_t step = 65535 / x_div * x_div, rows = batch - first < step ? batch - first : step;
    Q2Params p{w, s, b, x + (uint64_t)(first / x_div) * K, out + (uint64_t)first * N, N, K, rows, idx + first, estride_w, estride_s,
               n_experts, x_div};
    // as many workgroups per row as stay resident together (four per CU by their threads), at most one per row block
    uint32_t gx = 4u * (uint32_t)ctx().num_cus / rows;
    gx = gx < 1 ? 1 : (gx > N / kWaves ? N / kWaves : gx);
    const dim3 grid(gx, rows);
    switch (group_size) {
      case 32: hipLaunchKernelGGL((qmv_q2_kernel<32, true>), grid, dim3(kThreads), lds, stream, p); break;
      case 64: hipLaunchKernelGGL((qmv_q2_kernel<64, true>), grid, dim3(kThreads), lds, stream, p); break;
      default: hipLaunchKernelGGL((qmv_q2_kernel<128, true>), grid, dim3(kThreads), lds, stream, p); break;
    }
    RMLX_HIP_CHECK(hipGetLastError());
  }
  return RMLX_OK;
}

}  // namespace rmlx
