// Streaming quantized GEMV family for gfx950: qmv (M <= 8 rows per pass), gather_qmm and the
// two MoE expert projections (fused gate/up + SwiGLU, down).
//
// Replaces the reference's affine_qmv_fast_f16_q4 / affine_qmv_batched_f16_q4 /
// gather_qmv_fast_f16_q4 (crates/rmlx-core/src/ops/quantized.rs:798-979, 9752-9842).
//
// Design (wave64, MFMA):
//   * One workgroup = 4 waves = one tile of 16 weight rows; the K range is split across the
//     4 waves.  Every lane issues all of its 128-bit weight loads before anything else, so a
//     whole [16 x 4096] tile (32 KB) is in flight per workgroup.
//   * A "slab" is 16 rows x 128 k.  Lane (n = lane%16, g = lane/16) loads the 16 bytes holding
//     k in [32g, 32g+32) of row n; its four u32 words feed four v_mfma_f32_16x16x32_f16
//     (word j -> k = 32g + 8j + 0..7), weights as the B operand so that the accumulator lane
//     keeps column n.
//   * Nibbles are turned into f16 with mask-or only: (w & 0x000F000F) | 0x64006400 is the pair
//     (1024+q0, 1024+q4), (w & 0x00F000F0) | 0x54005400 is (64+q1, 64+q5).  The constant
//     offsets are removed exactly by starting the accumulator at -sum(off_k * x_k); the k order
//     inside a word (0,4,1,5,2,6,3,7) is matched by permuting x when it is staged into LDS.
//   * The two quantisation groups of a slab (group size 64) must be scaled separately.  With at
//     most 8 activation rows, accumulator rows 0-7 receive x restricted to the first group and
//     rows 8-15 the same x restricted to the second group (the other half of the A operand is
//     zero), so one accumulator tile yields both per-group integer dot products.  Each is then
//     folded into the f32 result with  acc += scale * dot + bias * xsum.
//   * The per-(row, group) sums  sum(x)  and  sum(off*x)  come from the same MFMA with a
//     constant B operand, computed while the weight loads are in flight.
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kChunkSlabs = 32;  // slabs of 128 k staged per pass (4096 k)
constexpr int kSpwMax = 8;       // slabs per wave per pass
constexpr int kSbStride = 65;    // dwords per row of the scale/bias image (64 groups + pad)

struct KParams {
  const uint32_t* w[2];
  const __half* s[2];
  const __half* b[2];
  const __half* x;
  const uint32_t* row_map;
  const uint32_t* chunk_tab;
  const uint32_t* n_chunks;
  void* out;
  uint64_t estride_w, estride_s;
  uint32_t K, row_div, ld_out, M, out_f32;
};

__device__ __forceinline__ h8 unpack_q4_word(uint32_t w) {
  uint32_t t = w >> 8;
  u4 p;
  p.x = (w & 0x000F000Fu) | 0x64006400u;  // k+0, k+4   (+1024)
  p.y = (w & 0x00F000F0u) | 0x54005400u;  // k+1, k+5   (+64)
  p.z = (t & 0x000F000Fu) | 0x64006400u;  // k+2, k+6   (+1024)
  p.w = (t & 0x00F000F0u) | 0x54005400u;  // k+3, k+7   (+64)
  return __builtin_bit_cast(h8, p);
}

// x halves (k0..k7) -> slot order (0,4,1,5,2,6,3,7), matching unpack_q4_word.
__device__ __forceinline__ u4 permute_x8(u4 d) {
  u4 o;
  o.x = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);
  return o;
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + __expf(-v)); }

// MR = activation rows staged per pass (1, 2, 4 or 8); TILES = 1, or 2 for fused gate/up.
template <int MR, int TILES>
__global__ __launch_bounds__(kThreads) void qmv_q4_kernel(KParams p) {
  constexpr int kSlots = 4 * MR;                              // 16-byte slots per (slab, j)
  constexpr int kXsBytes = kChunkSlabs * 4 * kSlots * 16;     // activation image
  constexpr int kRedBytes = kWaves * TILES * 256 * 4;
  constexpr int kXsAlloc = kXsBytes > kRedBytes ? kXsBytes : kRedBytes;
  __shared__ __attribute__((aligned(16))) char xs[kXsAlloc];
  __shared__ uint32_t sbs[TILES * 16 * kSbStride];
  __shared__ __attribute__((aligned(16))) float corr[kWaves * kSpwMax * 4 * 4 * 2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 15;   // weight row within the tile / accumulator column
  const int g = lane >> 4;   // k sub-block of the slab / accumulator row group
  const int par = g >> 1;    // which of the slab's two quantisation groups this lane scales

  // ---- which rows -----------------------------------------------------------------------
  uint32_t expert = 0, row0 = blockIdx.y * 8, rows;
  bool write_zeros = false;
  if (p.chunk_tab != nullptr) {
    if (p.n_chunks != nullptr && blockIdx.y >= *p.n_chunks) return;
    expert = p.chunk_tab[3 * blockIdx.y + 0];
    row0 = p.chunk_tab[3 * blockIdx.y + 1];
    rows = p.chunk_tab[3 * blockIdx.y + 2];
    write_zeros = (rows >> 31) != 0;
    rows &= 0x7FFFFFFFu;
  } else {
    rows = p.M - row0 < 8u ? p.M - row0 : 8u;
  }
  if (rows > (uint32_t)MR) rows = MR;  // host guarantees rows <= MR

  const uint32_t K = p.K;
  const uint32_t words_per_row = K >> 3;
  const uint32_t groups_per_row = K >> 6;
  const uint32_t tile_row = blockIdx.x * 16;

  const u4* wrow[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
    wrow[t] = reinterpret_cast<const u4*>(p.w[t] + expert * p.estride_w +
                                          (uint64_t)(tile_row + n) * words_per_row) + g;

  // A-operand activity: accumulator rows 0-7 take group 0 (g<2), rows 8-15 group 1 (g>=2).
  const int mslot = n;
  const int am = mslot & 7;
  const bool a_active = ((mslot < 8) == (g < 2)) && (am < MR);
  const int a_slot_off = (g * MR + am) * 16;

  // constant B operand for the x-side sums: column 0 = offsets, column 1 = ones
  h8 bconst;
  {
    const _Float16 o0 = (_Float16)1024.0f, o1 = (_Float16)64.0f, one = (_Float16)1.0f, z = (_Float16)0.0f;
    h8 offs = {o0, o0, o1, o1, o0, o0, o1, o1};
    h8 ones = {one, one, one, one, one, one, one, one};
    h8 zero = {z, z, z, z, z, z, z, z};
    bconst = n == 0 ? offs : (n == 1 ? ones : zero);
  }

  f4 F[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};

  for (uint32_t kc = 0; kc < K; kc += kChunkSlabs * 128) {
    const int nsl = (K - kc) / 128 < (uint32_t)kChunkSlabs ? (int)((K - kc) / 128) : kChunkSlabs;
    const int spw = (nsl + kWaves - 1) / kWaves;
    const int s0 = wave * spw;
    int my = nsl - s0;
    my = my < 0 ? 0 : (my > spw ? spw : my);

    // ---- 1. all weight loads of this pass, before anything else ----------------------------
    u4 wreg[TILES][kSpwMax];
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) {
      if (it < my) {
#pragma unroll
        for (int t = 0; t < TILES; ++t)
          wreg[t][it] = __builtin_nontemporal_load(wrow[t] + (kc >> 5) + (s0 + it) * 4);
      }
    }

    if (kc != 0) __syncthreads();  // previous pass finished reading xs / sbs

    // ---- 2. stage scales+biases (as half2 pairs) and the permuted activations ---------------
    {
      const int ngr = nsl * 2;  // groups in this pass
      for (int u = tid; u < TILES * 16 * 8; u += kThreads) {
        const int t = u / 128, r = (u % 128) / 8, c8 = u % 8;  // 8 groups per 16 B
        if (c8 * 8 < ngr) {
          const uint64_t off = expert * p.estride_s + (uint64_t)(tile_row + r) * groups_per_row + (kc >> 6) + c8 * 8;
          const u4 sv = *reinterpret_cast<const u4*>(p.s[t] + off);
          const u4 bv = *reinterpret_cast<const u4*>(p.b[t] + off);
          uint32_t* dst = sbs + (t * 16 + r) * kSbStride + c8 * 8;
          const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            dst[2 * q] = (sw[q] & 0xFFFFu) | (bw[q] << 16);
            dst[2 * q + 1] = (sw[q] >> 16) | (bw[q] & 0xFFFF0000u);
          }
        }
      }
      const int units = nsl * 16 * MR;  // 16-byte units (8 halves) of this pass
      for (int u = tid; u < units; u += kThreads) {
        const int m = u % MR, c = u / MR;
        u4 v = (u4){0u, 0u, 0u, 0u};
        if ((uint32_t)m < rows) {
          uint32_t src = row0 + m;
          if (p.row_map != nullptr) src = p.row_map[src] / p.row_div;
          v = *reinterpret_cast<const u4*>(p.x + (uint64_t)src * K + kc + c * 8);
        }
        const int slab = c >> 4, gg = (c >> 2) & 3, j = c & 3;
        *reinterpret_cast<u4*>(xs + ((slab * 4 + j) * kSlots + gg * MR + m) * 16) = permute_x8(v);
      }
    }
    __syncthreads();

    // ---- 3. x-side sums per (row, group) of this wave's slabs (wave-private LDS) -----------
    float* mycorr = corr + wave * (kSpwMax * 32);
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) {
      if (it < my) {
        f4 c2 = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h8 av = {0, 0, 0, 0, 0, 0, 0, 0};
          if (a_active) av = *reinterpret_cast<const h8*>(xs + (((s0 + it) * 4 + j) * kSlots) * 16 + a_slot_off);
          c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bconst, c2, 0, 0, 0);
        }
        if (n < 2) {
          const float sgn = n == 0 ? -1.0f : 1.0f;  // store -sum(off*x) and +sum(x)
#pragma unroll
          for (int i = 0; i < 4; ++i) mycorr[it * 32 + g * 8 + i * 2 + n] = sgn * c2[i];
        }
      }
    }

    // ---- 4. main loop: integer dot per group via MFMA, then scale/bias in f32 ---------------
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) {
      if (it < my) {
        const f4 c01 = *reinterpret_cast<const f4*>(mycorr + it * 32 + g * 8);      // (-xoff0,xsum0,-xoff1,xsum1)
        const f4 c23 = *reinterpret_cast<const f4*>(mycorr + it * 32 + g * 8 + 4);  // rows 2,3
        h8 av[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          av[j] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
          if (a_active) av[j] = *reinterpret_cast<const h8*>(xs + (((s0 + it) * 4 + j) * kSlots) * 16 + a_slot_off);
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          f4 c = (f4){c01[0], c01[2], c23[0], c23[2]};
          const u4 wv = wreg[t][it];
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[0], unpack_q4_word(wv.x), c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[1], unpack_q4_word(wv.y), c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[2], unpack_q4_word(wv.z), c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[3], unpack_q4_word(wv.w), c, 0, 0, 0);
          const uint32_t sb = sbs[(t * 16 + n) * kSbStride + (s0 + it) * 2 + par];
          const float sc = __half2float(__ushort_as_half((unsigned short)(sb & 0xFFFFu)));
          const float bi = __half2float(__ushort_as_half((unsigned short)(sb >> 16)));
          F[t][0] += sc * c[0] + bi * c01[1];
          F[t][1] += sc * c[1] + bi * c01[3];
          F[t][2] += sc * c[2] + bi * c23[1];
          F[t][3] += sc * c[3] + bi * c23[3];
        }
      }
    }
  }

  // ---- 5. reduce over waves and over the two group halves, write out ---------------------------
  __syncthreads();  // everyone is done with xs
  float* red = reinterpret_cast<float*>(xs);
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wave * TILES + t) * 16 + g * 4 + i) * 16 + n] = F[t][i];
  __syncthreads();
  if (tid < 128) {
    const int m = tid >> 4, nn = tid & 15;
    if ((uint32_t)m < rows) {
      float v[TILES];
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
          acc += red[((w * TILES + t) * 16 + m) * 16 + nn] + red[((w * TILES + t) * 16 + m + 8) * 16 + nn];
        v[t] = acc;
      }
      float r = v[0];
      if (TILES == 2) r = silu_f(v[0]) * v[TILES - 1];
      if (write_zeros) r = 0.f;
      const uint64_t o = (uint64_t)(row0 + m) * p.ld_out + tile_row + nn;
      if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = r;
      else reinterpret_cast<__half*>(p.out)[o] = __float2half(r);
    }
  }
}

template <int MR, int TILES>
void launch_t(const KParams& p, dim3 grid, hipStream_t s) {
  hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES>), grid, dim3(kThreads), 0, s, p);
}

__global__ void build_gather_chunks_kernel(const uint32_t* indices, uint32_t batch, uint32_t mpb,
                                           uint32_t n_experts, uint32_t* chunk_tab) {
  const uint32_t per = (mpb + 7) / 8;
  const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= batch * per) return;
  const uint32_t b = c / per, r = (c % per) * 8;
  uint32_t e = indices[b], rows = mpb - r < 8u ? mpb - r : 8u;
  if (e >= n_experts) { e = 0; rows |= 0x80000000u; }
  chunk_tab[3 * c + 0] = e;
  chunk_tab[3 * c + 1] = b * mpb + r;
  chunk_tab[3 * c + 2] = rows;
}

}  // namespace

int32_t launch_build_gather_chunks(const uint32_t* indices, uint32_t batch, uint32_t mpb, uint32_t n_experts,
                                   uint32_t* chunk_tab, hipStream_t s) {
  const uint32_t n = batch * ((mpb + 7) / 8);
  if (n == 0) return RMLX_OK;
  hipLaunchKernelGGL(build_gather_chunks_kernel, dim3((n + 255) / 256), dim3(256), 0, s, indices, batch, mpb,
                     n_experts, chunk_tab);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

bool qmv_q4_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  return group_size == 64 && N % 16 == 0 && K % 512 == 0 && N > 0 && K > 0;
}

int32_t launch_qmv_q4(const QmvArgs& a, hipStream_t s) {
  if (!qmv_q4_supported(a.N, a.K, 64)) return fail(RMLX_INVALID_SHAPE, "qmv_q4: N %% 16 and K %% 512 required (N=%u K=%u)", a.N, a.K);
  KParams p;
  p.w[0] = a.w0; p.s[0] = a.s0; p.b[0] = a.b0;
  p.w[1] = a.dual ? a.w1 : a.w0; p.s[1] = a.dual ? a.s1 : a.s0; p.b[1] = a.dual ? a.b1 : a.b0;
  p.x = a.x; p.row_map = a.row_map; p.chunk_tab = a.chunk_tab; p.n_chunks = a.n_chunks_dev;
  p.out = a.out; p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  p.K = a.K; p.row_div = a.row_div ? a.row_div : 1; p.ld_out = a.ld_out; p.M = a.M; p.out_f32 = a.out_f32;
  uint32_t chunks = a.chunk_tab ? a.max_chunks : (a.M + 7) / 8;
  if (chunks == 0) return RMLX_OK;
  dim3 grid(a.N / 16, chunks);
  int mr = a.mr;
  if (mr == 0) mr = a.chunk_tab ? 8 : (a.M >= 5 ? 8 : (a.M >= 3 ? 4 : (a.M == 2 ? 2 : 1)));
  if (a.dual) {
    switch (mr) {
      case 1: launch_t<1, 2>(p, grid, s); break;
      case 2: launch_t<2, 2>(p, grid, s); break;
      case 4: launch_t<4, 2>(p, grid, s); break;
      default: launch_t<8, 2>(p, grid, s); break;
    }
  } else {
    switch (mr) {
      case 1: launch_t<1, 1>(p, grid, s); break;
      case 2: launch_t<2, 1>(p, grid, s); break;
      case 4: launch_t<4, 1>(p, grid, s); break;
      default: launch_t<8, 1>(p, grid, s); break;
    }
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
