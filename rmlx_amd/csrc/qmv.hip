// Streaming quantized GEMV family for gfx950: qmv (M <= 8 rows per pass), gather_qmm and the
// two MoE expert projections (fused gate/up + SwiGLU, down).
//
// Replaces the reference's affine_qmv_fast_f16_q4 / affine_qmv_batched_f16_q4 /
// gather_qmv_fast_f16_q4 (crates/rmlx-core/src/ops/quantized.rs:798-979, 9752-9842).
//
// Design (wave64, MFMA):
//   * One workgroup = 8 waves = one tile of 16 weight rows; the K range is split across the
//     8 waves.  Every lane issues all of its 128-bit weight loads before anything else, so a
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
//   * The per-(row, group) sums  sum(x)  and  sum(off*x)  are formed by the threads that stage x
//     (8 consecutive threads hold one group) and parked in LDS; all of the x-side work happens
//     while the weight loads are in flight.
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kChunkSlabs = 32;  // slabs of 128 k staged per pass (4096 k)
constexpr int kSpwMax = 4;       // slabs per wave per pass
constexpr int kSbStride = 65;    // dwords per row of the scale/bias image (64 groups + pad)

// Field order matters: the first 16 dwords are preloaded into SGPRs at wave launch
// (-amdgpu-kernarg-preload-count), so everything the plain qmv path needs comes first.
struct KParams {
  const uint32_t* w0;
  const __half* s0;
  const __half* b0;
  const __half* x;
  void* out;
  uint32_t K, ld_out, M, out_f32;
  const uint32_t* w1;
  const __half* s1;
  const __half* b1;
  const uint32_t* row_map;
  const uint32_t* chunk_tab;
  const uint32_t* n_chunks;
  uint64_t estride_w, estride_s;
#ifdef QMV_TRACE
  unsigned long long* trace;  // development only: per-phase shader clock of workgroup 0 / each wave
#endif
};

#ifdef QMV_TRACE
#define QMV_MARK(p, i)                                                                   \
  do {                                                                                   \
    if ((p).trace != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && (threadIdx.x & 63) == 0) \
      (p).trace[(threadIdx.x >> 6) * 16 + (i)] = __builtin_readcyclecounter();           \
  } while (0)
#else
#define QMV_MARK(p, i) do {} while (0)
#endif

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

__device__ __forceinline__ uint32_t swap16(uint32_t v) {  // value of lane ^ 16
  return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F);
}

// One pass over up to 4096 k.
// FULLP: every wave owns exactly kSpwMax slabs.  Then the k range a wave consumes (512 k) is
// exactly the range its own 64 threads stage, so the activation image and the sums are
// wave-private and the pass needs no workgroup barrier; scales and biases come straight from
// global memory (8 consecutive groups = one aligned 16-byte load per lane, scales in the lanes
// with even g, biases in the lanes with odd g, exchanged with one swizzle per word).
// !FULLP (K not a multiple of 4096): slabs are dealt to the waves evenly, everything is
// staged through LDS for the whole workgroup with barriers.
template <int MR, int TILES, bool TAB, bool FULLP>
__device__ __forceinline__ void qmv_pass(const KParams& p, char* xs, float* sums, uint32_t* sbs,
                                         const u4* const (&wrow)[TILES], f4 (&F)[TILES], uint32_t kc, int nsl,
                                         uint32_t expert, uint32_t row0, uint32_t rows, uint32_t tile_row,
                                         bool first_pass) {
  constexpr int kSlots = 4 * MR;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4, par = g >> 1;
  const uint32_t K = p.K, groups_per_row = K >> 6;
  const int spw = (nsl + kWaves - 1) / kWaves;
  const int s0 = wave * spw;
  int my = nsl - s0;
  my = my < 0 ? 0 : (my > spw ? spw : my);

  // ---- 1. issue every global load of this pass up front.  The few activation / scale loads go
  //         first: the memory counter retires in order, so they can then be consumed while the
  //         weight loads (the bulk of the traffic) are still in flight. -----------------------
  constexpr int kXU = MR;  // 16-byte activation units per thread (kChunkSlabs*16*MR / kThreads)
  static_assert(kChunkSlabs * 16 == kThreads, "one activation unit per thread and row");
  const int ngr = nsl * 2;  // quantisation groups in this pass
  u4 xv[kXU];
  {
    uint32_t srcs[kXU];
#pragma unroll
    for (int m = 0; m < kXU; ++m) {
      srcs[m] = row0 + m;
      if (TAB && p.row_map != nullptr && (uint32_t)m < rows) srcs[m] = p.row_map[row0 + m];  // wave-uniform
    }
#pragma unroll
    for (int m = 0; m < kXU; ++m) {
      xv[m] = (u4){0u, 0u, 0u, 0u};
      if ((uint32_t)m < rows && tid < nsl * 16)
        xv[m] = *reinterpret_cast<const u4*>(p.x + (uint64_t)srcs[m] * K + kc + tid * 8);
    }
  }
  u4 sbv[TILES];
  const int st = tid / 128, sr = (tid % 128) / 8, sc8 = tid % 8;  // tile, row, 8-group block
  const bool s_active = !FULLP && tid < TILES * 128 && sc8 * 8 < ngr;
  u4 sv0 = (u4){0u, 0u, 0u, 0u}, bv0 = (u4){0u, 0u, 0u, 0u};
  if (FULLP) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const uint64_t off = (TAB ? expert * p.estride_s : 0) + (uint64_t)(tile_row + n) * groups_per_row + (kc >> 6) + s0 * 2;
      const __half* sp_ = t == 0 ? p.s0 : p.s1;
      const __half* bp_ = t == 0 ? p.b0 : p.b1;
      sbv[t] = *reinterpret_cast<const u4*>(((g & 1) ? bp_ : sp_) + off);
    }
  } else if (s_active) {
    const uint64_t off = (TAB ? expert * p.estride_s : 0) + (uint64_t)(tile_row + sr) * groups_per_row + (kc >> 6) + sc8 * 8;
    sv0 = *reinterpret_cast<const u4*>((st == 0 ? p.s0 : p.s1) + off);
    bv0 = *reinterpret_cast<const u4*>((st == 0 ? p.b0 : p.b1) + off);
  }
  // every wave has queued its small loads before any wave queues the bulk loads
  if (FULLP) __builtin_amdgcn_s_barrier();
  u4 wreg[TILES][kSpwMax];
#pragma unroll
  for (int it = 0; it < kSpwMax; ++it) {
    if (FULLP || it < my) {
#pragma unroll
      for (int t = 0; t < TILES; ++t) wreg[t][it] = *(wrow[t] + (kc >> 5) + (s0 + it) * 4);
    }
  }
  QMV_MARK(p, 1);

  if (!FULLP && !first_pass) __syncthreads();  // previous pass finished reading xs / sums / sbs

  // ---- 2. activations -> LDS in operand order; per-(row, group) sums -> LDS -------------------
  if (!FULLP && s_active) {
    uint32_t* dst = sbs + (st * 16 + sr) * kSbStride + sc8 * 8;
    const uint32_t sw[4] = {sv0.x, sv0.y, sv0.z, sv0.w}, bw[4] = {bv0.x, bv0.y, bv0.z, bv0.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      dst[2 * q] = (sw[q] & 0xFFFFu) | (bw[q] << 16);
      dst[2 * q + 1] = (sw[q] >> 16) | (bw[q] & 0xFFFF0000u);
    }
  }
  {
    const int c = tid, slab = c >> 4, gg = (c >> 2) & 3, j = c & 3;
#pragma unroll
    for (int m = 0; m < kXU; ++m) {
      if (c < nsl * 16)
        *reinterpret_cast<u4*>(xs + ((slab * 4 + j) * kSlots + gg * MR + m) * 16) = permute_x8(xv[m]);
      // this thread's 8 activations: plain sum and sum weighted by the unpack offsets
      // (even k -> 1024, odd k -> 64); 8 consecutive threads make up one group of 64
      const h8 hv = __builtin_bit_cast(h8, xv[m]);
      float xs8 = 0.f, xo8 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        xs8 += (float)hv[e] + (float)hv[e + 1];
        xo8 += 1024.0f * (float)hv[e] + 64.0f * (float)hv[e + 1];
      }
#pragma unroll
      for (int off = 1; off < 8; off <<= 1) {
        xs8 += __shfl_xor(xs8, off, 64);
        xo8 += __shfl_xor(xo8, off, 64);
      }
      if ((c & 7) == 0) {  // sums[group][m] = (-sum(off*x), sum(x)); rows >= MR stay unused
        sums[((c >> 3) * 8 + m) * 2 + 0] = -xo8;
        sums[((c >> 3) * 8 + m) * 2 + 1] = xs8;
      }
    }
  }
  QMV_MARK(p, 2);
  if (!FULLP) __syncthreads();
  QMV_MARK(p, 3);

  // ---- 3. weights: integer dot per group via MFMA (independent slabs interleaved), then
  //         acc += scale * (dot - sum(off*x)) + bias * sum(x) in f32; one tile set at a time to
  //         keep the register footprint at two workgroups per CU ----------------------------------
  // A-operand activity: accumulator rows 0-7 take group 0 (g<2), rows 8-15 group 1 (g>=2).
  const int am = n & 7;
  const bool a_active = ((n < 8) == (g < 2)) && (am < MR);
  const int a_slot_off = (g * MR + am) * 16;
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    f4 c[kSpwMax];
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) c[it] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      h8 av[kSpwMax];
#pragma unroll
      for (int it = 0; it < kSpwMax; ++it) {
        av[it] = (h8){0, 0, 0, 0, 0, 0, 0, 0};
        if ((FULLP || it < my) && a_active)
          av[it] = *reinterpret_cast<const h8*>(xs + (((s0 + it) * 4 + j) * kSlots) * 16 + a_slot_off);
      }
#pragma unroll
      for (int it = 0; it < kSpwMax; ++it) {
        if (FULLP || it < my) {
          const uint32_t wd = j == 0 ? wreg[t][it].x : (j == 1 ? wreg[t][it].y : (j == 2 ? wreg[t][it].z : wreg[t][it].w));
          c[it] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[it], unpack_q4_word(wd), c[it], 0, 0, 0);
        }
      }
    }
    u4 sv, bv;
    if (FULLP) {
      const u4 other = (u4){swap16(sbv[t].x), swap16(sbv[t].y), swap16(sbv[t].z), swap16(sbv[t].w)};
      sv = (g & 1) ? other : sbv[t];
      bv = (g & 1) ? sbv[t] : other;
    }
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) {
      if (FULLP || it < my) {
        const float* sp = sums + (((s0 + it) * 2 + par) * 8 + (g & 1) * 4) * 2;
        const f4 c01 = *reinterpret_cast<const f4*>(sp);      // (-xoff, xsum) of accumulator rows 4g, 4g+1
        const f4 c23 = *reinterpret_cast<const f4*>(sp + 4);  // rows 4g+2, 4g+3
        uint32_t sbits, bbits;
        if (FULLP) {  // group 2*it + par of the 8 loaded ones: word `it`, half `par`
          const uint32_t swd = it == 0 ? sv.x : (it == 1 ? sv.y : (it == 2 ? sv.z : sv.w));
          const uint32_t bwd = it == 0 ? bv.x : (it == 1 ? bv.y : (it == 2 ? bv.z : bv.w));
          sbits = par ? swd >> 16 : swd & 0xFFFFu;
          bbits = par ? bwd >> 16 : bwd & 0xFFFFu;
        } else {
          const uint32_t sb = sbs[(t * 16 + n) * kSbStride + (s0 + it) * 2 + par];
          sbits = sb & 0xFFFFu;
          bbits = sb >> 16;
        }
        const float sc = __half2float(__ushort_as_half((unsigned short)sbits));
        const float bi = __half2float(__ushort_as_half((unsigned short)bbits));
        F[t][0] += sc * (c[it][0] + c01[0]) + bi * c01[1];
        F[t][1] += sc * (c[it][1] + c01[2]) + bi * c01[3];
        F[t][2] += sc * (c[it][2] + c23[0]) + bi * c23[1];
        F[t][3] += sc * (c[it][3] + c23[2]) + bi * c23[3];
      }
    }
    if (TILES > 1) __builtin_amdgcn_sched_barrier(0);  // finish one tile set before the next (registers)
  }
  QMV_MARK(p, 4);
}

// MR = activation rows staged per pass (1, 2, 4 or 8); TILES = 1, or 2 for fused gate/up.
// ALLFULL: K is a multiple of 4096, the partial-pass code is not instantiated (fewer registers:
// two workgroups fit on a CU).
template <int MR, int TILES, bool TAB, bool ALLFULL>
__global__ __launch_bounds__(kThreads) void qmv_q4_kernel(KParams p) {
  constexpr int kSlots = 4 * MR;                              // 16-byte slots per (slab, j)
  constexpr int kXsBytes = kChunkSlabs * 4 * kSlots * 16;     // activation image
  constexpr int kRedBytes = kWaves * TILES * 256 * 4;
  constexpr int kXsAlloc = kXsBytes > kRedBytes ? kXsBytes : kRedBytes;
  __shared__ __attribute__((aligned(16))) char xs[kXsAlloc];
  __shared__ uint32_t sbs[TILES * 16 * kSbStride];
  __shared__ __attribute__((aligned(16))) float sums[kChunkSlabs * 2 * 8 * 2];  // [group][row 0..7][-xoff, xsum]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 15;   // weight row within the tile / accumulator column
  const int g = lane >> 4;   // k sub-block of the slab / accumulator row group

  // ---- which rows -----------------------------------------------------------------------
  uint32_t expert = 0, row0 = blockIdx.y * 8, rows;
  bool write_zeros = false;
  if (TAB) {
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
  const uint32_t tile_row = blockIdx.x * 16;

  const u4* wrow[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
    wrow[t] = reinterpret_cast<const u4*>((t == 0 ? p.w0 : p.w1) + (TAB ? expert * p.estride_w : 0) +
                                          (uint64_t)(tile_row + n) * words_per_row) + g;

  f4 F[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
  QMV_MARK(p, 0);

  for (uint32_t kc = 0; kc < K; kc += kChunkSlabs * 128) {
    const uint32_t left = (K - kc) / 128;
    if (ALLFULL || left >= (uint32_t)kChunkSlabs)
      qmv_pass<MR, TILES, TAB, true>(p, xs, sums, sbs, wrow, F, kc, kChunkSlabs, expert, row0, rows, tile_row, kc == 0);
    else if (!ALLFULL)
      qmv_pass<MR, TILES, TAB, false>(p, xs, sums, sbs, wrow, F, kc, (int)left, expert, row0, rows, tile_row, kc == 0);
  }

  // ---- 5. reduce over waves and over the two group halves, write out ---------------------------
  QMV_MARK(p, 5);
  __syncthreads();  // everyone is done with xs
  QMV_MARK(p, 6);
  float* red = reinterpret_cast<float*>(xs);
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wave * TILES + t) * 16 + g * 4 + i) * 16 + n] = F[t][i];
  __syncthreads();
  QMV_MARK(p, 7);
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
  QMV_MARK(p, 8);
}

template <int MR, int TILES>
void launch_t(const KParams& p, bool tab, dim3 grid, hipStream_t s) {
  const bool allfull = p.K % (kChunkSlabs * 128) == 0;
  if (tab) {
    if (allfull) hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, true, true>), grid, dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, true, false>), grid, dim3(kThreads), 0, s, p);
  } else {
    if (allfull) hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, false, true>), grid, dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, false, false>), grid, dim3(kThreads), 0, s, p);
  }
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

#ifdef QMV_TRACE
unsigned long long* g_qmv_trace = nullptr;
#endif

bool qmv_q4_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  return group_size == 64 && N % 16 == 0 && K % 512 == 0 && N > 0 && K > 0;
}

int32_t launch_qmv_q4(const QmvArgs& a, hipStream_t s) {
  if (!qmv_q4_supported(a.N, a.K, 64)) return fail(RMLX_INVALID_SHAPE, "qmv_q4: N %% 16 and K %% 512 required (N=%u K=%u)", a.N, a.K);
  KParams p{};
  p.w0 = a.w0; p.s0 = a.s0; p.b0 = a.b0;
  p.w1 = a.dual ? a.w1 : a.w0; p.s1 = a.dual ? a.s1 : a.s0; p.b1 = a.dual ? a.b1 : a.b0;
  p.x = a.x; p.row_map = a.row_map; p.chunk_tab = a.chunk_tab; p.n_chunks = a.n_chunks_dev;
  p.out = a.out; p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  p.K = a.K; p.ld_out = a.ld_out; p.M = a.M; p.out_f32 = a.out_f32;
#ifdef QMV_TRACE
  p.trace = g_qmv_trace;
#endif
  const bool tab = a.chunk_tab != nullptr;
  uint32_t chunks = tab ? a.max_chunks : (a.M + 7) / 8;
  if (chunks == 0) return RMLX_OK;
  dim3 grid(a.N / 16, chunks);
  int mr = a.mr;
  if (mr == 0) mr = tab ? 8 : (a.M >= 5 ? 8 : (a.M >= 3 ? 4 : (a.M == 2 ? 2 : 1)));
  if (a.dual) {
    switch (mr) {
      case 1: launch_t<1, 2>(p, tab, grid, s); break;
      case 2: launch_t<2, 2>(p, tab, grid, s); break;
      case 4: launch_t<4, 2>(p, tab, grid, s); break;
      default: launch_t<8, 2>(p, tab, grid, s); break;
    }
  } else {
    switch (mr) {
      case 1: launch_t<1, 1>(p, tab, grid, s); break;
      case 2: launch_t<2, 1>(p, tab, grid, s); break;
      case 4: launch_t<4, 1>(p, tab, grid, s); break;
      default: launch_t<8, 1>(p, tab, grid, s); break;
    }
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
