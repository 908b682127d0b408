// Single-row quantized GEMV for gfx950 (decode: one activation row per pass over the weights).
//
// Replaces the reference's affine_qmv_fast_q4 / affine_qmv_fast_q8 at M = 1
// (crates/rmlx-core/src/ops/quantized.rs:394-600, 620-695, dispatched from :1309-1411).
//
// With one activation row the matrix unit has nothing to share between rows, so this kernel is
// organised around the memory system instead:
//   * A wave-wide 16-byte load covers 1 KB of ONE weight row (2048 4-bit or 1024 8-bit values):
//     fully contiguous, where the MFMA operand layout of the multi-row kernel makes every lane
//     quad touch four different rows.  A wave owns one or two adjacent weight rows over the whole K, so a
//     workgroup (8 waves) streams one contiguous block, and every load of a pass is in
//     flight before the first one is consumed.  (One row per wave when K < 12288: finer-grained
//     waves overlap arrival and arithmetic better; measured.)  With a single activation row the
//     weights are loaded non-temporally: nothing reads them a second time.
//   * Lane l of a wave always works on the same k positions of a chunk, so its activations live
//     in registers for all rows: the workgroup stages x once into LDS (already permuted to the
//     order the nibble unpacking produces, together with the per-lane sums the offset removal
//     needs) and a wave reads its 16 registers per chunk from there.
//   * Dot products run on v_dot2_f32_f16 with exact magic-number int -> f16 conversion
//     ((w & 0x000F000F) | 0x64006400 = (1024 + q0, 1024 + q4), ...); per lane and row
//     acc = sum(x * (off + q)), and  scale * (acc - sum(off * x)) + bias * sum(x)  is added in f32.
//     A quantisation group is 1, 2, 4 or 8 whole lanes (group sizes 32 / 64 / 128), so no
//     cross-lane work is needed before the final wave-wide sum, and a wave writes its
//     outputs itself: no cross-wave reduction, one barrier (after staging x).
//   * K is any multiple of 32 (4-bit) or 16 (8-bit) values: the lanes of the last chunk that lie
//     past K meet zeros in the activation image.
//   * Up to four activation rows share a pass: the unpacked weight pairs are reused, each row adds
//     its own registers of x and 16 dot instructions per chunk and lane.
//   * Matrices with more row blocks than the chip keeps resident run a looping form of the kernel:
//     the grid is the resident workgroups, each stages the activations once and walks several row
//     blocks with the next block's weights in flight.  Long rows of a short matrix split K over 2 or
//     4 waves of the workgroup.
#include <vector>

#include "common.hpp"
#include "route.hpp"

namespace rmlx {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr uint32_t kMaxK = 32768;  // (the activation image and sums must also fit the default dynamic LDS limit)

struct M1Params {
  const uint32_t* w; const __half* s; const __half* b;
  const __half* x;
  __half* out;
  uint32_t N, K, M;
  int32_t epi_kind, epi_dtype;  // fused store epilogue: EPI_RESIDUAL / EPI_SWIGLU with an [M,N] f16 / f32 operand
  const void* epi;
  // fused RMSNorm prologue (null = none): x[m,k] <- (x[m,k] * half(inv_rms[m])) * norm_w[k], each product rounded to f16
  const __half* norm_w;
  const float* inv_rms;
  // GATHER kernels: activation row m (one row per pass) multiplies expert gather_idx[m] of stacked weights (strides in u32
  // words / halves); an index outside [0, n_experts) writes zeros
  const uint32_t* gather_idx;
  uint64_t estride_w, estride_s;
  uint32_t n_experts;
  // (gather_div consecutive rows share an index: row m of this launch, which starts at row gather_row0 of the call, takes
  // gather_idx[(gather_row0 + m) / gather_div]; 0 or 1 = an index per row)
  uint32_t gather_div = 1, gather_row0 = 0;
  int32_t x_bf16 = 0;  // 1: the activations are bf16 bits, 2: f32 values (kernels built with the conversion prologues only, see launch_r)
};

__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// sum over the 64 lanes, same value returned in every lane
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]: lane ^ 1
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]: lane ^ 2
  v = dpp_add<0x141>(v);  // row_half_mirror: the other quad of each 8
  v = dpp_add<0x140>(v);  // row_mirror: the other 8 of each 16
  v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
}

// sum over the 32 lanes of a half of the wave, returned in every lane of that half (the same additions as wave_sum up to its
// last one)
__device__ __forceinline__ float half_wave_sum(float v) {
  v = dpp_add<0xB1>(v);
  v = dpp_add<0x4E>(v);
  v = dpp_add<0x141>(v);
  v = dpp_add<0x140>(v);
  v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
  return v;
}

// x halves (k0..k7) -> pair order (k0,k4),(k1,k5),(k2,k6),(k3,k7) of the nibble unpacking
__device__ __forceinline__ u4 to_pair_order(u4 d) {
  u4 o;
  o.x = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);
  return o;
}

// ---- pieces shared by the two kernels below ---------------------------------------------------------------------
// Geometry of the activation image a workgroup keeps in LDS: per activation row the image [chunk][unit j][lane]
// (a unit = 8 consecutive k = 16 bytes), then the sums [chunk][lane] = (sum(off * x), sum(x)) of the lane's values.
template <int BITS, int MR>
struct XImage {
  static constexpr int kChunkK = 8192 / BITS;  // k values of one wave-wide 16-byte load: 2048 / 1024
  static constexpr int kLaneK = kChunkK / 64;  // values per lane and chunk: 32 / 16
  static constexpr int kXU = kLaneK / 8;       // 16-byte activation units per lane and chunk: 4 / 2
  char* lds;
  uint32_t K, KH, nunits, img_bytes, cs_bytes;  // KH whole chunks; image and sums bytes per activation row
  __device__ XImage(char* lds_, uint32_t K_)
      : lds(lds_), K(K_), KH((K_ + kChunkK - 1) / kChunkK), nunits(K_ / 8), img_bytes(KH * kChunkK * 2),
        cs_bytes(KH * 64 * (uint32_t)sizeof(float2)) {}
  __device__ u4* xl(int m) const { return reinterpret_cast<u4*>(lds + (size_t)m * img_bytes); }
  __device__ float2* cs(int m) const { return reinterpret_cast<float2*>(lds + (size_t)MR * img_bytes + (size_t)m * cs_bytes); }
};

// RMSNorm prologue of the reference's MMA kernel (`has_norm`, quantized.rs:3070-3095) applied to one 16-byte unit
__device__ __forceinline__ u4 normalise_unit(const __half* norm_w, const float* inv_rms, uint32_t row, uint32_t u,
                                             uint32_t nunits, u4 v) {
  const _Float16 rs = (_Float16)inv_rms[row];
  const h8 nw = __builtin_bit_cast(h8, reinterpret_cast<const u4*>(norm_w)[u < nunits ? u : nunits - 1]);
  const h8 scaled = __builtin_bit_cast(h8, v) * (h8){rs, rs, rs, rs, rs, rs, rs, rs};
  return __builtin_bit_cast(u4, scaled * nw);
}

// Prologue kinds of the activation staging (the NORM template parameter): none, the RMSNorm prologue, bf16 activations
// converted to f16 on the way (through f32, rounded to nearest even: what the separate cast kernel does).
constexpr int kPrologueNone = 0, kPrologueNorm = 1, kPrologueBf16 = 2, kPrologueF32 = 3;  // (f32: rounded to f16 on the way)

// 8 consecutive f32 activations (two 16-byte loads) -> one unit of 8 f16 values, rounded to nearest even
__device__ __forceinline__ u4 f32_unit_to_f16(u4 lo, u4 hi) {
  const float f[8] = {__uint_as_float(lo.x), __uint_as_float(lo.y), __uint_as_float(lo.z), __uint_as_float(lo.w),
                      __uint_as_float(hi.x), __uint_as_float(hi.y), __uint_as_float(hi.z), __uint_as_float(hi.w)};
  uint32_t w[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const h2 pair = {(_Float16)f[2 * e], (_Float16)f[2 * e + 1]};
    w[e] = __builtin_bit_cast(uint32_t, pair);
  }
  return (u4){w[0], w[1], w[2], w[3]};
}
// unit u of activation row `row` of x (f16 / bf16: 16 bytes; f32: 32 bytes, converted)
template <int NORM>
__device__ __forceinline__ u4 load_unit(const __half* x, uint64_t row, uint32_t K, uint32_t u) {
  if constexpr (NORM == kPrologueF32) {
    const u4* xg = reinterpret_cast<const u4*>(reinterpret_cast<const float*>(x) + row * K);
    return f32_unit_to_f16(xg[2 * u], xg[2 * u + 1]);
  } else {
    return reinterpret_cast<const u4*>(x + row * K)[u];
  }
}

__device__ __forceinline__ u4 bf16_unit_to_f16(u4 v) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
    const h2 pair = {(_Float16)lo, (_Float16)hi};
    w[e] = __builtin_bit_cast(uint32_t, pair);
  }
  return (u4){w[0], w[1], w[2], w[3]};
}

// 1. The activation loads of a workgroup (the first four rounds of 512 units; issued before the weight loads
//    because the memory counter retires in order), normalised on the way when NORM.  Rows past M repeat the last one.
template <int BITS, int MR, int NORM>
__device__ __forceinline__ void load_activations(const XImage<BITS, MR> g, const __half* x, uint32_t M, uint32_t mrow0,
                                                 const __half* norm_w, const float* inv_rms, int tid, u4 (&xv)[MR][4]) {
  const uint32_t nunits = g.nunits;
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const uint32_t rm = mrow0 + m < M ? mrow0 + m : M - 1;
    const uint32_t u0 = (uint32_t)tid < nunits ? (uint32_t)tid : nunits - 1;
    xv[m][0] = load_unit<NORM>(x, rm, g.K, u0);
#pragma unroll
    for (int i = 1; i < 4; ++i) {
      xv[m][i] = (u4){0u, 0u, 0u, 0u};
      if (nunits > (uint32_t)i * kThreads) {  // uniform; the last round may be partial (clamped, stored under a guard)
        const uint32_t u = tid + i * kThreads;
        xv[m][i] = load_unit<NORM>(x, rm, g.K, u < nunits ? u : nunits - 1);
      }
    }
  }
  if constexpr (NORM == kPrologueBf16) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) xv[m][i] = bf16_unit_to_f16(xv[m][i]);
  }
  if constexpr (NORM == kPrologueNorm) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const uint32_t rm = mrow0 + m < M ? mrow0 + m : M - 1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (i == 0 || nunits > (uint32_t)i * kThreads)
          xv[m][i] = normalise_unit(norm_w, inv_rms, rm, tid + i * kThreads, nunits, xv[m][i]);
    }
  }
}

// 2. Stage x: unit u = 8 consecutive k = (chunk, lane, j); image in the order a wave reads it, per-lane sums
//    beside it.  The caller puts the workgroup barrier behind it.
template <int BITS, int MR, int NORM>
__device__ __forceinline__ void stage_activations(const XImage<BITS, MR> g, const __half* x, uint32_t M, uint32_t mrow0,
                                                  const __half* norm_w, const float* inv_rms, int tid,
                                                  const u4 (&xv)[MR][4]) {
  constexpr int kXU = XImage<BITS, MR>::kXU;
  const uint32_t nunits = g.nunits, KH = g.KH;
  auto stage_unit = [&](int m, uint32_t u, const u4& v) {
    if (u < nunits) {
      const uint32_t c = u / (64 * kXU), rem = u % (64 * kXU), l = rem / kXU, j = rem % kXU;
      g.xl(m)[(c * kXU + j) * 64 + l] = BITS == 4 ? to_pair_order(v) : v;
      const h8 hv = __builtin_bit_cast(h8, v);
      float xs8 = 0.f, xo8 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        xs8 += (float)hv[e] + (float)hv[e + 1];
        xo8 += 1024.0f * (float)hv[e] + (BITS == 4 ? 64.0f : 1024.0f) * (float)hv[e + 1];
      }
      // the kXU units of a lane sit in adjacent threads of one quad (unit counts are multiples of 4)
      xs8 = dpp_add<0xB1>(xs8);
      xo8 = dpp_add<0xB1>(xo8);
      if (kXU == 4) {
        xs8 = dpp_add<0x4E>(xs8);
        xo8 = dpp_add<0x4E>(xo8);
      }
      if (j == 0) g.cs(m)[c * 64 + l] = make_float2(xo8, xs8);
    } else if (u < KH * 64 * kXU) {  // image positions past K: zeros
      const uint32_t c = u / (64 * kXU), rem = u % (64 * kXU), l = rem / kXU, j = rem % kXU;
      g.xl(m)[(c * kXU + j) * 64 + l] = (u4){0u, 0u, 0u, 0u};
      if (j == 0) g.cs(m)[c * 64 + l] = make_float2(0.f, 0.f);
    }
  };
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int i = 0; i < 4; ++i) stage_unit(m, tid + i * kThreads, xv[m][i]);
  // K > 16384: the remaining rounds, loaded here (behind the first weight loads; rare and long-running shapes)
  for (uint32_t u = tid + 4 * kThreads; u < KH * 64 * kXU; u += kThreads) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const uint32_t rm = mrow0 + m < M ? mrow0 + m : M - 1;
      u4 v = load_unit<NORM>(x, rm, g.K, u < nunits ? u : nunits - 1);
      if constexpr (NORM == kPrologueBf16) v = bf16_unit_to_f16(v);
      if constexpr (NORM == kPrologueNorm) v = normalise_unit(norm_w, inv_rms, rm, u, nunits, v);
      stage_unit(m, u, v);
    }
  }
}

// masks and offsets of the nibble unpacking, held in registers: and + or is one instruction
struct UnpackConsts { uint32_t m0, m1, k0, k1; };

// 3. One chunk of the wave's R rows against the registers of x read from LDS:
//    racc[r][m] += scale * (sum(x * (off + q)) - sum(off * x)) + bias * sum(x)
// (the products: xr = the lane's activations of the chunk in the order of the unpacking, k = their sums (sum(off * x), sum(x)))
template <int BITS, int R, int MR>
__device__ __forceinline__ void dot_rows(const uint32_t (&xr)[MR][XImage<BITS, MR>::kXU][4], const float2 (&k)[MR],
                                         const u4 (&w)[R], const uint32_t (&s)[R], const uint32_t (&b)[R],
                                         const UnpackConsts& uc, float (&racc)[R][MR]) {
  constexpr int kXU = XImage<BITS, MR>::kXU;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const u4 wv = w[r];
    const uint32_t wd[4] = {wv.x, wv.y, wv.z, wv.w};
    float acc0[MR], acc1[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc0[m] = acc1[m] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (BITS == 4) {
        const uint32_t hi = wd[j] >> 8;
        const h2 p0 = as_h2((wd[j] & uc.m0) | uc.k0), p1 = as_h2((wd[j] & uc.m1) | uc.k1);
        const h2 p2 = as_h2((hi & uc.m0) | uc.k0), p3 = as_h2((hi & uc.m1) | uc.k1);
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          acc0[m] = __builtin_amdgcn_fdot2(p0, as_h2(xr[m][j][0]), acc0[m], false);
          acc1[m] = __builtin_amdgcn_fdot2(p1, as_h2(xr[m][j][1]), acc1[m], false);
          acc0[m] = __builtin_amdgcn_fdot2(p2, as_h2(xr[m][j][2]), acc0[m], false);
          acc1[m] = __builtin_amdgcn_fdot2(p3, as_h2(xr[m][j][3]), acc1[m], false);
        }
      } else {  // bytes (q0,q1,q2,q3) -> (1024 + q0, 1024 + q1), (1024 + q2, 1024 + q3): natural order
        const int u = j >> 1, e = (j & 1) * 2;
        const h2 p0 = as_h2(__builtin_amdgcn_perm(0x64646464u, wd[j], 0x04010400u));
        const h2 p1 = as_h2(__builtin_amdgcn_perm(0x64646464u, wd[j], 0x04030402u));
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          acc0[m] = __builtin_amdgcn_fdot2(p0, as_h2(xr[m][u % kXU][e]), acc0[m], false);
          acc1[m] = __builtin_amdgcn_fdot2(p1, as_h2(xr[m][u % kXU][e + 1]), acc1[m], false);
        }
      }
    }
    const float sc = __half2float(__ushort_as_half((unsigned short)s[r]));
    const float bi = __half2float(__ushort_as_half((unsigned short)b[r]));
#pragma unroll
    for (int m = 0; m < MR; ++m) racc[r][m] += sc * ((acc0[m] + acc1[m]) - k[m].x) + bi * k[m].y;
  }
}

template <int BITS, int R, int MR>
__device__ __forceinline__ void dot_chunk(const XImage<BITS, MR> g, uint32_t c, int lane, const u4 (&w)[R],
                                          const uint32_t (&s)[R], const uint32_t (&b)[R], const UnpackConsts& uc,
                                          float (&racc)[R][MR]) {
  constexpr int kXU = XImage<BITS, MR>::kXU;
  uint32_t xr[MR][kXU][4];
  float2 k[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
#pragma unroll
    for (int j = 0; j < kXU; ++j) {
      const u4 v = g.xl(m)[(c * kXU + j) * 64 + lane];
      xr[m][j][0] = v.x; xr[m][j][1] = v.y; xr[m][j][2] = v.z; xr[m][j][3] = v.w;
    }
    k[m] = g.cs(m)[c * 64 + lane];
  }
  dot_rows<BITS, R, MR>(xr, k, w, s, b, uc, racc);
  // (several activation rows: keeps the LDS reads of the next chunk from being hoisted above this one, which would
  // double the registers of x that are live)
  if constexpr (MR > 1) __builtin_amdgcn_sched_barrier(0);
}

// R = weight rows per wave (1 or 2); NT = non-temporal weight loads (one pass over the weights);
// MR = activation rows per pass (1, 2 or 4): their registers share the unpacked weights, so a few
// rows cost one pass over the weights plus 16 dot instructions per row, chunk and lane.
// NORM = RMSNorm prologue applied while the activations are staged (kernels of their own: the extra
// registers would cost the plain kernels occupancy).
// KP = waves per weight row (1, 2 or 4; split K, the counterpart of affine_qmv_splitk_f16_q4 + qmm_splitk_accum_f16,
// quantized.rs:992-1233): wave w takes the chunks kp, kp + KP, ... of row w / KP (kp = w % KP) and the partial sums
// meet in workgroup memory.  For long rows of a short matrix, where one wave per row leaves most of the chip idle.
// GATHER = a weight matrix per activation row (gather_qmm with one row per index: the counterpart of
// gather_qmv_fast_f16_q4, quantized.rs:9752-9842); MR = 1.
template <int BITS, int GS, int R, bool NT, int MR, int NORM = 0, int KP = 1, bool GATHER = false>
// (8-bit, one row: asking the compiler for eight waves per SIMD changes no register count but the schedule;
// measured 4-13 % faster.  The 4-bit kernel would spill under that bound and is slower with it.  Two activation
// rows: without a bound the scheduler spends 124 registers on a schedule that is 12 % slower than the one it finds
// within the 96 of five waves per SIMD.)
__global__ __launch_bounds__(kThreads, (BITS == 8 && MR == 1 && R == 1) ? 8 : (MR == 2 ? 5 : 1)) void qmv_m1_kernel(M1Params p) {
  using Image = XImage<BITS, MR>;
  constexpr int kChunkK = Image::kChunkK, kLaneK = Image::kLaneK;
  constexpr int kLanesPerGroup = GS / kLaneK;  // whole lanes per quantisation group
  constexpr int kGroupsPerChunk = kChunkK / GS;
  static_assert(kLanesPerGroup >= 1, "a lane must not straddle quantisation groups");

  extern __shared__ __attribute__((aligned(16))) char lds[];
  // K need not be a multiple of the chunk: the lanes of the last chunk that lie past K read clamped
  // (valid) addresses and multiply them with a zeroed activation image, i.e. contribute nothing.
  const Image img(lds, p.K);
  const uint32_t K = p.K, KH = img.KH, G = K / GS;
  const uint32_t row_u4 = K / kLaneK;  // 16-byte pieces of a weight row

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  static_assert(KP == 1 || R == 1, "split rows: one row per wave group");
  const uint32_t row0 = blockIdx.x * (kWaves * R / KP) + (wave / KP) * R;
  const uint32_t kp = wave % KP;
  // this wave's chunks: kp, kp + KP, ... (KHw of them)
  const uint32_t KHw = KP == 1 ? KH : (KH > kp ? (KH - kp + KP - 1) / KP : 0u);
  const uint32_t mrow0 = blockIdx.y * MR;  // first activation row of this pass (rows past M repeat the last one, unstored)
  static_assert(!GATHER || (MR == 1 && KP == 1 && !NORM), "a weight matrix per activation row: one row per pass");
  uint64_t e_w = 0, e_s = 0;
  bool gather_zeros = false;
  if constexpr (GATHER) {
    const uint32_t e = p.gather_idx[p.gather_div > 1 ? (p.gather_row0 + mrow0) / p.gather_div : mrow0];
    gather_zeros = e >= p.n_experts;
    e_w = gather_zeros ? 0 : e * p.estride_w;
    e_s = gather_zeros ? 0 : e * p.estride_s;
  }

  // ---- 1. loads, small ones first (the memory counter retires in order): activations ... ------
  u4 xv[MR][4];
  load_activations<BITS, MR, NORM>(img, p.x, p.M, mrow0, p.norm_w, p.inv_rms, tid, xv);
  // ... the epilogue operand of the output this lane will write (lane r * MR + m) ...
  const uint32_t out_m = mrow0 + lane % MR, out_n = row0 + lane / MR;
  const bool writes = lane < R * MR && out_m < p.M;
  float epi_val = 0.f;
  if (p.epi_kind != EPI_NONE && writes) {
    const uint64_t oi = (uint64_t)out_m * p.N + out_n;
    epi_val = p.epi_dtype == RMLX_DTYPE_F32 ? static_cast<const float*>(p.epi)[oi]
                                            : __half2float(static_cast<const __half*>(p.epi)[oi]);
  }
  // ---- ... then the first two chunks of the wave's rows with their scales and biases ----------------
  struct Batch { u4 w[2][R]; uint32_t s[2][R], b[2][R]; };  // [chunk of the batch][row]
  const u4* wrow[R];
  const unsigned short* srow[R];
  const unsigned short* brow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    wrow[r] = reinterpret_cast<const u4*>(p.w + e_w + (uint64_t)(row0 + r) * (K * BITS / 32));
    srow[r] = reinterpret_cast<const unsigned short*>(p.s + e_s) + (uint64_t)(row0 + r) * G;
    brow[r] = reinterpret_cast<const unsigned short*>(p.b + e_s) + (uint64_t)(row0 + r) * G;
  }
  auto load_batch = [&](uint32_t c0, Batch& t) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = c0 + cc < KHw ? kp + KP * (c0 + cc) : KH - 1;  // an odd chunk count re-reads the last chunk (unused)
      uint32_t wi = c * 64 + lane, gi = c * kGroupsPerChunk + lane / kLanesPerGroup;
      wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K (last chunk of a K that is no chunk multiple)
      gi = gi < G ? gi : G - 1;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        t.s[cc][r] = srow[r][gi];
        t.b[cc][r] = brow[r][gi];
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
        t.w[cc][r] = NT ? __builtin_nontemporal_load(wrow[r] + wi) : wrow[r][wi];
    }
  };
  Batch ba, bb;
  load_batch(0, ba);

  // ---- 2. stage x into the LDS image ---------------------------------------------------------------------
  stage_activations<BITS, MR, NORM>(img, p.x, p.M, mrow0, p.norm_w, p.inv_rms, tid, xv);
  __syncthreads();

  // ---- 3. chunk by chunk: registers of x from LDS, then the wave's rows --------------------------------
  float racc[R][MR];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) racc[r][m] = 0.f;
  UnpackConsts uc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(uc.m0), "+s"(uc.m1), "+v"(uc.k0), "+v"(uc.k1));
  auto process = [&](uint32_t c0, const Batch& t) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = kp + KP * (c0 + cc);
      if (c0 + cc < KHw) dot_chunk<BITS, R, MR>(img, c, lane, t.w[cc], t.s[cc], t.b[cc], uc, racc);
    }
  };
  for (uint32_t c0 = 0; c0 < KHw; c0 += 4) {
    const bool more1 = c0 + 2 < KHw, more2 = c0 + 4 < KHw;
    if (more1) load_batch(c0 + 2, bb);
    process(c0, ba);
    if (more1) {
      if (more2) load_batch(c0 + 4, ba);
      process(c0 + 2, bb);
    }
  }

  // ---- 4. wave-wide sums; lane r * MR + m writes the output of (weight row r, activation row m) ------
  float mine = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float t = wave_sum(racc[r][m]);
      mine = lane == r * MR + m ? t : mine;
    }
  if constexpr (KP > 1) {  // partial sums of a row's KP waves, added in wave order by the first of them
    float* part = reinterpret_cast<float*>(lds);
    __syncthreads();  // every wave has read its activations
    if (lane < MR) part[wave * MR + lane] = mine;
    __syncthreads();
    if (lane < MR) {
      mine = part[wave * MR + lane];
#pragma unroll
      for (int q = 1; q < KP; ++q) mine += kp == 0 ? part[(wave + q) * MR + lane] : 0.f;
    }
  }
  if (writes && kp == 0) {  // residual add / SwiGLU gate in f32, one rounding (quantized.rs:3206-3246)
    if (p.epi_kind == EPI_RESIDUAL) mine += epi_val;
    else if (p.epi_kind == EPI_SWIGLU) mine = epi_val / (1.0f + __expf(-epi_val)) * mine;
    if (GATHER && gather_zeros) mine = 0.f;
    p.out[(uint64_t)out_m * p.N + out_n] = __float2half(mine);
  }
}

// The same kernel for matrices with more row blocks than the chip keeps resident: the grid is sized to the resident
// workgroups and each of them walks several row blocks (see `my_blocks`).
template <int BITS, int GS, int R, bool NT, int MR, int NORM = 0, bool GATHER = false>
// (8-bit, one row: asking the compiler for eight waves per SIMD changes no register count but the schedule;
// measured 4-13 % faster.  The 4-bit kernel would spill under that bound and is slower with it.)
__global__ __launch_bounds__(kThreads, 1) void qmv_m1_loop_kernel(M1Params p) {
  using Image = XImage<BITS, MR>;
  constexpr int kChunkK = Image::kChunkK, kLaneK = Image::kLaneK;
  constexpr int kLanesPerGroup = GS / kLaneK;  // whole lanes per quantisation group
  constexpr int kGroupsPerChunk = kChunkK / GS;
  static_assert(kLanesPerGroup >= 1, "a lane must not straddle quantisation groups");

  extern __shared__ __attribute__((aligned(16))) char lds[];
  // K need not be a multiple of the chunk: the lanes of the last chunk that lie past K read clamped
  // (valid) addresses and multiply them with a zeroed activation image, i.e. contribute nothing.
  const Image img(lds, p.K);
  const uint32_t K = p.K, KH = img.KH, G = K / GS;
  const uint32_t row_u4 = K / kLaneK;  // 16-byte pieces of a weight row

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t mrow0 = blockIdx.y * MR;  // first activation row of this pass (rows past M repeat the last one, unstored)
  static_assert(!GATHER || (MR == 1 && !NORM), "a weight matrix per activation row: one row per pass");
  uint64_t e_w = 0, e_s = 0;
  bool gather_zeros = false;
  if constexpr (GATHER) {
    const uint32_t e = p.gather_idx[p.gather_div > 1 ? (p.gather_row0 + mrow0) / p.gather_div : mrow0];
    gather_zeros = e >= p.n_experts;
    e_w = gather_zeros ? 0 : e * p.estride_w;
    e_s = gather_zeros ? 0 : e * p.estride_s;
  }
  // Row blocks (kWaves * R weight rows) of this workgroup: blockIdx.x, blockIdx.x + gridDim.x, ...  The launcher
  // sizes the grid to what the chip keeps resident, so the activations are staged once per workgroup and the
  // next block's weights are already in flight while the current block is multiplied.
  const uint32_t nblk = p.N / (kWaves * R);
  const uint32_t my_blocks = blockIdx.x < nblk ? (nblk - 1 - blockIdx.x) / gridDim.x + 1 : 0u;
  auto block_row0 = [&](uint32_t i) { return (blockIdx.x + i * gridDim.x) * (kWaves * R) + wave * R; };

  // ---- 1. loads, small ones first (the memory counter retires in order): activations ... ------
  u4 xv[MR][4];
  load_activations<BITS, MR, NORM>(img, p.x, p.M, mrow0, p.norm_w, p.inv_rms, tid, xv);
  // ---- ... then the first two chunks of the wave's rows with their scales and biases ----------------
  // A batch is two chunks of the wave's rows in one block; the batches of all blocks of the workgroup form one
  // sequence (block 0: chunks 0-1, 2-3, ..., block 1: chunks 0-1, ...) that is loaded one batch ahead.
  struct Batch { u4 w[2][R]; uint32_t s[2][R], b[2][R]; float epi; };  // [chunk of the batch][row]; epi: see below
  const uint32_t batches_per_block = (KH + 1) / 2, n_batches = my_blocks * batches_per_block;
  // the output this lane writes at the end of a block: (weight row lane / MR, activation row lane % MR)
  const uint32_t out_m = mrow0 + lane % MR;
  const bool writes = lane < R * MR && out_m < p.M;
  uint32_t ld_blk = 0, ld_c0 = 0;  // block and first chunk of the next batch to load
  auto load_batch = [&](Batch& t) {
    const uint32_t row0 = block_row0(ld_blk);
    const u4* wrow[R];
    const unsigned short* srow[R];
    const unsigned short* brow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      wrow[r] = reinterpret_cast<const u4*>(p.w + e_w + (uint64_t)(row0 + r) * (K * BITS / 32));
      srow[r] = reinterpret_cast<const unsigned short*>(p.s + e_s) + (uint64_t)(row0 + r) * G;
      brow[r] = reinterpret_cast<const unsigned short*>(p.b + e_s) + (uint64_t)(row0 + r) * G;
    }
    // the epilogue operand of the block's outputs travels with its first batch
    t.epi = 0.f;
    if (ld_c0 == 0 && p.epi_kind != EPI_NONE && writes) {
      const uint64_t oi = (uint64_t)out_m * p.N + row0 + lane / MR;
      t.epi = p.epi_dtype == RMLX_DTYPE_F32 ? static_cast<const float*>(p.epi)[oi]
                                            : __half2float(static_cast<const __half*>(p.epi)[oi]);
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = ld_c0 + cc < KH ? ld_c0 + cc : KH - 1;  // an odd chunk count re-reads the last chunk (unused)
      uint32_t wi = c * 64 + lane, gi = c * kGroupsPerChunk + lane / kLanesPerGroup;
      wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K (last chunk of a K that is no chunk multiple)
      gi = gi < G ? gi : G - 1;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        t.s[cc][r] = srow[r][gi];
        t.b[cc][r] = brow[r][gi];
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
        t.w[cc][r] = NT ? __builtin_nontemporal_load(wrow[r] + wi) : wrow[r][wi];
    }
    ld_c0 += 2;
    if (ld_c0 >= KH) { ld_c0 = 0; ++ld_blk; }
  };
  Batch ba, bb;
  if (n_batches > 0) load_batch(ba);

  // ---- 2. stage x into the LDS image ---------------------------------------------------------------------
  stage_activations<BITS, MR, NORM>(img, p.x, p.M, mrow0, p.norm_w, p.inv_rms, tid, xv);
  __syncthreads();

  // ---- 3. batch by batch: registers of x from LDS, then the wave's rows; 4. at the end of a block the wave-wide
  //         sums: lane r * MR + m writes the output of (weight row r, activation row m) ---------------------------
  float racc[R][MR];
  UnpackConsts uc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(uc.m0), "+s"(uc.m1), "+v"(uc.k0), "+v"(uc.k1));
  uint32_t pr_blk = 0, pr_c0 = 0;  // block and first chunk of the batch being processed
  float epi_val = 0.f;
  auto process = [&](const Batch& t) {
    if (pr_c0 == 0) {
      epi_val = t.epi;
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) racc[r][m] = 0.f;
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = pr_c0 + cc;
      if (c < KH) dot_chunk<BITS, R, MR>(img, c, lane, t.w[cc], t.s[cc], t.b[cc], uc, racc);
    }
    pr_c0 += 2;
    if (pr_c0 >= KH) {  // the block is complete
      float mine = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const float t2 = wave_sum(racc[r][m]);
          mine = lane == r * MR + m ? t2 : mine;
        }
      if (writes) {  // residual add / SwiGLU gate in f32, one rounding (quantized.rs:3206-3246)
        if (p.epi_kind == EPI_RESIDUAL) mine += epi_val;
        else if (p.epi_kind == EPI_SWIGLU) mine = epi_val / (1.0f + __expf(-epi_val)) * mine;
        if (GATHER && gather_zeros) mine = 0.f;
        p.out[(uint64_t)out_m * p.N + block_row0(pr_blk) + lane / MR] = __float2half(mine);
      }
      pr_c0 = 0;
      ++pr_blk;
    }
  };
  for (uint32_t u = 0; u < n_batches; u += 2) {
    const bool more1 = u + 1 < n_batches, more2 = u + 2 < n_batches;
    if (more1) load_batch(bb);
    process(ba);
    if (more1) {
      if (more2) load_batch(ba);
      process(bb);
    }
  }
}

// ---- gate / up projection of single rows through chosen experts (routed blocks of one token or a few) ---------------
// Assignment a (blockIdx.y) multiplies activation row a / top_k with expert idx[a] of two stacked matrices: a wave owns
// gate row r and up row r of that expert over the whole K (the two-row form of the kernel above: the activation
// registers read from LDS serve both) and writes silu(gate . x) * (up . x), rounded once, to out[a, r].  An expert index
// outside [0, n_experts) writes zeros.  The counterpart of gather_qmv_fast_f16_q4 (quantized.rs:9752-9842, one activation
// row per index) with the SwiGLU of ExpertGroup::grouped_forward (crates/rmlx-nn/src/expert_group.rs:445-524) behind it.
struct M1GateUpParams {
  const uint32_t* w0; const __half* s0; const __half* b0;  // gate, expert 0
  const uint32_t* w1; const __half* s1; const __half* b1;  // up, expert 0
  uint64_t estride_w, estride_s;                           // u32 words / halves per expert
  const __half* x;       // [T, K] f16
  const uint32_t* idx;   // [assignments] expert of every assignment
  __half* out;           // [assignments, N] f16
  uint32_t N, K, top_k, n_experts;
  // Routing done by the workgroups themselves (idx == null): f32 logits [T, n_experts], optional bias [n_experts]; every
  // workgroup ranks its token's experts (one wave, the routing kernels' own code, while the activations arrive), and the
  // first workgroup of a token's first assignment also writes the token's picks and weights
  const float* route_logits;
  const float* route_bias;
  uint32_t* route_idx_out;
  float* route_w_out;
  int32_t route_renorm;
};

// The expert of assignment a: from the list, or ranked here by the workgroup (after the caller has requested its
// activations).
__device__ __forceinline__ uint32_t gate_up_expert(const M1GateUpParams& p, uint32_t a, bool first_wg) {
  if (p.idx != nullptr) return p.idx[a];
  __shared__ __attribute__((aligned(16))) uint32_t ws[512];
  __shared__ uint32_t pick_idx[8];
  __shared__ float pick_w[8];
  const uint32_t t = a / p.top_k, pick = a - t * p.top_k;
  route::token_picks_workgroup(p.route_logits, p.route_bias, p.n_experts, p.top_k, p.route_renorm, t, ws, pick_idx, pick_w);
  if (first_wg && pick == 0 && threadIdx.x < p.top_k) {
    p.route_idx_out[(size_t)t * p.top_k + threadIdx.x] = pick_idx[threadIdx.x];
    p.route_w_out[(size_t)t * p.top_k + threadIdx.x] = pick_w[threadIdx.x];
  }
  return pick_idx[pick];
}

template <int BITS, int GS, bool XBF = false>  // XBF: the activations are bf16 bits, converted while they are staged
__global__ __launch_bounds__(kThreads, 1) void qmv_m1_gate_up_kernel(M1GateUpParams p) {
  using Image = XImage<BITS, 1>;
  constexpr int kChunkK = Image::kChunkK, kLaneK = Image::kLaneK;
  constexpr int kLanesPerGroup = GS / kLaneK, kGroupsPerChunk = kChunkK / GS;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const Image img(lds, p.K);
  const uint32_t K = p.K, KH = img.KH, G = K / GS, row_u4 = K / kLaneK;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t a = blockIdx.y, row = blockIdx.x * kWaves + wave;
  const __half* x = p.x + (uint64_t)(a / p.top_k) * K;

  // loads, small ones first (the memory counter retires in order): the activations, the expert, then the rows
  u4 xv[1][4];
  load_activations<BITS, 1, XBF ? kPrologueBf16 : kPrologueNone>(img, x, 1u, 0u, nullptr, nullptr, tid, xv);
  uint32_t expert = gate_up_expert(p, a, blockIdx.x == 0);
  const bool zeros = expert >= p.n_experts;
  expert = zeros ? 0u : expert;
  struct Batch { u4 w[2][2]; uint32_t s[2][2], b[2][2]; };  // [chunk of the batch][gate, up]
  const u4* wrow[2];
  const unsigned short* srow[2];
  const unsigned short* brow[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    wrow[r] = reinterpret_cast<const u4*>((r == 0 ? p.w0 : p.w1) + expert * p.estride_w + (uint64_t)row * (K * BITS / 32));
    srow[r] = reinterpret_cast<const unsigned short*>((r == 0 ? p.s0 : p.s1) + expert * p.estride_s) + (uint64_t)row * G;
    brow[r] = reinterpret_cast<const unsigned short*>((r == 0 ? p.b0 : p.b1) + expert * p.estride_s) + (uint64_t)row * G;
  }
  auto load_batch = [&](uint32_t c0, Batch& t) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = c0 + cc < KH ? c0 + cc : KH - 1;  // an odd chunk count re-reads the last chunk (unused)
      uint32_t wi = c * 64 + lane, gi = c * kGroupsPerChunk + lane / kLanesPerGroup;
      wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K (last chunk of a K that is no chunk multiple)
      gi = gi < G ? gi : G - 1;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        t.s[cc][r] = srow[r][gi];
        t.b[cc][r] = brow[r][gi];
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) t.w[cc][r] = __builtin_nontemporal_load(wrow[r] + wi);
    }
  };
  Batch ba, bb;
  load_batch(0, ba);
  stage_activations<BITS, 1, XBF ? kPrologueBf16 : kPrologueNone>(img, x, 1u, 0u, nullptr, nullptr, tid, xv);
  __syncthreads();

  float racc[2][1] = {{0.f}, {0.f}};
  UnpackConsts uc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(uc.m0), "+s"(uc.m1), "+v"(uc.k0), "+v"(uc.k1));
  auto process = [&](uint32_t c0, const Batch& t) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
      if (c0 + cc < KH) dot_chunk<BITS, 2, 1>(img, c0 + cc, lane, t.w[cc], t.s[cc], t.b[cc], uc, racc);
  };
  for (uint32_t c0 = 0; c0 < KH; c0 += 4) {
    const bool more1 = c0 + 2 < KH, more2 = c0 + 4 < KH;
    if (more1) load_batch(c0 + 2, bb);
    process(c0, ba);
    if (more1) {
      if (more2) load_batch(c0 + 4, ba);
      process(c0 + 2, bb);
    }
  }
  const float g = wave_sum(racc[0][0]), u = wave_sum(racc[1][0]);
  if (lane == 0) p.out[(uint64_t)a * p.N + row] = __float2half(zeros ? 0.f : g / (1.0f + __expf(-g)) * u);
}

// The same for more row blocks than the chip keeps resident (a few tokens: assignments x N / 8 blocks): the grid is
// (resident workgroups / assignments, assignments) and a workgroup walks the row blocks blockIdx.x, blockIdx.x + gridDim.x,
// ... of its assignment, staging the activations once, the next block's weights in flight while the current one is multiplied.
template <int BITS, int GS, bool XBF = false>
__global__ __launch_bounds__(kThreads, 1) void qmv_m1_gate_up_loop_kernel(M1GateUpParams p) {
  using Image = XImage<BITS, 1>;
  constexpr int kChunkK = Image::kChunkK, kLaneK = Image::kLaneK;
  constexpr int kLanesPerGroup = GS / kLaneK, kGroupsPerChunk = kChunkK / GS;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const Image img(lds, p.K);
  const uint32_t K = p.K, KH = img.KH, G = K / GS, row_u4 = K / kLaneK;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t a = blockIdx.y;
  const __half* x = p.x + (uint64_t)(a / p.top_k) * K;
  const uint32_t nblk = p.N / kWaves;
  const uint32_t my_blocks = blockIdx.x < nblk ? (nblk - 1 - blockIdx.x) / gridDim.x + 1 : 0u;
  auto block_row = [&](uint32_t i) { return (blockIdx.x + i * gridDim.x) * kWaves + wave; };

  u4 xv[1][4];
  load_activations<BITS, 1, XBF ? kPrologueBf16 : kPrologueNone>(img, x, 1u, 0u, nullptr, nullptr, tid, xv);
  uint32_t expert = gate_up_expert(p, a, blockIdx.x == 0);
  const bool zeros = expert >= p.n_experts;
  expert = zeros ? 0u : expert;
  struct Batch { u4 w[2][2]; uint32_t s[2][2], b[2][2]; };  // [chunk of the batch][gate, up]
  const uint32_t batches_per_block = (KH + 1) / 2, n_batches = my_blocks * batches_per_block;
  uint32_t ld_blk = 0, ld_c0 = 0;  // block and first chunk of the next batch to load
  auto load_batch = [&](Batch& t) {
    const uint32_t row = block_row(ld_blk);
    const u4* wrow[2];
    const unsigned short* srow[2];
    const unsigned short* brow[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      wrow[r] = reinterpret_cast<const u4*>((r == 0 ? p.w0 : p.w1) + expert * p.estride_w + (uint64_t)row * (K * BITS / 32));
      srow[r] = reinterpret_cast<const unsigned short*>((r == 0 ? p.s0 : p.s1) + expert * p.estride_s) + (uint64_t)row * G;
      brow[r] = reinterpret_cast<const unsigned short*>((r == 0 ? p.b0 : p.b1) + expert * p.estride_s) + (uint64_t)row * G;
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const uint32_t c = ld_c0 + cc < KH ? ld_c0 + cc : KH - 1;  // an odd chunk count re-reads the last chunk (unused)
      uint32_t wi = c * 64 + lane, gi = c * kGroupsPerChunk + lane / kLanesPerGroup;
      wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K (last chunk of a K that is no chunk multiple)
      gi = gi < G ? gi : G - 1;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        t.s[cc][r] = srow[r][gi];
        t.b[cc][r] = brow[r][gi];
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) t.w[cc][r] = __builtin_nontemporal_load(wrow[r] + wi);
    }
    ld_c0 += 2;
    if (ld_c0 >= KH) { ld_c0 = 0; ++ld_blk; }
  };
  Batch ba, bb;
  if (n_batches > 0) load_batch(ba);
  stage_activations<BITS, 1, XBF ? kPrologueBf16 : kPrologueNone>(img, x, 1u, 0u, nullptr, nullptr, tid, xv);
  __syncthreads();

  float racc[2][1];
  UnpackConsts uc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(uc.m0), "+s"(uc.m1), "+v"(uc.k0), "+v"(uc.k1));
  uint32_t pr_blk = 0, pr_c0 = 0;  // block and first chunk of the batch being processed
  auto process = [&](const Batch& t) {
    if (pr_c0 == 0) { racc[0][0] = 0.f; racc[1][0] = 0.f; }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
      if (pr_c0 + cc < KH) dot_chunk<BITS, 2, 1>(img, pr_c0 + cc, lane, t.w[cc], t.s[cc], t.b[cc], uc, racc);
    pr_c0 += 2;
    if (pr_c0 >= KH) {  // the block is complete
      const float g = wave_sum(racc[0][0]), u = wave_sum(racc[1][0]);
      if (lane == 0) p.out[(uint64_t)a * p.N + block_row(pr_blk)] = __float2half(zeros ? 0.f : g / (1.0f + __expf(-g)) * u);
      pr_c0 = 0;
      ++pr_blk;
    }
  };
  for (uint32_t u = 0; u < n_batches; u += 2) {
    const bool more1 = u + 1 < n_batches, more2 = u + 2 < n_batches;
    if (more1) load_batch(bb);
    process(ba);
    if (more1) {
      if (more2) load_batch(ba);
      process(bb);
    }
  }
}

// ---- down projection of a few tokens with the weighted combine behind it, single-row layout -----------------------
// One workgroup per (token t, block of R output columns): wave k multiplies the hidden row of the token's k-th
// assignment (row t * top_k + k of h) with R weight rows of that assignment's expert; K is at most NC chunks, so a lane
// keeps its activations (and their sums) in registers -- no image in LDS, no barrier before the products.  The eight
// waves' results meet in LDS and thread r adds out[t, n] = sum_k w[t,k] * y_k[n] in ascending k, the order and f32
// arithmetic of the combine kernel, and writes f16.  An expert index outside [0, n_experts) contributes nothing.
struct M1DownParams {
  const uint32_t* w; const __half* s; const __half* b;  // stacked down weights, expert 0
  uint64_t estride_w, estride_s;                        // u32 words / halves per expert
  const __half* h;        // [T * top_k, K] f16
  const uint32_t* idx;    // [T * top_k]
  const float* wts;       // [T * top_k]
  __half* out;            // [T, N] f16
  uint32_t N, K, top_k, n_experts;
};

// HALF (rows of at most 32 sixteen-byte pieces: K <= 1024 at 4 bits, 512 at 8): the two halves of a wave take R weight rows each
// -- lanes 0-31 rows n0 .. n0+R-1, lanes 32-63 the next R -- so a short row does not leave more than half of the lanes
// without a load (K = 768 at 4 bits: 24 of 32 lanes busy instead of 24 of 64).  Same products, same summation order per row.
template <int BITS, int GS, int NC, int R, bool HALF = false>
__global__ __launch_bounds__(kThreads, 2) void qmv_m1_down_combine_kernel(M1DownParams p) {
  static_assert(!HALF || NC == 1, "half-wave rows: one chunk");
  using Image = XImage<BITS, 1>;
  constexpr int kChunkK = Image::kChunkK, kLaneK = Image::kLaneK, kXU = Image::kXU;
  constexpr int kLanesPerGroup = GS / kLaneK, kGroupsPerChunk = kChunkK / GS;
  constexpr int RW = HALF ? 2 * R : R;  // weight rows per wave
  __shared__ float red[kWaves][RW];
  const int tid = threadIdx.x, wlane = tid & 63, lane = HALF ? (wlane & 31) : wlane, half = HALF ? (wlane >> 5) : 0;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t K = p.K, G = K / GS, row_u4 = K / kLaneK, nunits = K / 8;
  const uint32_t t = blockIdx.y, n0 = blockIdx.x * RW + half * R, a = t * p.top_k + wave;
  uint32_t expert = 0xFFFFFFFFu;
  float cw = 0.f;
  if ((uint32_t)wave < p.top_k) {
    expert = p.idx[a];
    cw = p.wts[a];
  }
  float res[R];
#pragma unroll
  for (int r = 0; r < R; ++r) res[r] = 0.f;
  if (expert < p.n_experts) {  // (wave-uniform)
    // loads, small ones first: the lane's activations, the scales and biases, then the weights
    const u4* xg = reinterpret_cast<const u4*>(p.h + (uint64_t)a * K);
    u4 xv[NC][kXU];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int j = 0; j < kXU; ++j) {
        const uint32_t u = (c * 64 + lane) * kXU + j;
        xv[c][j] = xg[u < nunits ? u : nunits - 1];
      }
    u4 wv[NC][R];
    uint32_t sv[NC][R], bv[NC][R];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      uint32_t wi = c * 64 + lane, gi = c * kGroupsPerChunk + lane / kLanesPerGroup;
      wi = wi < row_u4 ? wi : row_u4 - 1;  // lanes past K meet zeros in the activations
      gi = gi < G ? gi : G - 1;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        sv[c][r] = reinterpret_cast<const unsigned short*>(p.s + expert * p.estride_s)[(uint64_t)(n0 + r) * G + gi];
        bv[c][r] = reinterpret_cast<const unsigned short*>(p.b + expert * p.estride_s)[(uint64_t)(n0 + r) * G + gi];
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
        wv[c][r] = reinterpret_cast<const u4*>(p.w + expert * p.estride_w + (uint64_t)(n0 + r) * (K * BITS / 32))[wi];
    }
    UnpackConsts uc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(uc.m0), "+s"(uc.m1), "+v"(uc.k0), "+v"(uc.k1));
    float racc[R][1];
#pragma unroll
    for (int r = 0; r < R; ++r) racc[r][0] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      // the lane's activations in the order of the unpacking and their sums (zeros past K)
      uint32_t xr[1][kXU][4];
      float xs = 0.f, xo = 0.f;
#pragma unroll
      for (int j = 0; j < kXU; ++j) {
        const bool inside = (c * 64 + lane) * kXU + j < nunits;
        const u4 raw = inside ? xv[c][j] : (u4){0u, 0u, 0u, 0u};
        const u4 v = BITS == 4 ? to_pair_order(raw) : raw;
        xr[0][j][0] = v.x; xr[0][j][1] = v.y; xr[0][j][2] = v.z; xr[0][j][3] = v.w;
        const h8 hv = __builtin_bit_cast(h8, raw);
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          xs += (float)hv[e] + (float)hv[e + 1];
          xo += 1024.0f * (float)hv[e] + (BITS == 4 ? 64.0f : 1024.0f) * (float)hv[e + 1];
        }
      }
      const float2 k1[1] = {make_float2(xo, xs)};
      dot_rows<BITS, R, 1>(xr, k1, wv[c], sv[c], bv[c], uc, racc);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) res[r] = (HALF ? half_wave_sum(racc[r][0]) : wave_sum(racc[r][0])) * cw;
  }
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) red[wave][half * R + r] = res[r];
  }
  __syncthreads();
  if (tid < RW) {
    float acc = 0.f;
    for (uint32_t k = 0; k < p.top_k; ++k) acc += red[k][tid];  // ascending k, as the combine kernel adds
    p.out[(uint64_t)t * p.N + blockIdx.x * RW + tid] = __float2half(acc);
  }
}

// LDS bytes per activation row: image and per-lane sums over whole chunks
template <int BITS>
size_t lds_per_row(uint32_t K) {
  const size_t chunk_k = 8192 / BITS, chunks = (K + chunk_k - 1) / chunk_k;
  return chunks * (chunk_k * 2 + 64 * sizeof(float2));
}

// Workgroups of `kernel` that the chip keeps resident at once (cached per host thread, kernel and LDS size: kernels of
// one signature share this function, so the kernel's address is part of the key).
template <typename Kernel>
uint32_t resident_workgroups(Kernel kernel, size_t lds) {
  struct Entry { const void* fn; size_t lds; uint32_t wgs; };
  static thread_local std::vector<Entry> cache;
  const void* fn = reinterpret_cast<const void*>(kernel);
  for (const Entry& e : cache)
    if (e.fn == fn && e.lds == lds) return e.wgs;
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, lds) != hipSuccess || per_cu < 1) per_cu = 1;
  const uint32_t wgs = (uint32_t)per_cu * (uint32_t)ctx().num_cus;
  cache.push_back({fn, lds, wgs});
  return wgs;
}

template <int BITS, int GS, int R, bool NT, int MR, int NORM, int KP = 1, bool GATHER = false>
void launch_k(const M1Params& p, size_t lds, hipStream_t s) {
  if constexpr (KP > 1) {  // split rows: short matrices only, every row group has its workgroup
    hipLaunchKernelGGL((qmv_m1_kernel<BITS, GS, R, NT, MR, NORM, KP>), dim3(p.N / (kWaves / KP), (p.M + MR - 1) / MR),
                       dim3(kThreads), lds, s, p);
    return;
  }
  // one workgroup per row block while all of them are resident together, else as many as are (they loop)
  auto looping = qmv_m1_loop_kernel<BITS, GS, R, NT, MR, NORM, GATHER>;
  const uint32_t nblk = p.N / (kWaves * R), passes = (p.M + MR - 1) / MR;
  uint32_t gx = resident_workgroups(looping, lds) / passes;
  gx = gx < 1 ? 1 : gx;
  // (as many workgroups as are resident, even where that leaves some of them one block more than others: fewer
  // workgroups with equal shares are slower, 8.1 against 6.7 us at N = 9216)
  if (gx < nblk) hipLaunchKernelGGL(looping, dim3(gx, passes), dim3(kThreads), lds, s, p);
  else hipLaunchKernelGGL((qmv_m1_kernel<BITS, GS, R, NT, MR, NORM, 1, GATHER>), dim3(nblk, passes), dim3(kThreads), lds, s, p);
}

template <int BITS, int R, bool NT, int MR, int KP = 1>
void launch_r(const M1Params& p, uint32_t group_size, hipStream_t s) {
  const size_t lds = (size_t)MR * lds_per_row<BITS>(p.K);
  if constexpr (KP > 1) {
    switch (group_size) {
      case 32: launch_k<BITS, 32, R, NT, MR, false, KP>(p, lds, s); break;
      case 64: launch_k<BITS, 64, R, NT, MR, false, KP>(p, lds, s); break;
      default: launch_k<BITS, 128, R, NT, MR, false, KP>(p, lds, s); break;
    }
    return;
  }
  if constexpr (NT && MR <= 2) {  // the prologues are fused for one or two rows in one pass
    if (p.norm_w != nullptr) {
      switch (group_size) {
        case 32: launch_k<BITS, 32, R, NT, MR, kPrologueNorm>(p, lds, s); break;
        case 64: launch_k<BITS, 64, R, NT, MR, kPrologueNorm>(p, lds, s); break;
        default: launch_k<BITS, 128, R, NT, MR, kPrologueNorm>(p, lds, s); break;
      }
      return;
    }
    if (p.x_bf16 == 1) {
      switch (group_size) {
        case 32: launch_k<BITS, 32, R, NT, MR, kPrologueBf16>(p, lds, s); break;
        case 64: launch_k<BITS, 64, R, NT, MR, kPrologueBf16>(p, lds, s); break;
        default: launch_k<BITS, 128, R, NT, MR, kPrologueBf16>(p, lds, s); break;
      }
      return;
    }
    if (p.x_bf16 == 2) {
      switch (group_size) {
        case 32: launch_k<BITS, 32, R, NT, MR, kPrologueF32>(p, lds, s); break;
        case 64: launch_k<BITS, 64, R, NT, MR, kPrologueF32>(p, lds, s); break;
        default: launch_k<BITS, 128, R, NT, MR, kPrologueF32>(p, lds, s); break;
      }
      return;
    }
  }
  switch (group_size) {
    case 32: launch_k<BITS, 32, R, NT, MR, kPrologueNone>(p, lds, s); break;
    case 64: launch_k<BITS, 64, R, NT, MR, kPrologueNone>(p, lds, s); break;
    default: launch_k<BITS, 128, R, NT, MR, kPrologueNone>(p, lds, s); break;
  }
}

template <int BITS>
void launch_bits(const M1Params& p, uint32_t group_size, hipStream_t s) {
  // activation rows per pass: as many of 4 / 2 as fit the default dynamic LDS limit
  const size_t per_row = lds_per_row<BITS>(p.K);
  int mr = p.M >= 3 ? 4 : (int)p.M;
  while (mr > 1 && (size_t)mr * per_row > 65536) mr /= 2;
  const bool one_pass = (p.M + mr - 1) / mr == 1;  // several passes re-read the weights from L2: no non-temporal loads
  if (mr == 4) {
    if (one_pass) launch_r<BITS, 1, true, 4>(p, group_size, s); else launch_r<BITS, 1, false, 4>(p, group_size, s);
  } else if (mr == 2) {
    if (one_pass) launch_r<BITS, 1, true, 2>(p, group_size, s); else launch_r<BITS, 1, false, 2>(p, group_size, s);
  } else {
    // two weight rows per wave for long rows (more bytes in flight per wave) and, with 4-bit weights, for
    // tall matrices (the activation registers read from LDS serve both rows; measured 3-9 % from N = 12288
    // on; the 8-bit kernel reads half as many activations per weight byte and is faster with one), else one
    // (also where two rows per wave make the grid a whole number of workgroups per CU, at least two: N = 8192 on 256 CUs
    // 5.8 against 6.2 us at K = 4096, 10.0 against 10.5 us at K = 8192; N = 4096, one workgroup per CU: 4.25 against 4.04)
    const uint32_t cus_m1 = (uint32_t)ctx().num_cus;
    const bool two = (p.K >= 12288 || (BITS == 4 && (p.N >= 12288 || (p.N % (kWaves * 2 * cus_m1) == 0 && p.N >= kWaves * 4 * cus_m1)))) &&
                     p.N % (kWaves * 2) == 0;
    // Long rows of a short matrix (the reference's split-K case, K > 8192 and N <= 2048, quantized.rs:7246-7250):
    // with one wave per row the grid would not fill the chip, so 2 or 4 waves share a row until there are two
    // workgroups per CU (every wave keeps at least two chunks).
    const uint32_t chunks = (p.K * BITS + 8191) / 8192, cus = (uint32_t)ctx().num_cus;
    int kp = 1;
    while (kp < 4 && p.N / kWaves * kp < 2 * cus && chunks >= 4u * kp && p.N % (kWaves / (2 * kp)) == 0) kp *= 2;
    if (kp > 1 && p.norm_w == nullptr && !p.x_bf16 && one_pass) {
      if (kp == 2) launch_r<BITS, 1, true, 1, 2>(p, group_size, s); else launch_r<BITS, 1, true, 1, 4>(p, group_size, s);
      return;
    }
    if (one_pass) {
      if (two) launch_r<BITS, 2, true, 1>(p, group_size, s); else launch_r<BITS, 1, true, 1>(p, group_size, s);
    } else {
      if (two) launch_r<BITS, 2, false, 1>(p, group_size, s); else launch_r<BITS, 1, false, 1>(p, group_size, s);
    }
  }
}

}  // namespace

bool qmv_m1_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  if (bits != 4 && bits != 8) return false;
  if (group_size != 32 && group_size != 64 && group_size != 128) return false;
  // a lane's 16 bytes of a row must be whole (32 values at 4 bits, 16 at 8) and groups must not straddle lanes
  if (!(N > 0 && K > 0 && N % kWaves == 0 && K % (128 / bits) == 0 && K % group_size == 0 && K <= kMaxK)) return false;
  return (bits == 4 ? lds_per_row<4>(K) : lds_per_row<8>(K)) <= 65536;
}

// The RMSNorm prologue is fused when all rows (at most two) share one pass over the weights.
bool qmv_m1_fuses_norm(uint32_t M, uint32_t K, uint32_t bits) {
  return M >= 1 && M <= 2 && (size_t)M * (bits == 4 ? lds_per_row<4>(K) : lds_per_row<8>(K)) <= 65536;
}

int32_t launch_qmv_m1(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, int epi_kind, const void* epi,
                      int32_t epi_dtype, const __half* norm_w, const float* inv_rms, hipStream_t stream, int32_t x_bf16) {
  if (!qmv_m1_supported(N, K, group_size, bits))
    return fail(RMLX_INVALID_SHAPE, "qmv_m1: unsupported shape N=%u K=%u bits=%u group_size=%u", N, K, bits, group_size);
  if (x_bf16 && (norm_w != nullptr || !qmv_m1_fuses_norm(M, K, bits)))
    return fail(RMLX_RUNTIME_ERROR, "qmv_m1: bf16 activations are converted inside for at most two rows in one pass and without the RMSNorm prologue (M=%u K=%u)", M, K);
  if (M == 0) return RMLX_OK;
  if (M > 65535) return fail(RMLX_INVALID_SHAPE, "qmv_m1: at most 65535 rows per launch (M=%u)", M);
  if (norm_w != nullptr && !qmv_m1_fuses_norm(M, K, bits))
    return fail(RMLX_RUNTIME_ERROR, "qmv_m1: the RMSNorm prologue is fused for at most two rows in one pass (M=%u K=%u)", M, K);
  M1Params p{w, s, b, x, out, N, K, M, epi_kind, epi_dtype, epi, norm_w, inv_rms};
  p.x_bf16 = x_bf16;
  if (bits == 4) launch_bits<4>(p, group_size, stream);
  else launch_bits<8>(p, group_size, stream);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

namespace {
template <int BITS>
void launch_gather_bits(const M1Params& p, uint32_t group_size, bool two, hipStream_t stream) {
  const size_t lds = lds_per_row<BITS>(p.K);
  switch (group_size) {
    case 32: if (two) launch_k<BITS, 32, 2, false, 1, false, 1, true>(p, lds, stream); else launch_k<BITS, 32, 1, false, 1, false, 1, true>(p, lds, stream); break;
    case 64: if (two) launch_k<BITS, 64, 2, false, 1, false, 1, true>(p, lds, stream); else launch_k<BITS, 64, 1, false, 1, false, 1, true>(p, lds, stream); break;
    default: if (two) launch_k<BITS, 128, 2, false, 1, false, 1, true>(p, lds, stream); else launch_k<BITS, 128, 1, false, 1, false, 1, true>(p, lds, stream); break;
  }
}
}  // namespace

// gather_qmm with one activation row per index: row m of x [batch, K] through expert idx[m] of the stacked 4- or 8-bit
// weights, out [batch, N] f16.  One launch, no chunk table: the activation row of a pass picks its matrix.
int32_t launch_qmv_m1_gather(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                             uint32_t n_experts, const __half* x, const uint32_t* idx, uint32_t batch, __half* out, uint32_t N,
                             uint32_t K, uint32_t group_size, uint32_t bits, hipStream_t stream, uint32_t rows_per_index) {
  if (!qmv_m1_supported(N, K, group_size, bits))
    return fail(RMLX_INVALID_SHAPE, "qmv_m1 gather: unsupported shape N=%u K=%u bits=%u group_size=%u", N, K, bits, group_size);
  // (weights loaded with the ordinary cache policy: two indices may name one expert)
  const bool two = (K >= 12288 || (bits == 4 && N >= 12288)) && N % (kWaves * 2) == 0;
  for (uint32_t first = 0; first < batch; first += 65535) {  // the activation row is the second grid dimension
    const uint32_t rows = batch - first < 65535 ? batch - first : 65535;
    M1Params p{w, s, b, x + (uint64_t)first * K, out + (uint64_t)first * N, N, K, rows, EPI_NONE, 0, nullptr, nullptr, nullptr,
               rows_per_index > 1 ? idx : idx + first, estride_w, estride_s, n_experts};
    if (rows_per_index > 1) { p.gather_div = rows_per_index; p.gather_row0 = first; }
    if (bits == 4) launch_gather_bits<4>(p, group_size, two, stream);
    else launch_gather_bits<8>(p, group_size, two, stream);
    RMLX_HIP_CHECK(hipGetLastError());
  }
  return RMLX_OK;
}

bool qmv_m1_gate_up_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  return qmv_m1_supported(N, K, group_size, bits);
}

namespace {
template <int BITS, int GS, bool XBF>
void launch_gate_up_x(const M1GateUpParams& p, uint32_t assignments, hipStream_t stream) {
  const size_t lds = lds_per_row<BITS>(p.K);
  const uint32_t nblk = p.N / kWaves;
  // one workgroup per row block while all of them are resident together, else as many as are (they loop)
  auto looping = qmv_m1_gate_up_loop_kernel<BITS, GS, XBF>;
  uint32_t gx = resident_workgroups(looping, lds) / assignments;
  gx = gx < 1 ? 1 : gx;
  if (gx < nblk) hipLaunchKernelGGL(looping, dim3(gx, assignments), dim3(kThreads), lds, stream, p);
  else hipLaunchKernelGGL((qmv_m1_gate_up_kernel<BITS, GS, XBF>), dim3(nblk, assignments), dim3(kThreads), lds, stream, p);
}
template <int BITS, int GS>
void launch_gate_up(const M1GateUpParams& p, uint32_t assignments, bool x_bf16, hipStream_t stream) {
  if (x_bf16) launch_gate_up_x<BITS, GS, true>(p, assignments, stream);
  else launch_gate_up_x<BITS, GS, false>(p, assignments, stream);
}
}  // namespace

int32_t launch_qmv_m1_gate_up(const QmvArgs& a, uint32_t bits, const uint32_t* idx, uint32_t assignments, uint32_t top_k,
                              uint32_t n_experts, hipStream_t stream) {
  if (!qmv_m1_gate_up_supported(a.N, a.K, a.group_size, bits))
    return fail(RMLX_INVALID_SHAPE, "qmv_m1 gate/up: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, bits, a.group_size);
  if (assignments == 0) return RMLX_OK;
  const bool routes = idx == nullptr;
  if (assignments > 65535 || top_k == 0 || a.w1 == nullptr || a.out_f32 || a.ld_out != a.N ||
      (routes && (a.route_logits == nullptr || a.route_idx_out == nullptr || a.route_w_out == nullptr || top_k > 8 ||
                  n_experts > 256 || assignments % top_k != 0)))
    return fail(RMLX_RUNTIME_ERROR, "qmv_m1 gate/up: needs an expert per assignment (or logits of whole tokens, at most 8 picks "
                                    "of 256 experts), both matrices and a dense f16 output");
  M1GateUpParams p{a.w0, a.s0, a.b0, a.w1, a.s1, a.b1, a.expert_stride_w, a.expert_stride_s, a.x, idx,
                   static_cast<__half*>(a.out), a.N, a.K, top_k, n_experts,
                   a.route_logits, a.route_bias, a.route_idx_out, a.route_w_out, a.route_renorm};
  if (bits == 4) {
    switch (a.group_size) {
      case 32: launch_gate_up<4, 32>(p, assignments, a.x_bf16 != 0, stream); break;
      case 64: launch_gate_up<4, 64>(p, assignments, a.x_bf16 != 0, stream); break;
      default: launch_gate_up<4, 128>(p, assignments, a.x_bf16 != 0, stream); break;
    }
  } else {
    switch (a.group_size) {
      case 32: launch_gate_up<8, 32>(p, assignments, a.x_bf16 != 0, stream); break;
      case 64: launch_gate_up<8, 64>(p, assignments, a.x_bf16 != 0, stream); break;
      default: launch_gate_up<8, 128>(p, assignments, a.x_bf16 != 0, stream); break;
    }
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

// Chunks of K the down + combine kernel keeps in registers (0: the shape is not for it)
// (8-bit weights only: with 4-bit rows a wave's share is too small to pay -- hidden 4096 / intermediate 1536, 4 tokens at
// top-8: the block 64.7 us with four rows per wave, 70.0 us with eight, against 59.7 us with the wave-per-tile kernel)
static int down_combine_chunks(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, uint32_t top_k) {
  if ((bits != 4 && bits != 8) || (group_size != 32 && group_size != 64 && group_size != 128)) return 0;
  const uint32_t chunk_k = 8192 / bits;
  if (N == 0 || K == 0 || N % 4 != 0 || K % (128 / bits) != 0 || K % group_size != 0 || top_k < 1 || top_k > 8) return 0;
  return K <= chunk_k ? 1 : (K <= 2 * chunk_k ? 2 : 0);
}

bool qmv_m1_down_combine_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, uint32_t top_k) {
  return down_combine_chunks(N, K, group_size, bits, top_k) != 0;
}

namespace {
template <int BITS, int GS>
void launch_down_combine(const M1DownParams& p, int chunks, uint32_t T, hipStream_t stream) {
  // (four rows per wave: the weights of a pass fit the registers of two workgroups per CU)
  // (short rows, N in whole blocks of 8: two groups of four rows per wave)
  if (chunks == 1 && p.K * BITS / 8 <= 512 && p.N % 8 == 0)
    hipLaunchKernelGGL((qmv_m1_down_combine_kernel<BITS, GS, 1, 4, true>), dim3(p.N / 8, T), dim3(kThreads), 0, stream, p);
  else if (chunks == 1) hipLaunchKernelGGL((qmv_m1_down_combine_kernel<BITS, GS, 1, 4>), dim3(p.N / 4, T), dim3(kThreads), 0, stream, p);
  else hipLaunchKernelGGL((qmv_m1_down_combine_kernel<BITS, GS, 2, 4>), dim3(p.N / 4, T), dim3(kThreads), 0, stream, p);
}
}  // namespace

int32_t launch_qmv_m1_down_combine(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                                   uint32_t n_experts, const __half* h, const uint32_t* idx, const float* wts, uint32_t T,
                                   uint32_t top_k, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, __half* out,
                                   hipStream_t stream) {
  const int chunks = down_combine_chunks(N, K, group_size, bits, top_k);
  if (chunks == 0)
    return fail(RMLX_INVALID_SHAPE, "qmv_m1 down + combine: unsupported shape N=%u K=%u bits=%u group_size=%u top_k=%u", N, K, bits,
                group_size, top_k);
  if (T == 0) return RMLX_OK;
  if (T > 65535) return fail(RMLX_INVALID_SHAPE, "qmv_m1 down + combine: at most 65535 tokens per launch (T=%u)", T);
  M1DownParams p{w, s, b, estride_w, estride_s, h, idx, wts, out, N, K, top_k, n_experts};
  if (bits == 8) {
    switch (group_size) {
      case 32: launch_down_combine<8, 32>(p, chunks, T, stream); break;
      case 64: launch_down_combine<8, 64>(p, chunks, T, stream); break;
      default: launch_down_combine<8, 128>(p, chunks, T, stream); break;
    }
  } else {
    switch (group_size) {
      case 32: launch_down_combine<4, 32>(p, chunks, T, stream); break;
      case 64: launch_down_combine<4, 64>(p, chunks, T, stream); break;
      default: launch_down_combine<4, 128>(p, chunks, T, stream); break;
    }
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
