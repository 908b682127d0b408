// Quantized GEMM for gfx950 (prefill, M > 16): dequantize weight tiles into LDS, f16 / bf16
// MFMA with f32 accumulation, f16 output.
//
// Replaces the reference's affine_qmm_nax_q4 / affine_qmm_steel4sg_splitk_q4 /
// affine_qmm_mma_q8 (crates/rmlx-core/src/ops/quantized.rs:3331-3565, 4572-4786, 5838-5971).
//
// Tile BM x 64 x 64, 256 threads = 4 waves stacked along M, v_mfma_f32_16x16x32_{f16,bf16}.
// Per 64-wide k step every thread dequantizes 16 weights once for the whole workgroup
// (w = scale*q + bias evaluated in packed f16 after an exact magic-number int->f16 conversion;
// in f32 for the bf16 variant) and writes them to LDS in natural k order; the four waves read
// the weight fragments from there.  Activations never touch LDS: each wave loads its own rows
// from global memory directly in MFMA operand layout (LDS bandwidth is the scarce resource
// here).  Global loads run kDepth steps ahead in a register ring; LDS is double-buffered with
// one barrier per step.  Workgroup ids are remapped so that the tiles sharing a
// weight panel run on the same XCD (shared L2).
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int BK = 64;
constexpr int LDK = BK + 8;  // padded LDS row (halves)
constexpr int kDepth = 4;    // global-load prefetch distance in k-steps (must be even)

struct QmmParams {
  const uint32_t* w; const __half* s; const __half* b;
  const uint16_t* x;  // f16 or bf16 bits in fragment-major layout (see relayout_a_kernel)
  __half* out;
  uint32_t M, N, K;
  uint32_t Kx;  // columns of the fragment-major activations: K rounded up to whole unrolled iterations, zeros past K
  uint32_t group_size;
  // grouped launches (one expert per 64-row tile): table of (expert, first row, rows; bit 31 of the rows: an expert index out of
  // range, zeros are written) per row tile and its length on the device, expert strides in u32 words / halves
  const uint32_t* tile_tab; const uint32_t* n_tiles;
  uint64_t estride_w, estride_s;
  // K split (SPLITK launches): workgroup (x, y) runs steps y * Kx / 64 / ksplit .. of tile x and writes f32 partial sums
  // [ksplit, M, N]; splitk_sum_kernel adds them up
  float* partial; uint32_t ksplit;
};


__device__ __forceinline__ uint32_t h2bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// 8 Q4 values of one word -> 8 f16 weights (natural k order), w = s*q + b.
__device__ __forceinline__ u4 dequant_q4_word_f16(uint32_t w, h2 s2, h2 b2) {
  const uint32_t t = w >> 8;
  const h2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f}, k64 = {(_Float16)64.0f, (_Float16)64.0f};
  h2 p0 = __builtin_bit_cast(h2, (w & 0x000F000Fu) | 0x64006400u) - k1024;  // q0, q4
  h2 p1 = __builtin_bit_cast(h2, (w & 0x00F000F0u) | 0x54005400u) - k64;    // q1, q5
  h2 p2 = __builtin_bit_cast(h2, (t & 0x000F000Fu) | 0x64006400u) - k1024;  // q2, q6
  h2 p3 = __builtin_bit_cast(h2, (t & 0x00F000F0u) | 0x54005400u) - k64;    // q3, q7
  const uint32_t f0 = h2bits(p0 * s2 + b2), f1 = h2bits(p1 * s2 + b2);
  const uint32_t f2 = h2bits(p2 * s2 + b2), f3 = h2bits(p3 * s2 + b2);
  u4 o;
  o.x = __builtin_amdgcn_perm(f1, f0, 0x05040100u);  // w0, w1
  o.y = __builtin_amdgcn_perm(f3, f2, 0x05040100u);  // w2, w3
  o.z = __builtin_amdgcn_perm(f1, f0, 0x07060302u);  // w4, w5
  o.w = __builtin_amdgcn_perm(f3, f2, 0x07060302u);  // w6, w7
  return o;
}

// 4 Q8 values of one word -> 4 f16 weights.
__device__ __forceinline__ u2 dequant_q8_word_f16(uint32_t w, h2 s2, h2 b2) {
  const h2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  h2 p0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) - k1024;  // q0, q1
  h2 p1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) - k1024;  // q2, q3
  u2 o;
  o.x = h2bits(p0 * s2 + b2);
  o.y = h2bits(p1 * s2 + b2);
  return o;
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  bf2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}

// 4 Q8 values -> 4 bf16 weights, arithmetic in f32.
__device__ __forceinline__ u2 dequant_q8_word_bf16(uint32_t w, float s, float b) {
  const float q0 = (float)(w & 0xFFu), q1 = (float)((w >> 8) & 0xFFu);
  const float q2 = (float)((w >> 16) & 0xFFu), q3 = (float)(w >> 24);
  u2 o;
  o.x = pack_bf16(s * q0 + b, s * q1 + b);
  o.y = pack_bf16(s * q2 + b, s * q3 + b);
  return o;
}

// TAIL: K is a multiple of 64 but not of 256.  The loop runs over the activations' padded width; the steps past K multiply
// zero activations by the weights of the last real step (weight, scale and bias loads are clamped to the row), and scales
// and biases are fetched as single halves (a row of them starts on a 2-byte boundary only when K / 64 is odd).
// GS: the quantisation group size.  A thread's 16 values of a step lie in one group at every size; at 32 and 128 the
// (scale, bias) of a step is fetched as single halves like in the TAIL form (group 2 * step + quarter / 2, step / 2).
// GROUPED: row tile t of the grid takes its expert and its rows from the tile table; its activations are tile t of the
// fragment-major workspace (relayout_grouped_kernel), so p.M is the grid's row extent, max_tiles * BM.
// SPLITK: few tiles (a short batch over a narrow matrix) leave most CUs idle, so the k loop is cut into p.ksplit ranges of
// whole unrolled iterations, each of which begins before K ends (checked on the host).
template <int BM, int BN, int BITS, bool XBF16, bool TAIL, int GS, bool GROUPED = false, bool SPLITK = false>
__global__ __launch_bounds__(kThreads) void qmm_kernel(QmmParams p) {
  static_assert(GS == 32 || GS == 64 || GS == 128, "group sizes of the format");
  constexpr bool kHalfLoads = TAIL || GS != 64;
  constexpr int WM = BM / 4;                   // rows per wave: the 4 waves are stacked along M
  constexpr int TI = WM / 16, TJ = BN / 16;    // 16x16 MFMA tiles per wave
  constexpr int KK = BK / 32;                  // MFMA k-substeps per step
  constexpr int kValuPerMfma = (BITS == 4 ? 48 : 40) / (KK * TI * TJ) + 1;  // staging VALU ops slotted after each MFMA
  constexpr int WPT = BN * BK * BITS / 32 / kThreads;  // weight words per thread per step
  static_assert(BN == 64, "weight staging assumes 4 threads per weight row");
  static_assert(WPT == (BITS == 4 ? 2 : 4), "16 weights per thread per step");

  // Only the dequantized weight tile goes through LDS (it is shared by the four waves).  Each
  // wave reads its own activation rows straight from global memory in MFMA operand layout.
  // Four LDS buffers: step s multiplies out of registers filled from buffer s%4 one step earlier,
  // prefetches the fragments of step s+1 from buffer (s+1)%4 and writes the tile of step s+2.
  __shared__ __attribute__((aligned(16))) uint16_t Bs[4][BN * LDK];
  static_assert(kDepth == 4, "buffer indices below are derived from the unrolled step index");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;

  // ---- tile assignment: consecutive ids go to different XCDs; give each XCD whole weight panels
  const uint32_t tiles_m = (p.M + BM - 1) / BM, tiles_n = p.N / BN;
  const uint32_t total = tiles_m * tiles_n;
  uint32_t id = blockIdx.x;
  if (!GROUPED && total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const uint32_t m0 = (GROUPED ? id / tiles_n : id % tiles_m) * BM, n0 = (GROUPED ? id % tiles_n : id / tiles_m) * BN;
  uint32_t row_lo = 0, row_cnt = 0;
  uint64_t e_w = 0, e_s = 0;
  if (GROUPED) {
    const uint32_t te = m0 / BM;
    if (te >= *p.n_tiles) return;
    const uint32_t expert = p.tile_tab[3 * te], c = p.tile_tab[3 * te + 2];
    row_lo = p.tile_tab[3 * te + 1];
    row_cnt = c & 0x7FFFFFFFu;
    if (c >> 31) {  // rows whose expert index is out of range: zeros
      for (uint32_t i = threadIdx.x; i < row_cnt * BN; i += kThreads)
        p.out[(uint64_t)(row_lo + i / BN) * p.N + n0 + i % BN] = __float2half(0.f);
      return;
    }
    e_w = expert * p.estride_w;
    e_s = expert * p.estride_s;
  }

  const uint32_t K = p.K, gpr = K / GS;
  const uint32_t Kx = TAIL ? p.Kx : K;
  const int steps = SPLITK ? (int)(Kx / BK / p.ksplit) : (int)(Kx / BK);  // a multiple of kDepth (checked on the host)
  const int sbase = SPLITK ? (int)blockIdx.y * steps : 0;                 // the first step of this workgroup's range
  const int wlast = (int)(K / BK) - 1 - sbase;  // the last step that has weights, counted from sbase (>= 0)

  // weight staging coordinates
  const int brow = tid >> 2, bq = tid & 3;  // weight row in tile, 16-value quarter of the 64-k step
  const uint32_t* wptr = p.w + e_w + (uint64_t)(n0 + brow) * (K * BITS / 32) + bq * WPT + (uint32_t)sbase * (BK * BITS / 32);
  const __half* sptr = p.s + e_s + (uint64_t)(n0 + brow) * gpr + (uint32_t)sbase * BK / GS;
  const __half* bptr = p.b + e_s + (uint64_t)(n0 + brow) * gpr + (uint32_t)sbase * BK / GS;

  // activation fragments: block (16-row tile, 32-wide k chunk) = 64 lanes x 16 bytes, contiguous,
  // already in MFMA operand order.  Tiles past the last one re-read the last tile (their results
  // are never stored); unconditional loads keep the number of outstanding loads known to the
  // compiler, i.e. exact s_waitcnt vmcnt counts.
  // A wave of a grouped tile whose rows all lie past the tile's last row (its results are never stored) reads the rows of
  // wave 0 instead of its own zeros: those lines are in the CU's cache already, so a tile of few rows fetches them once.
  const u4* aptr[TI];
  const uint32_t mt_last = (p.M + 15) / 16 - 1;
  const uint32_t wrow = GROUPED && (uint32_t)(wave * WM) >= row_cnt ? 0u : (uint32_t)(wave * WM);
#pragma unroll
  for (int i = 0; i < TI; ++i) {
    const uint32_t mt = (m0 + wrow) / 16 + i;
    aptr[i] = reinterpret_cast<const u4*>(p.x) + (uint64_t)(mt < mt_last ? mt : mt_last) * (Kx / 32) * 64 + lane +
              (uint32_t)sbase * (KK * 64);
  }

  // Register ring of kDepth k-steps: global loads run kDepth steps ahead of the MFMAs.  Scales
  // and biases are fetched four groups (one unrolled iteration) at a time.
  u4 areg[kDepth][KK][TI];
  uint32_t wreg[kDepth][WPT];
  u2 sb_cur[2], sb_next[2];  // [0] scales, [1] biases of 4 consecutive groups

  auto load_a = [&](int step, int slot) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int i = 0; i < TI; ++i)
        areg[slot][kk][i] = aptr[i][(step * KK + kk) * 64];
  };
  auto load_w = [&](int step, int slot) {
    if (TAIL) step = step < wlast ? step : wlast;
    if (BITS == 4) {
      const u2 v = *reinterpret_cast<const u2*>(wptr + step * (BK * BITS / 32));
      wreg[slot][0] = v.x; wreg[slot][1] = v.y;
    } else {
      const u4 v = *reinterpret_cast<const u4*>(wptr + step * (BK * BITS / 32));
      wreg[slot][0] = v.x; wreg[slot][1] = v.y; wreg[slot][WPT - 2] = v.z; wreg[slot][WPT - 1] = v.w;
    }
  };
  // single halves (kHalfLoads): loaded as they are and packed into the two words only when the round that requested them
  // ends -- packed at once, every round would wait for its own loads
  auto load_halves = [&](int step0, uint32_t (&sv)[4], uint32_t (&bv)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int st = step0 + e < wlast ? step0 + e : wlast;
      const int gq = GS == 32 ? 2 * st + (bq >> 1) : GS == 128 ? st >> 1 : st;
      sv[e] = reinterpret_cast<const uint16_t*>(sptr)[gq];
      bv[e] = reinterpret_cast<const uint16_t*>(bptr)[gq];
    }
  };
  auto pack_halves = [&](const uint32_t (&sv)[4], const uint32_t (&bv)[4], u2 (&dst)[2]) {
    dst[0] = (u2){sv[0] | (sv[1] << 16), sv[2] | (sv[3] << 16)};
    dst[1] = (u2){bv[0] | (bv[1] << 16), bv[2] | (bv[3] << 16)};
  };
  auto load_sb = [&](int group0, u2 (&dst)[2]) {
    if (kHalfLoads) {  // group0 is a step index: the groups of this thread's quarter of steps group0 .. group0 + 3
      uint32_t sv[4], bv[4];
      load_halves(group0, sv, bv);
      pack_halves(sv, bv, dst);
    } else {
      dst[0] = *reinterpret_cast<const u2*>(sptr + group0);
      dst[1] = *reinterpret_cast<const u2*>(bptr + group0);
    }
  };
  auto pick16 = [](const u2& v, int e) -> uint16_t {  // element e (0..3) of four packed halves
    const uint32_t wd = e < 2 ? v.x : v.y;
    return (uint16_t)((e & 1) ? wd >> 16 : wd & 0xFFFFu);
  };

  // dequantize the weights held in ring slot `slot` (scale / bias bits given) into LDS buffer `buf`
  auto store_lds = [&](int buf, int slot, uint16_t sbits, uint16_t bbits) {
    uint16_t* dst = &Bs[buf][brow * LDK + bq * 16];
    if (XBF16) {
      const float s = __half2float(__ushort_as_half(sbits)), b = __half2float(__ushort_as_half(bbits));
      const u2 lo = dequant_q8_word_bf16(wreg[slot][0], s, b), l2 = dequant_q8_word_bf16(wreg[slot][1], s, b);
      const u2 h1 = dequant_q8_word_bf16(wreg[slot][WPT - 2], s, b), h2v = dequant_q8_word_bf16(wreg[slot][WPT - 1], s, b);
      *reinterpret_cast<u4*>(dst) = (u4){lo.x, lo.y, l2.x, l2.y};
      *reinterpret_cast<u4*>(dst + 8) = (u4){h1.x, h1.y, h2v.x, h2v.y};
    } else {
      const _Float16 sh = __builtin_bit_cast(_Float16, sbits), bh = __builtin_bit_cast(_Float16, bbits);
      const h2 s2 = {sh, sh}, b2 = {bh, bh};
      if (BITS == 4) {
        *reinterpret_cast<u4*>(dst) = dequant_q4_word_f16(wreg[slot][0], s2, b2);
        *reinterpret_cast<u4*>(dst + 8) = dequant_q4_word_f16(wreg[slot][1], s2, b2);
      } else {
        const u2 a0 = dequant_q8_word_f16(wreg[slot][0], s2, b2), a1 = dequant_q8_word_f16(wreg[slot][1], s2, b2);
        const u2 a2 = dequant_q8_word_f16(wreg[slot][WPT - 2], s2, b2), a3 = dequant_q8_word_f16(wreg[slot][WPT - 1], s2, b2);
        *reinterpret_cast<u4*>(dst) = (u4){a0.x, a0.y, a1.x, a1.y};
        *reinterpret_cast<u4*>(dst + 8) = (u4){a2.x, a2.y, a3.x, a3.y};
      }
    }
  };
  auto read_frags = [&](int buf, u4 (&bf)[KK][TJ]) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
        bf[kk][j] = *reinterpret_cast<const u4*>(&Bs[buf][(j * 16 + r16) * LDK + kk * 32 + g * 8]);
  };

  f4 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

  // ---- prologue: fill the ring, stage tiles 0 and 1, fetch the fragments of step 0 ------------------
  const int last = steps - 1;
  load_sb(0, sb_cur);
  load_sb(steps > 4 ? 4 : 0, sb_next);
#pragma unroll
  for (int d = 0; d < kDepth; ++d) { load_a(d, d); load_w(d, d); }
  store_lds(0, 0, pick16(sb_cur[0], 0), pick16(sb_cur[1], 0));
  store_lds(1, 1, pick16(sb_cur[0], 1), pick16(sb_cur[1], 1));
  // weight slots 0 and 1 are consumed: refill them with steps 4 and 5
  load_w(4 < last ? 4 : last, 0);
  load_w(5 < last ? 5 : last, 1);
  __syncthreads();
  u4 bf[2][KK][TJ];
  read_frags(0, bf[0]);

  for (int step0 = 0; step0 < steps; step0 += kDepth) {
    // scales / biases of groups step0+8 .. step0+11 (needed two iterations from now)
    u2 sb_nn[2];
    uint32_t sv_nn[4], bv_nn[4];
    if (kHalfLoads) load_halves(step0 + 8 < steps ? step0 + 8 : 0, sv_nn, bv_nn);
    else load_sb(step0 + 8 < steps ? step0 + 8 : 0, sb_nn);
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int step = step0 + d;
      // fragments of the next step (its tile was written during the previous step)
      read_frags((d + 1) & 3, bf[(d + 1) & 1]);
      // tile of step+2: weights sit in ring slot (d+2)&3, their group is step+2
      {
        const int e = (d + 2) & 3;
        const u2& sv = d < 2 ? sb_cur[0] : sb_next[0];
        const u2& bv = d < 2 ? sb_cur[1] : sb_next[1];
        store_lds((d + 2) & 3, e, pick16(sv, e), pick16(bv, e));
      }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
          for (int j = 0; j < TJ; ++j) {
            if (XBF16)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, areg[d][kk][i]),
                                                                  __builtin_bit_cast(b8, bf[d & 1][kk][j]), acc[i][j], 0, 0, 0);
            else
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, areg[d][kk][i]),
                                                                 __builtin_bit_cast(h8, bf[d & 1][kk][j]), acc[i][j], 0, 0, 0);
          }
      // refill: activations of step+4 into slot d, weights of step+6 into slot (d+2)&3 (both just
      // consumed); the tail re-reads the last step instead of branching around the loads
      load_a(step + 4 < last ? step + 4 : last, d);
      load_w(step + 6 < last ? step + 6 : last, (d + 2) & 3);
      // recipe: LDS reads first, then each MFMA followed by a few staging VALU ops; the two LDS
      // writes and the global loads are spread over the second half
      __builtin_amdgcn_sched_group_barrier(0x100, KK * TJ, 0);
#pragma unroll
      for (int q = 0; q < KK * TI * TJ; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0);
        if (q >= KK * TI * TJ / 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        if (q == KK * TI * TJ / 2 || q == KK * TI * TJ / 2 + 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
      __syncthreads();
    }
    sb_cur[0] = sb_next[0]; sb_cur[1] = sb_next[1];
    if (kHalfLoads) pack_halves(sv_nn, bv_nn, sb_nn);
    sb_next[0] = sb_nn[0]; sb_next[1] = sb_nn[1];
  }

  // accumulator lane (r16, g) holds column n = r16 and rows 4g..4g+3 of each 16x16 tile
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const uint32_t m = m0 + wave * WM + i * 16 + g * 4 + v;
        const uint32_t nn = n0 + j * 16 + r16;
        if (GROUPED) {
          const uint32_t local = m - m0;
          if (local < row_cnt) p.out[(uint64_t)(row_lo + local) * p.N + nn] = __float2half(acc[i][j][v]);
        } else if (SPLITK) {
          if (m < p.M) p.partial[((uint64_t)blockIdx.y * p.M + m) * p.N + nn] = acc[i][j][v];
        } else if (m < p.M) {
          p.out[(uint64_t)m * p.N + nn] = __float2half(acc[i][j][v]);
        }
      }
}

// Activations [M,K] (f16 / bf16 / f32, row-major) -> fragment-major f16 or bf16: for every
// 16-row tile and 32-wide k chunk, 64 consecutive 16-byte units, unit (r + 16 g) = row r of the
// tile, k = 8g..8g+7 of the chunk -- exactly what lane r+16g feeds to the MFMA.  A fragment load
// in the GEMM is then one fully coalesced 1 KB access instead of 16 half-used cache lines.
// The dtype cast is fused in.
__global__ __launch_bounds__(256) void relayout_a_kernel(const void* __restrict__ src, int src_dtype,
                                                         u4* __restrict__ dst, uint32_t M, uint32_t K,
                                                         uint32_t Kx, int to_bf16) {
  const uint32_t kchunks = Kx / 32;  // chunks past K hold zeros
  const uint64_t units = (uint64_t)((M + 15) / 16) * kchunks * 64;
  for (uint64_t u = (uint64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += (uint64_t)gridDim.x * 256) {
    const uint32_t lane = (uint32_t)(u & 63);
    const uint64_t blk = u >> 6;
    const uint32_t mt = (uint32_t)(blk / kchunks), kc = (uint32_t)(blk % kchunks);
    uint32_t row = mt * 16 + (lane & 15);
    if (row >= M) row = M - 1;
    const uint64_t off = (uint64_t)row * K + kc * 32 + (lane >> 4) * 8;
    u4 o;
    if (kc * 32 >= K) {
      o = (u4){0u, 0u, 0u, 0u};
    } else if (src_dtype == RMLX_DTYPE_F32) {
      const float* f = reinterpret_cast<const float*>(src) + off;
      uint32_t w[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (to_bf16) w[q] = pack_bf16(f[2 * q], f[2 * q + 1]);
        else {
          const h2 v = {(_Float16)f[2 * q], (_Float16)f[2 * q + 1]};
          w[q] = h2bits(v);
        }
      }
      o = (u4){w[0], w[1], w[2], w[3]};
    } else {
      o = *reinterpret_cast<const u4*>(reinterpret_cast<const uint16_t*>(src) + off);
      const bool is_bf16 = src_dtype == RMLX_DTYPE_BF16;
      if (is_bf16 != (to_bf16 != 0)) {  // bf16 <-> f16 through f32
        uint32_t w[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float lo, hi;
          if (is_bf16) {
            lo = __uint_as_float(w[q] << 16);
            hi = __uint_as_float(w[q] & 0xFFFF0000u);
          } else {
            const h2 v = __builtin_bit_cast(h2, w[q]);
            lo = (float)v[0];
            hi = (float)v[1];
          }
          if (to_bf16) w[q] = pack_bf16(lo, hi);
          else {
            const h2 v = {(_Float16)lo, (_Float16)hi};
            w[q] = h2bits(v);
          }
        }
        o = (u4){w[0], w[1], w[2], w[3]};
      }
    }
    dst[u] = o;
  }
}

// The same layout for the row tiles of a grouped launch: tile t (16 * frags rows of one expert: positions first .. first +
// rows - 1 of the table entry, through the row map where there is one; rows past the entry's repeat its last row) fills
// fragments frags * t .. frags * t + frags - 1 of the workspace.  f16 activations.
__global__ __launch_bounds__(256) void relayout_grouped_kernel(const __half* __restrict__ src, const uint32_t* __restrict__ row_map,
                                                               const uint32_t* __restrict__ tile_tab, const uint32_t* __restrict__ n_tiles,
                                                               uint32_t max_tiles, u4* __restrict__ dst, uint32_t K, uint32_t Kx,
                                                               uint32_t frags) {
  const uint32_t kchunks = Kx / 32, per_tile = frags * kchunks * 64, nt = *n_tiles;
  const uint64_t units = (uint64_t)max_tiles * per_tile;
  for (uint64_t u = (uint64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += (uint64_t)gridDim.x * 256) {
    const uint32_t te = (uint32_t)(u / per_tile);
    if (te >= nt) return;  // (units ascend with the thread's stride)
    const uint32_t r = (uint32_t)(u % per_tile), lane = r & 63, blk = r >> 6, frag = blk / kchunks, kc = blk % kchunks;
    const uint32_t cnt = tile_tab[3 * te + 2] & 0x7FFFFFFFu;
    uint32_t local = frag * 16 + (lane & 15);
    if (local >= cnt) local = cnt - 1;
    uint32_t row = tile_tab[3 * te + 1] + local;
    if (row_map != nullptr) row = row_map[row];
    u4 o = (u4){0u, 0u, 0u, 0u};
    if (kc * 32 < K) o = *reinterpret_cast<const u4*>(src + (uint64_t)row * K + kc * 32 + (lane >> 4) * 8);
    dst[u] = o;
  }
}

// out[m, n] = sum over the K ranges of partial[r, m, n], four columns per thread.
__global__ __launch_bounds__(256) void splitk_sum_kernel(const float* __restrict__ partial, __half* __restrict__ out, uint64_t quads,
                                                         uint32_t ksplit) {
  const uint64_t q = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= quads) return;
  f4 a = reinterpret_cast<const f4*>(partial)[q];
  for (uint32_t r = 1; r < ksplit; ++r) {
    const f4 b = reinterpret_cast<const f4*>(partial)[r * quads + q];
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
  }
  const h2 lo = {(_Float16)a.x, (_Float16)a.y}, hi = {(_Float16)a.z, (_Float16)a.w};
  reinterpret_cast<u2*>(out)[q] = (u2){h2bits(lo), h2bits(hi)};
}

template <int BITS, int GS>
void launch_grouped_t(const QmmParams& p, uint32_t max_tiles, uint32_t tile_rows, hipStream_t s) {
  const uint32_t tiles = max_tiles * (p.N / 64);
  if (tile_rows == 128) {
    if (p.Kx != p.K) hipLaunchKernelGGL((qmm_kernel<128, 64, BITS, false, true, GS, true>), dim3(tiles), dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmm_kernel<128, 64, BITS, false, false, GS, true>), dim3(tiles), dim3(kThreads), 0, s, p);
  } else {
    if (p.Kx != p.K) hipLaunchKernelGGL((qmm_kernel<64, 64, BITS, false, true, GS, true>), dim3(tiles), dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmm_kernel<64, 64, BITS, false, false, GS, true>), dim3(tiles), dim3(kThreads), 0, s, p);
  }
}

template <int BM, int BITS, bool XBF16>
void launch_t(const QmmParams& p, hipStream_t s) {
  const uint32_t tiles = ((p.M + BM - 1) / BM) * (p.N / 64);
  const bool tail = p.Kx != p.K;
  if (!XBF16 && p.group_size == 32) {
    if (tail) hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, false, true, 32>), dim3(tiles), dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, false, false, 32>), dim3(tiles), dim3(kThreads), 0, s, p);
  } else if (!XBF16 && p.group_size == 128) {
    if (tail) hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, false, true, 128>), dim3(tiles), dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, false, false, 128>), dim3(tiles), dim3(kThreads), 0, s, p);
  } else {
    if (tail) hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, XBF16, true, 64>), dim3(tiles), dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((qmm_kernel<BM, 64, BITS, XBF16, false, 64>), dim3(tiles), dim3(kThreads), 0, s, p);
  }
}

uint32_t padded_k(uint32_t K) { return (K + BK * kDepth - 1) / (BK * kDepth) * (BK * kDepth); }

}  // namespace


bool qmm_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  return (group_size == 32 || group_size == 64 || group_size == 128) && (bits == 4 || bits == 8) && N % 64 == 0 && K % BK == 0 &&
         K % group_size == 0 && N > 0 && K >= BK * kDepth;
}

namespace {
// Into how many K ranges a launch of 64-row tiles is cut, and the padded K that goes with it: few tiles (fewer than half the
// CUs), K padded to whole unrolled iterations per range, every range at least two iterations long and begun before K ends.
// Of the splits that qualify, the one with the shortest k loop.  ks = 1: no split.
struct LdsPlan { uint32_t ks, Kx; };
LdsPlan lds_plan(uint32_t M, uint32_t N, uint32_t K, bool may_split) {
  LdsPlan best{1, padded_k(K)};
  const uint32_t tiles = ((M + 63) / 64) * (N / 64), real = K / BK, cus = (uint32_t)ctx().num_cus;
  if (!may_split || M > 128 || tiles * 2 > cus) return best;
  for (uint32_t ks = 2; ks <= 4; ++ks) {
    const uint32_t unit = ks * BK * kDepth, Kx = (K + unit - 1) / unit * unit, per = Kx / BK / ks;
    if (per < 2 * kDepth || (ks - 1) * per >= real || tiles * ks > 2 * cus) continue;
    if (per < best.Kx / BK / best.ks) best = LdsPlan{ks, Kx};
  }
  return best;
}
size_t relayout_bytes(uint32_t M, uint32_t Kx) { return ((size_t)((M + 15) / 16) * 16 * Kx * 2 + 255) / 256 * 256; }
}  // namespace

// The fragment-major activations; with N given (f16 multiplies), the partial sums of a K split behind them.
size_t qmm_workspace_bytes(uint32_t M, uint32_t K, uint32_t N) {
  const LdsPlan pl = lds_plan(M, N, K, N != 0);
  return relayout_bytes(M, pl.Kx) + (pl.ks > 1 ? (size_t)pl.ks * M * N * 4 : 0);
}

size_t qmm_grouped_workspace_bytes(uint32_t max_tiles, uint32_t K, uint32_t tile_rows) {
  return (size_t)max_tiles * tile_rows * padded_k(K) * 2;
}

// Grouped launch over row tiles of 64 or 128 rows of one expert each (see GroupedQmmArgs; one weight per launch, f16 output):
// what the routed block runs on where the register-weights grouped GEMM does not take the shape (dimensions in multiples
// of 64 that are no multiples of 128).  `workspace`: qmm_grouped_workspace_bytes(max_tiles, K, tile_rows) bytes.
int32_t launch_qmm_grouped(const GroupedQmmArgs& a, void* workspace, hipStream_t s) {
  if (!qmm_supported(a.N, a.K, a.group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "grouped qmm: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, a.bits, a.group_size);
  if (a.max_tiles == 0) return RMLX_OK;
  if (a.w1 != nullptr || a.out_f32 || (a.tile_rows != 64 && a.tile_rows != 128) || a.tile_tab == nullptr || a.n_tiles_dev == nullptr || workspace == nullptr)
    return fail(RMLX_RUNTIME_ERROR, "grouped qmm (LDS-staged): one weight, f16 output, tiles of 64 or 128 rows, a tile table and a workspace");
  if ((uint64_t)a.max_tiles * (a.N / 64) > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "grouped qmm: grid too large");
  const uint32_t Kx = padded_k(a.K);
  {
    const uint64_t units = (uint64_t)a.max_tiles * (a.tile_rows / 16) * (Kx / 32) * 64;
    uint64_t blocks = (units + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(relayout_grouped_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a.x, a.row_map, a.tile_tab, a.n_tiles_dev,
                       a.max_tiles, reinterpret_cast<u4*>(workspace), a.K, Kx, a.tile_rows / 16);
  }
  QmmParams p{a.w, a.s, a.b, reinterpret_cast<const uint16_t*>(workspace), static_cast<__half*>(a.out), a.max_tiles * a.tile_rows, a.N, a.K, Kx,
              a.group_size, a.tile_tab, a.n_tiles_dev, a.expert_stride_w, a.expert_stride_s};
  if (a.bits == 4) {
    if (a.group_size == 32) launch_grouped_t<4, 32>(p, a.max_tiles, a.tile_rows, s);
    else if (a.group_size == 128) launch_grouped_t<4, 128>(p, a.max_tiles, a.tile_rows, s);
    else launch_grouped_t<4, 64>(p, a.max_tiles, a.tile_rows, s);
  } else {
    if (a.group_size == 32) launch_grouped_t<8, 32>(p, a.max_tiles, a.tile_rows, s);
    else if (a.group_size == 128) launch_grouped_t<8, 128>(p, a.max_tiles, a.tile_rows, s);
    else launch_grouped_t<8, 64>(p, a.max_tiles, a.tile_rows, s);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_qmm(const QmmArgs& a, hipStream_t s) {
  if (!qmm_supported(a.N, a.K, a.group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "qmm: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, a.bits, a.group_size);
  if (a.bf16_mfma && a.group_size != 64) return fail(RMLX_INVALID_SHAPE, "qmm: the bf16 MFMA form takes group size 64");
  if (a.M == 0) return RMLX_OK;
  if (a.workspace == nullptr) return fail(RMLX_RUNTIME_ERROR, "qmm: missing activation workspace");
  const bool want_bf16 = a.bf16_mfma && a.bits == 8 && a.x_dtype == RMLX_DTYPE_BF16;
  const LdsPlan plan = lds_plan(a.M, a.N, a.K, a.workspace_has_partials && !want_bf16);
  const uint32_t Kx = plan.Kx, ks = plan.ks;
  {
    const uint64_t units = (uint64_t)((a.M + 15) / 16) * (Kx / 32) * 64;
    uint64_t blocks = (units + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(relayout_a_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a.x, a.x_dtype,
                       reinterpret_cast<u4*>(a.workspace), a.M, a.K, Kx, want_bf16 ? 1 : 0);
  }
  QmmParams p{a.w, a.s, a.b, reinterpret_cast<const uint16_t*>(a.workspace), a.out, a.M, a.N, a.K, Kx, a.group_size, nullptr, nullptr, 0, 0};
  if (ks > 1) {  // few tiles: the k loop in ks ranges, f32 partial sums behind the activations, one pass that adds them up
    p.ksplit = ks;
    p.partial = reinterpret_cast<float*>(static_cast<char*>(a.workspace) + relayout_bytes(a.M, Kx));
    const dim3 grid(((a.M + 63) / 64) * (a.N / 64), ks);
    const bool tail = Kx != a.K;
#define SPLIT_LAUNCH(BITSV, GSV)                                                                                                   \
  if (tail) hipLaunchKernelGGL((qmm_kernel<64, 64, BITSV, false, true, GSV, false, true>), grid, dim3(kThreads), 0, s, p);         \
  else hipLaunchKernelGGL((qmm_kernel<64, 64, BITSV, false, false, GSV, false, true>), grid, dim3(kThreads), 0, s, p);
    if (a.bits == 4) {
      if (a.group_size == 32) { SPLIT_LAUNCH(4, 32) } else if (a.group_size == 128) { SPLIT_LAUNCH(4, 128) } else { SPLIT_LAUNCH(4, 64) }
    } else {
      if (a.group_size == 32) { SPLIT_LAUNCH(8, 32) } else if (a.group_size == 128) { SPLIT_LAUNCH(8, 128) } else { SPLIT_LAUNCH(8, 64) }
    }
#undef SPLIT_LAUNCH
    const uint64_t quads = (uint64_t)a.M * a.N / 4;
    hipLaunchKernelGGL(splitk_sum_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, p.partial, a.out, quads, ks);
    RMLX_HIP_CHECK(hipGetLastError());
    return RMLX_OK;
  }
  // 128-row tiles only when they still give (most of) the CUs a workgroup
  const uint32_t tiles128 = ((a.M + 127) / 128) * (a.N / 64);
  const bool big = a.M > 64 && tiles128 * 4 >= (uint32_t)ctx().num_cus * 3;
  if (a.bits == 4) {
    if (big) launch_t<128, 4, false>(p, s); else launch_t<64, 4, false>(p, s);
  } else if (want_bf16) {
    if (big) launch_t<128, 8, true>(p, s); else launch_t<64, 8, true>(p, s);
  } else {
    if (big) launch_t<128, 8, false>(p, s); else launch_t<64, 8, false>(p, s);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
