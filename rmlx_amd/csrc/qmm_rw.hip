// Quantized GEMM for gfx950 (prefill, M > 16) with the weights kept in registers.
//
// Replaces the reference's affine_qmm_nax_q4 / affine_qmm_steel4sg_splitk_q4 /
// affine_qmm_mma_q8 (crates/rmlx-core/src/ops/quantized.rs:3331-3565, 4572-4786, 5838-5971).
//
// Design (wave64, v_mfma_f32_16x16x32_f16, f32 accumulation, f16 output):
//   * Weights never touch LDS.  Lane (n = lane%16, g = lane/16) of a wave loads 16 bytes of
//     weight row n: the 32 (Q4) or 16 (Q8) values of its lane group inside a 128-wide k block.
//     Word j of that load is dequantized in registers straight into the MFMA operand of product
//     j of the block (exact magic-number int -> f16 conversion, then w = s*q + b in packed f16),
//     so product j multiplies a k set that is not a contiguous run; the activation operand is
//     laid out to match.  With group size 64 all values of a lane belong to one quantisation
//     group, so a lane needs a single (scale, bias) pair per load; the pairs of four iterations
//     come in one 16-byte load per weight row.
//   * The waves of a workgroup (4 or 8) split the N extent of the tile: every weight is loaded
//     and dequantized by exactly one wave.
//   * Activations are shared by the waves and go through LDS.  They are read from the row-major
//     [M,K] matrix (f16, or bf16 converted on the way) with coalesced 16-byte loads (16 lanes
//     per 256-byte row piece), permuted to
//     the slot order of the nibble unpacking and written to an xor-swizzled operand layout, so
//     both the writes and the 16-byte operand reads are bank-conflict free.  No prepass, no
//     workspace.
//   * Register rings keep global loads four 128-wide k blocks ahead (weights) and the LDS copy two
//     blocks ahead (4-stage LDS ring); one barrier per block.  Every step of a block (the MFMAs
//     of one weight fragment and product) carries its share of the block's LDS writes and global
//     loads and unpacks the next weight operand, so memory instructions, VALU work and MFMAs
//     alternate in the instruction stream instead of arriving in bursts.
//   * Workgroup ids are remapped so that the tiles sharing a weight panel run on one XCD (one L2).
#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

struct __attribute__((packed, aligned(4))) U4Tail { uint32_t v[4]; };  // a 16-byte load from a 4-byte aligned address

constexpr int kBlockK = 128;  // k extent of one main-loop iteration
constexpr int kStages = 4;
constexpr int kUnroll = 4;   // main-loop unrolling = depth of the weight register ring

struct RwParams {
  const uint32_t* w; const __half* s; const __half* b;
  const __half* x;   // [M,K] row-major, f16 (or bf16 bits when XBF16)
  __half* out;
  uint32_t M, N, K;
  uint32_t tiles_m, tiles_n;
  int32_t epi_kind, epi_dtype;  // fused store epilogue: EPI_RESIDUAL / EPI_SWIGLU with an [M,N] f16 / f32 operand
  const void* epi;
  // split-K: grid.y = ksplit workgroups per tile, each over K / ksplit; f32 partial sums [ksplit, M, N]
  // are added up (and the epilogue applied) by splitk_reduce_kernel
  uint32_t ksplit;
  float* partial;
  // grouped launches (one expert per row tile): table of (expert, first row, rows) per row tile and its
  // length on the device, optional gather of the activation rows, expert strides in u32 words / f16
  // elements, the second weight of a gate/up pair (fragment 1 of every wave), f32 output
  const uint32_t* tile_tab; const uint32_t* n_tiles; const uint32_t* row_map;
  uint64_t estride_w, estride_s;
  const uint32_t* w1; const __half* s1; const __half* b1;
  int32_t out_f32;
};

__device__ __forceinline__ uint32_t h2bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// 8 Q4 values of one word -> 8 f16 weights in slot order (k0,k4,k1,k5,k2,k6,k3,k7), w = s*q + b.
// The int -> f16 conversion is exact: (w & 0x000F000F) | 0x64006400 is the pair (1024+q0, 1024+q4),
// (w & 0x00F000F0) | 0x54005400 is (64+q1, 64+q5); the offsets are subtracted before scaling.
struct DqConst { uint32_t m0, m1, k0, k1; };
__device__ __forceinline__ h8 dequant_q4_word(uint32_t w, h2 s2, h2 b2, const DqConst& c) {
  const uint32_t t = w >> 8;
  const h2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f}, k64 = {(_Float16)64.0f, (_Float16)64.0f};
  const h2 p0 = __builtin_bit_cast(h2, (w & c.m0) | c.k0) - k1024;
  const h2 p1 = __builtin_bit_cast(h2, (w & c.m1) | c.k1) - k64;
  const h2 p2 = __builtin_bit_cast(h2, (t & c.m0) | c.k0) - k1024;
  const h2 p3 = __builtin_bit_cast(h2, (t & c.m1) | c.k1) - k64;
  u4 o;
  o.x = h2bits(p0 * s2 + b2);
  o.y = h2bits(p1 * s2 + b2);
  o.z = h2bits(p2 * s2 + b2);
  o.w = h2bits(p3 * s2 + b2);
  return __builtin_bit_cast(h8, o);
}

// 8 Q8 values of two words -> 8 f16 weights in natural order.
__device__ __forceinline__ h8 dequant_q8_pair(uint32_t w0, uint32_t w1, h2 s2, h2 b2) {
  const h2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  const h2 p0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)) - k1024;
  const h2 p1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)) - k1024;
  const h2 p2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)) - k1024;
  const h2 p3 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)) - k1024;
  u4 o;
  o.x = h2bits(p0 * s2 + b2);
  o.y = h2bits(p1 * s2 + b2);
  o.z = h2bits(p2 * s2 + b2);
  o.w = h2bits(p3 * s2 + b2);
  return __builtin_bit_cast(h8, o);
}

// MF = 16-row activation fragments per workgroup (tile rows = 16*MF), NF = 16-row weight fragments
// per wave (tile columns = 64*NF), BITS = 4 or 8.
// GS = quantisation group size (32, 64 or 128): it only decides which (scale, bias) pair a lane uses.
// MODE 0: one weight, row tiles of one [M,K] matrix.  MODE 1: grouped -- row tile t of the grid takes its
// expert and its rows from the tile table (rows of different experts never share a tile); workgroups past
// the table's length leave at once.  MODE 2: grouped gate/up pair -- fragment 0 of a wave multiplies gate
// rows, fragment 1 the same rows of the up weight (NF == 2), and the store writes silu(gate) * up.
// TAIL (group sizes 32 and 64): K is a multiple of 128 but not of 512.  The last unrolled round of the loop then holds iterations past
// K: their activation chunks are written to LDS as zeros, weight loads repeat the last block, and the scales and biases
// of the last round come from loads that end with the row.
template <int MF, int NF, int BITS, int NW, bool XBF16, int GS, int MODE, bool TAIL = false>
__device__ __forceinline__ void qmm_rw_body(const RwParams p) {  // by value: a reference makes every store a possible change of p
  static_assert(MODE != 2 || NF == 2, "a gate/up pair takes two weight fragments per wave");
  static_assert(!TAIL || GS != 128, "the tail form is built for group sizes 32 and 64");
  constexpr int kSbWords = 4 * (kBlockK / GS) / 2;  // 32-bit words of scales of one row and four iterations: 8 / 4 / 2
  constexpr int kSbVecs = (kSbWords + 3) / 4;       // 16-byte registers holding them
  constexpr int kThreads = 64 * NW;
  constexpr int AL = MF * 256 / kThreads;      // 16-byte activation loads per thread and chunk
  static_assert(AL * kThreads == MF * 256, "chunk must divide over the workgroup");
  constexpr int kChunk = MF * 4 * 64;          // 16-byte units of one activation chunk
  constexpr int WL = BITS == 4 ? 1 : 2;        // 16-byte weight loads per lane, fragment and iteration
  __shared__ u4 a_lds[kStages * kChunk];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;

  // Workgroup -> tile.  Consecutive workgroup ids go round-robin over the 8 XCDs (one L2 each), so
  // XCD x = id % 8 runs the ids congruent to x.  Give every XCD a compact block of tiles, half of
  // the row tiles x a quarter of the column tiles when those divide, so that what its L2 has to
  // fetch (its activation rows + its weight panels) is smallest; else whole weight panels per XCD.
  uint32_t wg = blockIdx.x, mt = 0, nt;
  uint32_t row_lo = 0, row_hi = 0;  // rows of the activation / output matrix this tile covers: [row_lo, row_hi)
  const uint32_t* wbase[2] = {p.w, p.w1};
  const __half* sbase[2] = {p.s, p.s1};
  const __half* bbase[2] = {p.b, p.b1};
  const uint32_t total = p.tiles_m * p.tiles_n;
  if (MODE != 0) {
    // Consecutive workgroup ids go round-robin over the 8 XCDs.  XCD x takes a contiguous run of the table
    // (an eighth of its row tiles) and walks it row tile by row tile, column tiles inside: the workgroups that
    // share a row tile's activations, and the consecutive row tiles of one expert that share its weight panels,
    // run on one XCD at about the same time, so each is fetched into one L2 once.
    const uint32_t n_t = *p.n_tiles, run = (n_t + 7) / 8;
    const uint32_t xcd = wg % 8, local = wg / 8, tl = local / p.tiles_n;
    nt = local % p.tiles_n;
    const uint32_t te = xcd * run + tl;
    if (tl >= run || te >= n_t) return;
    const uint32_t expert = p.tile_tab[3 * te];
    row_lo = p.tile_tab[3 * te + 1];
    const uint32_t cnt = p.tile_tab[3 * te + 2];
    row_hi = row_lo + (cnt & 0x7FFFFFFFu);
    if (MODE == 1 && (cnt >> 31)) {  // rows whose expert index is out of range: zeros
      constexpr uint32_t cols = NW * 16 * NF;
      for (uint32_t i = threadIdx.x; i < (row_hi - row_lo) * cols; i += 64 * NW) {
        const uint64_t o = (uint64_t)(row_lo + i / cols) * p.N + nt * cols + i % cols;
        if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = 0.f;
        else p.out[o] = __float2half(0.f);
      }
      return;
    }
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      wbase[d] += (uint64_t)expert * p.estride_w;
      sbase[d] += (uint64_t)expert * p.estride_s;
      bbase[d] += (uint64_t)expert * p.estride_s;
    }
  } else if (total % 8 == 0 && p.tiles_m % 2 == 0 && p.tiles_n % 4 == 0) {
    const uint32_t xcd = wg % 8, local = wg / 8, bm = p.tiles_m / 2, bn = p.tiles_n / 4;
    mt = (xcd % 2) * bm + local % bm;
    nt = (xcd / 2) * bn + local / bm;
  } else {
    if (total % 8 == 0) wg = (wg % 8) * (total / 8) + wg / 8;
    mt = wg % p.tiles_m;
    nt = wg / p.tiles_m;
  }
  if (MODE == 0) { row_lo = mt * (16 * MF); row_hi = p.M; }

  const uint32_t K = p.K, G = K / GS;
  const uint32_t S = K / kBlockK / p.ksplit;   // iterations of this workgroup
  const uint32_t it_first = blockIdx.y * S;    // its first 128-wide k block
  const uint32_t row_base = MODE == 2 ? nt * (NW * 16) + wave * 16 + n : nt * (NW * 16 * NF) + wave * (16 * NF) + n;

  const u4* wptr[NF];
  const __half* sptr[NF];
  const __half* bptr[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const uint64_t row = MODE == 2 ? row_base : row_base + f * 16;
    const int d = MODE == 2 ? f : 0;
    wptr[f] = reinterpret_cast<const u4*>(wbase[d] + row * (K * BITS / 32)) + g + (uint64_t)it_first * (4 * WL);
    sptr[f] = sbase[d] + row * G + it_first * (kBlockK / GS);
    bptr[f] = bbase[d] + row * G + it_first * (kBlockK / GS);
  }
  // Activation chunk of an iteration: 16*MF rows x 128 k = 16 sixteen-byte segments per row.  Unit
  // q*kThreads + tid -> (row, segment): 16 consecutive lanes read one row's 256 contiguous bytes.
  // Segment seg holds k offsets 8*seg..8*seg+7, i.e. product j / lane group gq of the operand
  // layout; inside LDS the 16-byte slot of (fragment i, product j, lane gq*16 + r) is
  // (i*4 + j)*64 + gq*16 + (r ^ (4*j + gq)): the xor spreads the 16 lanes of a row over all banks
  // on the write and stays a permutation of a product's 64 slots on the read.
  const __half* xsrc[AL];
  uint32_t lds_w[AL];
#pragma unroll
  for (int q = 0; q < AL; ++q) {
    const uint32_t unit = q * kThreads + tid, r = unit >> 4, seg = unit & 15;
    uint32_t row = row_lo + r;
    if (row >= row_hi) row = row_hi - 1;  // rows past the end are computed on stale data and never stored
    if (MODE != 0 && p.row_map != nullptr) row = p.row_map[row];
    xsrc[q] = p.x + (uint64_t)row * K + seg * 8 + (uint64_t)it_first * kBlockK;
    const uint32_t j = BITS == 4 ? (seg & 3) : (2 * (seg >> 3) + (seg & 1));
    const uint32_t gq = BITS == 4 ? (seg >> 2) : ((seg >> 1) & 3);
    lds_w[q] = ((r >> 4) * 4 + j) * 64 + gq * 16 + ((r & 15) ^ (4 * j + gq));
  }
  uint32_t lds_r[4];  // read slot of this lane for product j (fragment i adds 256)
#pragma unroll
  for (int j = 0; j < 4; ++j) lds_r[j] = j * 64 + g * 16 + (n ^ (4 * j + g));

  f4 acc[MF][NF];
#pragma unroll
  for (int i = 0; i < MF; ++i)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[i][f] = (f4){0.f, 0.f, 0.f, 0.f};

  // Register rings: activation chunks travel global -> registers -> LDS (two sets: a chunk is loaded
  // three iterations before it is used and written to LDS one iteration before); weights are
  // loaded four iterations ahead (set = iteration % 4); the scales and biases of four iterations
  // (eight groups = 16 bytes per row) come in one load per fragment, one block of four ahead.
  // The loop is unrolled by four so that every ring index is a compile-time constant.
  u4 ra[2][AL];
  u4 wq[kUnroll][NF][WL];
  u4 s_cur[NF][kSbVecs], b_cur[NF][kSbVecs], s_nxt[NF][kSbVecs], b_nxt[NF][kSbVecs];

  // Q4: halves (k0..k7) -> slots (k0,k4,k1,k5,k2,k6,k3,k7), the order the nibble unpacking produces
  auto to_slot_order = [&](u4 v) {
    if (XBF16) {  // bf16 activations: to f16 through f32 (exact for normal-range values), round to nearest even
      uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
        w[e] = h2bits((h2){(_Float16)lo, (_Float16)hi});
      }
      v = (u4){w[0], w[1], w[2], w[3]};
    }
    if (BITS != 4) return v;
    u4 o;
    o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
    o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
    o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
    o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    return o;
  };
  auto load_a = [&](uint32_t it, u4 (&dst)[AL]) {
#pragma unroll
    for (int q = 0; q < AL; ++q) {
      dst[q] = *reinterpret_cast<const u4*>(xsrc[q] + (uint64_t)it * kBlockK);
    }
  };
  auto store_a = [&](uint32_t stage, const u4 (&src)[AL]) {
#pragma unroll
    for (int q = 0; q < AL; ++q) a_lds[stage * kChunk + lds_w[q]] = to_slot_order(src[q]);
  };
  auto load_sb = [&](uint32_t blk, u4 (&ds)[NF][kSbVecs], u4 (&db)[NF][kSbVecs]) {
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      if (TAIL) {
        // kWordsPerIt words per iteration (one at group size 64, two at 32), S * kWordsPerIt >= 4 * kWordsPerIt words per
        // row.  The 16-byte loads of a round that would run past the row's end start early enough to end with the row
        // (4-byte aligned: enough for the hardware), and the words move down to their places; what then sits behind
        // the row's last word belongs to iterations past K.
        // (the move happens late in the round before, see settle_sb: done here it would wait for the load at once)
        constexpr uint32_t kWordsPerIt = GS == 128 ? 1 : kBlockK / GS / 2, kRound = 4 * kWordsPerIt;  // (no tail form at group size 128)
        const uint32_t want = blk * kRound, wo = want < S * kWordsPerIt - kRound ? want : S * kWordsPerIt - kRound;  // (wave-uniform)
#pragma unroll
        for (int v = 0; v < kSbVecs; ++v) {
          const U4Tail sv = *reinterpret_cast<const U4Tail*>(reinterpret_cast<const uint32_t*>(sptr[f]) + wo + 4 * v);
          const U4Tail bv = *reinterpret_cast<const U4Tail*>(reinterpret_cast<const uint32_t*>(bptr[f]) + wo + 4 * v);
          ds[f][v] = (u4){sv.v[0], sv.v[1], sv.v[2], sv.v[3]};
          db[f][v] = (u4){bv.v[0], bv.v[1], bv.v[2], bv.v[3]};
        }
      } else if (GS == 128) {  // 4 groups = 8 bytes per row and four iterations
        const u2 sv = reinterpret_cast<const u2*>(sptr[f])[blk], bv = reinterpret_cast<const u2*>(bptr[f])[blk];
        ds[f][0] = (u4){sv.x, sv.y, 0u, 0u};
        db[f][0] = (u4){bv.x, bv.y, 0u, 0u};
      } else {
#pragma unroll
        for (int v = 0; v < kSbVecs; ++v) {
          ds[f][v] = reinterpret_cast<const u4*>(sptr[f])[blk * kSbVecs + v];
          db[f][v] = reinterpret_cast<const u4*>(bptr[f])[blk * kSbVecs + v];
        }
      }
    }
  };
  // tail form: the words of round blk, as loaded by load_sb, move down to their places (by whole iterations)
  auto settle_sb = [&](uint32_t blk, u4 (&ds)[NF][kSbVecs], u4 (&db)[NF][kSbVecs]) {
    constexpr uint32_t kWordsPerIt = GS == 128 ? 1 : kBlockK / GS / 2, kRound = 4 * kWordsPerIt;  // (no tail form at group size 128)
    const uint32_t want = blk * kRound, wo = want < S * kWordsPerIt - kRound ? want : S * kWordsPerIt - kRound;
    const uint32_t its = (want - wo) / kWordsPerIt;  // (wave-uniform: 0 .. 3 iterations)
    auto moved = [&](u4 (&v)[kSbVecs]) {
      uint32_t in[kRound], out[kRound];
#pragma unroll
      for (int c = 0; c < (int)kRound; ++c) in[c] = c % 4 == 0 ? v[c / 4].x : (c % 4 == 1 ? v[c / 4].y : (c % 4 == 2 ? v[c / 4].z : v[c / 4].w));
#pragma unroll
      for (int c = 0; c < (int)kRound; ++c) {
        constexpr int last = (int)kRound - 1, k = (int)kWordsPerIt;
        const uint32_t a1 = in[c + k < last ? c + k : last], a2 = in[c + 2 * k < last ? c + 2 * k : last], a3 = in[c + 3 * k < last ? c + 3 * k : last];
        out[c] = its == 0 ? in[c] : (its == 1 ? a1 : (its == 2 ? a2 : a3));
      }
#pragma unroll
      for (int q = 0; q < kSbVecs; ++q) v[q] = (u4){out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
    };
#pragma unroll
    for (int f = 0; f < NF; ++f) { moved(ds[f]); moved(db[f]); }
  };
  auto load_w = [&](uint32_t it, u4 (&dst)[NF][WL]) {
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int h = 0; h < WL; ++h) {
        dst[f][h] = wptr[f][(uint64_t)it * (4 * WL) + h * 4];
      }
  };
  const uint32_t last = S - 1, last_blk = (S + kUnroll - 1) / kUnroll - 1;
  auto clampi = [&](uint32_t it) { return it < last ? it : last; };

  // Constants of the unpacking kept in registers so that and+or is one instruction.
  DqConst dq;
  dq.m0 = 0x000F000Fu; dq.m1 = 0x00F000F0u; dq.k0 = 0x64006400u; dq.k1 = 0x54005400u;
  asm volatile("" : "+s"(dq.m0), "+s"(dq.m1), "+v"(dq.k0), "+v"(dq.k1));
  // Which f16 of a scale word a lane uses.  Half h of a row's scale block belongs to iteration h / GPB
  // and group h % GPB of its 128-wide k block (GPB = 128 / GS groups per block); a lane's k values lie
  // in group (32g) / GS (Q4) or (64h + 16g) / GS (Q8, load h).
  constexpr uint32_t kSelLo = 0x01000100u, kSelHi = 0x03020302u;
  const uint32_t sel_g1 = (g >> 1) ? kSelHi : kSelLo, sel_g0 = (g & 1) ? kSelHi : kSelLo;

  // scale / bias operand pairs of iteration slot u of the current block (u == kUnroll: first
  // iteration of the next block)
  auto word_of = [](const u4& v, int c) { return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w)); };
  auto scale_pair = [&](int u, int f, int h, h2& s2, h2& b2) {
    const u4 (&sv)[kSbVecs] = u < kUnroll ? s_cur[f] : s_nxt[f];
    const u4 (&bv)[kSbVecs] = u < kUnroll ? b_cur[f] : b_nxt[f];
    const int w = u % kUnroll;
    uint32_t sw, bw, sel;
    if (GS == 64) {         // word w = (group 0, group 1) of iteration w
      sw = word_of(sv[0], w); bw = word_of(bv[0], w);
      sel = BITS == 4 ? sel_g1 : (h ? kSelHi : kSelLo);
    } else if (GS == 128) {  // half w = the one group of iteration w
      sw = word_of(sv[0], w >> 1); bw = word_of(bv[0], w >> 1);
      sel = (w & 1) ? kSelHi : kSelLo;
    } else if (BITS == 4) {  // GS 32: half 4w + g
      const int c = 2 * (w & 1);
      sw = (g >> 1) ? word_of(sv[w >> 1], c + 1) : word_of(sv[w >> 1], c);
      bw = (g >> 1) ? word_of(bv[w >> 1], c + 1) : word_of(bv[w >> 1], c);
      sel = sel_g0;
    } else {                 // GS 32, Q8: half 4w + 2h + g/2
      sw = word_of(sv[w >> 1], 2 * (w & 1) + h); bw = word_of(bv[w >> 1], 2 * (w & 1) + h);
      sel = sel_g1;
    }
    s2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(sw, sw, sel));
    b2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(bw, bw, sel));
  };
  // weight operand of step (j, f) of iteration slot u (u == kUnroll: slot 0 of the next block)
  auto weight_operand = [&](int u, int j, int f) -> h8 {
    h2 s2, b2;
    if (BITS == 4) {
      const u4 q = wq[u % kUnroll][f][0];
      const uint32_t word = j == 0 ? q.x : (j == 1 ? q.y : (j == 2 ? q.z : q.w));
      scale_pair(u, f, 0, s2, b2);
      return dequant_q4_word(word, s2, b2, dq);
    } else {
      constexpr int hmax = WL - 1;
      const int h = (j >> 1) < hmax ? (j >> 1) : hmax;
      const u4 q = wq[u % kUnroll][f][h];
      const uint32_t w0 = (j & 1) ? q.z : q.x, w1 = (j & 1) ? q.w : q.y;
      scale_pair(u, f, h, s2, b2);
      return dequant_q8_pair(w0, w1, s2, b2);
    }
  };

  // ---- prologue: chunks 0 and 1 go to LDS, chunks 2 and 3 wait in the register sets ---------------
  load_a(0, ra[0]);
  load_a(clampi(1), ra[1]);
  load_sb(0, s_cur, b_cur);
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) load_w(clampi(u), wq[u]);
  store_a(0, ra[0]);
  store_a(1, ra[1]);
  load_a(clampi(2), ra[0]);
  load_a(clampi(3), ra[1]);
  __syncthreads();

  constexpr int NS = 4 * NF;  // steps of an iteration: (product j, fragment f), MF MFMAs each
  h8 a_cur[MF], a_nxt[MF];
#pragma unroll
  for (int i = 0; i < MF; ++i) a_cur[i] = __builtin_bit_cast(h8, a_lds[i * 256 + lds_r[0]]);
  h8 wv_cur = weight_operand(0, 0, 0), wv_nxt;

  for (uint32_t it0 = 0; it0 < S; it0 += kUnroll) {
    const uint32_t blk = it0 / kUnroll;
    load_sb(blk < last_blk ? blk + 1 : last_blk, s_nxt, b_nxt);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const uint32_t it = it0 + u;
      // (the next round's scales and biases were requested three iterations ago; its first weight operand is unpacked in
      // this iteration's last step)
      if (TAIL && u == kUnroll - 1) settle_sb(blk < last_blk ? blk + 1 : last_blk, s_nxt, b_nxt);
      const u4* a_stage = a_lds + (it % kStages) * kChunk;
      const u4* a_stage_next = a_lds + ((it + 1) % kStages) * kChunk;
      u4* a_stage_write = a_lds + ((it + 2) % kStages) * kChunk;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int j = s / NF, f = s % NF;
        // operands of the next product (of the next iteration after the last one: that chunk was
        // written two iterations ago, so it is visible before this iteration's barrier)
        if (f == 0) {
#pragma unroll
          for (int i = 0; i < MF; ++i)
            a_nxt[i] = __builtin_bit_cast(h8, j < 3 ? a_stage[i * 256 + lds_r[j < 3 ? j + 1 : 0]] : a_stage_next[i * 256 + lds_r[0]]);
        }
        // this step's share of the ring traffic: LDS writes of chunk it+2 in the first half, the
        // global loads of chunk it+4 into the same registers in the second half, weights last
#pragma unroll
        for (int q = 0; q < AL; ++q) {
          if (s == q * NS / (2 * AL)) {
            u4 av = to_slot_order(ra[u % 2][q]);
            if (TAIL && it + 2 >= S) av = (u4){0u, 0u, 0u, 0u};  // (a chunk past K: these iterations add nothing)
            a_stage_write[lds_w[q]] = av;
          }
          if (s == NS / 2 + q * NS / (2 * AL)) {
            ra[u % 2][q] = *reinterpret_cast<const u4*>(xsrc[q] + (uint64_t)clampi(it + 4) * kBlockK);
          }
        }
        // next weight operand (the one of the first step of the next iteration after the last step)
        if (s + 1 < NS) wv_nxt = weight_operand(u, (s + 1) / NF, (s + 1) % NF);
        else wv_nxt = weight_operand(u + 1, 0, 0);
#pragma unroll
        for (int i = 0; i < MF; ++i)
          acc[i][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv_cur, a_cur[i], acc[i][f], 0, 0, 0);
        if (s == NS - 1) load_w(clampi(it + kUnroll), wq[u]);  // every word of wq[u] has been unpacked
        if (f == NF - 1) {
#pragma unroll
          for (int i = 0; i < MF; ++i) a_cur[i] = a_nxt[i];
        }
        wv_cur = wv_nxt;
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
    }
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int v = 0; v < kSbVecs; ++v) { s_cur[f][v] = s_nxt[f][v]; b_cur[f][v] = b_nxt[f][v]; }
  }

  // ---- epilogue: lane holds row m = lane%16 of fragment i, columns 4g..4g+3 of fragment f ------
#pragma unroll
  for (int i = 0; i < MF; ++i) {
    const uint32_t m = row_lo + i * 16 + n;
    if (m < row_hi) {
      if (MODE == 2) {  // h = silu(gate) * up in f32, one rounding; p.N = columns of h
        const uint32_t col = nt * (NW * 16) + wave * 16 + 4 * g;
        f4 v;
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = acc[i][0][q] / (1.0f + __expf(-acc[i][0][q])) * acc[i][NF - 1][q];
        const h2 lo = {(_Float16)v[0], (_Float16)v[1]};
        const h2 hi = {(_Float16)v[2], (_Float16)v[3]};
        *reinterpret_cast<u2*>(p.out + (uint64_t)m * p.N + col) = (u2){h2bits(lo), h2bits(hi)};
        continue;
      }
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        const uint32_t col = nt * (NW * 16 * NF) + wave * (16 * NF) + f * 16 + 4 * g;
        f4 v = acc[i][f];
        if (MODE == 0 && p.ksplit > 1) {
          *reinterpret_cast<f4*>(p.partial + ((uint64_t)blockIdx.y * p.M + m) * p.N + col) = v;
          continue;
        }
        if (MODE == 1 && p.out_f32) {
          *reinterpret_cast<f4*>(reinterpret_cast<float*>(p.out) + (uint64_t)m * p.N + col) = v;
          continue;
        }
        if (p.epi_kind != EPI_NONE) {  // residual add / SwiGLU gate in f32, one rounding (quantized.rs:3206-3246)
          f4 e;
          if (p.epi_dtype == RMLX_DTYPE_F32) {
            e = *reinterpret_cast<const f4*>(static_cast<const float*>(p.epi) + (uint64_t)m * p.N + col);
          } else {
            const u2 eb = *reinterpret_cast<const u2*>(static_cast<const __half*>(p.epi) + (uint64_t)m * p.N + col);
            // (copy the elements to scalars first: __builtin_bit_cast applied to a vector element
            // expression reads element 0 with this compiler)
            const uint32_t ex = eb.x, ey = eb.y;
            const h2 e0 = __builtin_bit_cast(h2, ex), e1 = __builtin_bit_cast(h2, ey);
            e = (f4){(float)e0[0], (float)e0[1], (float)e1[0], (float)e1[1]};
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = p.epi_kind == EPI_RESIDUAL ? v[q] + e[q] : e[q] / (1.0f + __expf(-e[q])) * v[q];
        }
        const h2 lo = {(_Float16)v[0], (_Float16)v[1]};
        const h2 hi = {(_Float16)v[2], (_Float16)v[3]};
        *reinterpret_cast<u2*>(p.out + (uint64_t)m * p.N + col) = (u2){h2bits(lo), h2bits(hi)};
      }
    }
  }
}

template <int MF, int NF, int BITS, int NW, bool XBF16, int GS, bool TAIL>
__global__ __launch_bounds__(64 * NW) void qmm_rw_kernel(RwParams p) {
  qmm_rw_body<MF, NF, BITS, NW, XBF16, GS, 0, TAIL>(p);
}

// DUAL: gate/up pair with the SwiGLU store (see MODE 2 above)
template <int MF, int NF, int BITS, int NW, bool DUAL, int GS = 64, bool TAIL = false>
__global__ __launch_bounds__(64 * NW) void qmm_rw_grouped_kernel(RwParams p) {
  qmm_rw_body<MF, NF, BITS, NW, false, GS, DUAL ? 2 : 1, TAIL>(p);
}

// out[m, c..c+3] = epilogue(sum over the ksplit partial sums, in split order); one thread per four columns
__global__ __launch_bounds__(256) void splitk_reduce_kernel(RwParams p) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4, total = (size_t)p.M * p.N;
  if (i >= total) return;
  f4 v = *reinterpret_cast<const f4*>(p.partial + i);
  for (uint32_t z = 1; z < p.ksplit; ++z) v += *reinterpret_cast<const f4*>(p.partial + z * total + i);
  if (p.epi_kind != EPI_NONE) {
    f4 e;
    if (p.epi_dtype == RMLX_DTYPE_F32) {
      e = *reinterpret_cast<const f4*>(static_cast<const float*>(p.epi) + i);
    } else {
      const u2 eb = *reinterpret_cast<const u2*>(static_cast<const __half*>(p.epi) + i);
      const uint32_t ex = eb.x, ey = eb.y;
      const h2 e0 = __builtin_bit_cast(h2, ex), e1 = __builtin_bit_cast(h2, ey);
      e = (f4){(float)e0[0], (float)e0[1], (float)e1[0], (float)e1[1]};
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = p.epi_kind == EPI_RESIDUAL ? v[q] + e[q] : e[q] / (1.0f + __expf(-e[q])) * v[q];
  }
  const h2 lo = {(_Float16)v[0], (_Float16)v[1]};
  const h2 hi = {(_Float16)v[2], (_Float16)v[3]};
  *reinterpret_cast<u2*>(p.out + i) = (u2){h2bits(lo), h2bits(hi)};
}

template <int MF, int NF, int BITS, int NW, int GS = 64>
void launch_rw(RwParams p, bool x_bf16, hipStream_t s) {
  p.tiles_m = (p.M + 16 * MF - 1) / (16 * MF);
  p.tiles_n = p.N / (NW * 16 * NF);
  const dim3 grid(p.tiles_m * p.tiles_n, p.ksplit), block(64 * NW);
  const bool tail = (p.K / kBlockK / p.ksplit) % kUnroll != 0;  // (group sizes 32 and 64 only: checked by qmm_rw_supported)
  constexpr int kTailGs = GS == 128 ? 64 : GS;
  if (GS != 128 && tail) {
    if (x_bf16) hipLaunchKernelGGL((qmm_rw_kernel<MF, NF, BITS, NW, true, kTailGs, true>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((qmm_rw_kernel<MF, NF, BITS, NW, false, kTailGs, true>), grid, block, 0, s, p);
  } else {
    if (x_bf16) hipLaunchKernelGGL((qmm_rw_kernel<MF, NF, BITS, NW, true, GS, false>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((qmm_rw_kernel<MF, NF, BITS, NW, false, GS, false>), grid, block, 0, s, p);
  }
}

}  // namespace

bool qmm_rw_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  // (group sizes 32 and 64 also take K in whole 128-wide blocks, at least four: the tail form)
  return (group_size == 32 || group_size == 64 || group_size == 128) && (bits == 4 || bits == 8) && N > 0 && K > 0 && N % 64 == 0 &&
         (K % (kBlockK * kUnroll) == 0 || (group_size != 128 && K % kBlockK == 0 && K >= 4 * kBlockK));
}


namespace {
struct RwPlan { int mf, nf, nw; uint32_t ksplit; };

// Tile choice {MF, NF, NW} (tile rows 16*MF, tile columns 16*NF*NW): least estimated time =
// rounds of workgroups over the CUs x work per tile / measured relative efficiency of the tile.
// Split-K: a launch that leaves SIMDs empty is bound by the length of its k loop (every 128-wide k block
// is a dependent chain of loads, LDS traffic and a barrier); splitting K over 2 or 4 workgroups per tile
// shortens the loop and fills the SIMDs, at the price of a small reduction kernel.  It stops paying as
// soon as every SIMD has a wave: the unpacking keeps the SIMDs busy, so more waves only take turns.
RwPlan plan_rw(uint32_t M, uint32_t N, uint32_t K, uint32_t group_size) {
  const uint32_t cus = (uint32_t)ctx().num_cus;
  static const struct { int mf, nf, nw; float eff; } cand[] = {
      {8, 1, 8, 1.01f}, {4, 2, 8, 1.0f}, {4, 1, 8, 0.93f}, {4, 2, 4, 0.9f}, {2, 2, 4, 0.7f}, {2, 1, 4, 0.55f}, {2, 1, 8, 0.45f}};
  RwPlan r{2, 1, 4, 1};
  float best = 0.f;
  uint32_t best_wgs = 0;
  for (const auto& c : cand) {
    const uint32_t bn = 16 * c.nf * c.nw;
    if (N % bn != 0) continue;
    // group sizes 32 / 128 are built for two tiles only (64 x 128 and 32 x 64)
    if (group_size != 64 && !((c.mf == 4 && c.nf == 1 && c.nw == 8) || (c.mf == 2 && c.nf == 1 && c.nw == 4))) continue;
    const uint32_t wgs = ((M + 16 * c.mf - 1) / (16 * c.mf)) * (N / bn);
    const float cost = (float)((wgs + cus - 1) / cus) * (float)(c.mf * c.nf * c.nw) / c.eff;
    if (best == 0.f || cost < best) { best = cost; r.mf = c.mf; r.nf = c.nf; r.nw = c.nw; best_wgs = wgs; }
  }
  // time ~ fixed + (k blocks per workgroup) x (block time, which grows once a SIMD holds more than one
  // wave: the unpacking keeps a SIMD busy) + the reduction pass; measured: 0.33 us per block, 3 us
  const float waves = (float)(best_wgs * (uint32_t)r.nw), simds = (float)(cus * 4), blocks = (float)(K / kBlockK);
  float best_t = 0.f;
  for (uint32_t ks = 1; ks <= 4; ks *= 2) {
    // (a split leaves whole unrolled rounds; where K itself has a tail, whole blocks, at least four)
    const uint32_t nb = K / kBlockK;
    if (K % (kBlockK * kUnroll) == 0 ? K % (ks * kBlockK * kUnroll) != 0 : (nb % ks != 0 || nb / ks < 4)) continue;
    const float load = waves * (float)ks / simds;
    const float t = blocks / (float)ks * 0.33f * (load > 1.f ? load : 1.f) + (ks > 1 ? 3.f : 0.f);
    if (best_t == 0.f || t < best_t - 0.5f) { best_t = t; r.ksplit = ks; }
  }
  return r;
}
}  // namespace

uint32_t qmm_rw_tile_work(uint32_t M, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  if (M == 0 || !qmm_rw_supported(N, K, group_size, bits)) return 0;
  const RwPlan r = plan_rw(M, N, K, group_size);
  return (uint32_t)(r.mf * r.nf * r.nw);
}

size_t qmm_rw_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  if (M == 0 || !qmm_rw_supported(N, K, group_size, bits)) return 0;
  const RwPlan r = plan_rw(M, N, K, group_size);
  return r.ksplit > 1 ? (size_t)r.ksplit * M * N * sizeof(float) : 0;
}

int32_t launch_qmm_rw(const QmmArgs& a, uint32_t group_size, hipStream_t s) {
  if (!qmm_rw_supported(a.N, a.K, group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "qmm: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, a.bits, group_size);
  if (a.M == 0) return RMLX_OK;
  if (a.x_dtype != RMLX_DTYPE_F16 && a.x_dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_RUNTIME_ERROR, "qmm: f32 activations must be cast to f16 first");
  const bool x_bf16 = a.x_dtype == RMLX_DTYPE_BF16;
  RwPlan plan = plan_rw(a.M, a.N, a.K, group_size);
  if (a.workspace == nullptr) plan.ksplit = 1;  // no room for partial sums: one workgroup per tile
  const int mf = plan.mf, nf = plan.nf, nw = plan.nw;
  RwParams p{};
  p.w = a.w; p.s = a.s; p.b = a.b;
  p.x = static_cast<const __half*>(a.x);
  p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K;
  p.epi_kind = a.epi_kind; p.epi = a.epi; p.epi_dtype = a.epi_dtype;
  p.ksplit = plan.ksplit; p.partial = static_cast<float*>(a.workspace);
#define RW_CASE(MFV, NFV, NWV)                                                                 \
  if (mf == MFV && nf == NFV && nw == NWV) {                                                   \
    if (a.bits == 4) launch_rw<MFV, NFV, 4, NWV>(p, x_bf16, s); else launch_rw<MFV, NFV, 8, NWV>(p, x_bf16, s); \
  }
#define RW_CASE_GS(MFV, NFV, NWV, GSV)                                                         \
  if (mf == MFV && nf == NFV && nw == NWV && group_size == GSV) {                              \
    if (a.bits == 4) launch_rw<MFV, NFV, 4, NWV, GSV>(p, x_bf16, s); else launch_rw<MFV, NFV, 8, NWV, GSV>(p, x_bf16, s); \
  }
  if (group_size == 64) {
    RW_CASE(4, 2, 8) RW_CASE(4, 1, 8) RW_CASE(2, 1, 8) RW_CASE(2, 1, 4) RW_CASE(4, 2, 4) RW_CASE(2, 2, 4)
    RW_CASE(8, 1, 8)
  } else {
    RW_CASE_GS(4, 1, 8, 32) RW_CASE_GS(2, 1, 4, 32) RW_CASE_GS(4, 1, 8, 128) RW_CASE_GS(2, 1, 4, 128)
  }
#undef RW_CASE_GS
#undef RW_CASE
  RMLX_HIP_CHECK(hipGetLastError());
  if (p.ksplit > 1) {
    const size_t quads = (size_t)p.M * p.N / 4;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, p);
    RMLX_HIP_CHECK(hipGetLastError());
  }
  return RMLX_OK;
}

bool qmm_rw_grouped_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  // (group sizes 32 and 64 also take K in whole 128-wide blocks, at least four: the tail form)
  return (group_size == 32 || group_size == 64 || group_size == 128) && (bits == 4 || bits == 8) && N > 0 && K > 0 &&
         N % 128 == 0 && (K % (kBlockK * kUnroll) == 0 || (group_size != 128 && K % kBlockK == 0 && K >= 4 * kBlockK));
}

int32_t launch_qmm_rw_grouped(const GroupedQmmArgs& a, hipStream_t s) {
  if (!qmm_rw_grouped_supported(a.N, a.K, a.group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "grouped qmm: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, a.bits,
                a.group_size);
  if (a.max_tiles == 0) return RMLX_OK;
  const bool dual = a.w1 != nullptr;
  if (dual && a.out_f32) return fail(RMLX_RUNTIME_ERROR, "grouped qmm: the gate/up pair writes f16");
  if (a.tile_tab == nullptr || a.n_tiles_dev == nullptr) return fail(RMLX_RUNTIME_ERROR, "grouped qmm: no tile table");
  RwParams p{};
  p.w = a.w; p.s = a.s; p.b = a.b; p.w1 = a.w1; p.s1 = a.s1; p.b1 = a.b1;
  p.x = a.x; p.row_map = a.row_map;
  p.out = static_cast<__half*>(a.out); p.out_f32 = a.out_f32;
  p.M = 0; p.N = a.N; p.K = a.K;
  p.epi_kind = EPI_NONE; p.ksplit = 1;
  p.tile_tab = a.tile_tab; p.n_tiles = a.n_tiles_dev;
  p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  p.tiles_m = (a.max_tiles + 7) / 8 * 8;  // (the grid covers eight equal runs of row tiles, one per XCD)
  // row tiles of 16 * 4 = kGroupedTileRows rows, 8 waves; a pair: 128 columns of each weight per workgroup,
  // one weight: 256 columns when they divide, else 128
  const uint32_t nw = a.tile_rows == 16 ? 4 : 8;
  const bool wide = !dual && a.N % (nw * 32) == 0;
  p.tiles_n = a.N / (wide ? nw * 32 : nw * 16);
  if ((uint64_t)p.tiles_m * p.tiles_n > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "grouped qmm: grid too large");
  if (a.tile_rows != 16 && a.tile_rows != 32 && a.tile_rows != kGroupedTileRows)
    return fail(RMLX_RUNTIME_ERROR, "grouped qmm: row tiles of %u rows", a.tile_rows);
  const dim3 grid(p.tiles_m * p.tiles_n), block(64 * nw);
  const bool tail = a.K % (kBlockK * kUnroll) != 0;
#define RWG_FORMS(MFV, NWV, BITSV, GSV, TAILV)                                                                              \
  if (dual) hipLaunchKernelGGL((qmm_rw_grouped_kernel<MFV, 2, BITSV, NWV, true, GSV, TAILV>), grid, block, 0, s, p);          \
  else if (wide) hipLaunchKernelGGL((qmm_rw_grouped_kernel<MFV, 2, BITSV, NWV, false, GSV, TAILV>), grid, block, 0, s, p);    \
  else hipLaunchKernelGGL((qmm_rw_grouped_kernel<MFV, 1, BITSV, NWV, false, GSV, TAILV>), grid, block, 0, s, p);
#define RWG_LAUNCH(MFV, NWV, BITSV, GSV)                                         \
  if (GSV != 128 && tail) { RWG_FORMS(MFV, NWV, BITSV, (GSV == 128 ? 64 : GSV), true) } else { RWG_FORMS(MFV, NWV, BITSV, GSV, false) }
#define RWG_TILE(BITSV, GSV)                                     \
  if (a.tile_rows == 16) { if (GSV == 64) { RWG_LAUNCH(1, 4, BITSV, 64) } }  \
  else if (a.tile_rows == 32) { RWG_LAUNCH(2, 8, BITSV, GSV) } else { RWG_LAUNCH(4, 8, BITSV, GSV) }
#define RWG_BITS(GSV) \
  if (a.bits == 4) { RWG_TILE(4, GSV) } else { RWG_TILE(8, GSV) }
  if (a.group_size == 64) { RWG_BITS(64) } else if (a.group_size == 32) { RWG_BITS(32) } else { RWG_BITS(128) }
#undef RWG_BITS
#undef RWG_TILE
#undef RWG_LAUNCH
#undef RWG_FORMS
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
