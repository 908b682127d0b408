// Quantized GEMM for gfx950, prefill-sized batches (M from about 100 rows on): weights in registers, 32x32x16
// MFMAs, the K extent of every 128-wide block split over two halves of the workgroup.
//
// Replaces the reference's affine_qmm_nax_q4 / affine_qmm_mma_q8 for large M
// (crates/rmlx-core/src/ops/quantized.rs:3331-3565, 5838-5971).
//
// What bounds a quantized GEMM tile on this part, per 128-wide k block of a 64 x 128 tile (measured):
//   matrix unit   512 clk per SIMD;   L2 -> CU fill  about 45 B/clk per CU (25 KB of activations + weights: 570 clk);
//   LDS           about 150 B/clk per CU;   vector unit  13 instructions per 8 weights unpacked.
// The layout keeps all four near the matrix time:
//   * v_mfma_f32_32x32x16_f16: a 1 KB operand feeds 32 768 flop, twice the 16x16x32 form, so the activation
//     operands read from LDS per block halve (64 KB instead of 128 KB per workgroup).
//   * Tile 64 activation rows x 128 weight rows, eight waves = 4 column groups (32 weight rows each) x 2 k halves.
//     Wave (wn, kh) multiplies its 32 weight rows by all 64 activation rows over k half kh of every block: 4 k steps
//     x 2 activation fragments = 8 MFMAs per block.  Every weight is loaded and unpacked by exactly one wave: lane
//     (row, half) loads 16 contiguous bytes (Q4: 32 values; Q8: 2 x 16 bytes) and dequantises word ks straight
//     into the operand of k step ks.  Weights never touch LDS.
//   * Activations go global -> registers -> LDS (permuted to the slot order of the nibble unpacking, xor-swizzled:
//     writes and reads are bank-conflict free), two stages; operands are read one block ahead into the registers
//     the previous block has just released.
//   * Addresses are buffer resources (uniform base in scalar registers) plus one 32-bit offset per thread, and the
//     loads past the last block are simply not issued, so every s_waitcnt count is exact.
//   * At the end the two k halves are added through LDS (fixed order: deterministic), which also transposes the
//     accumulator layout into row-contiguous stores, with the fused epilogue.
//   * The vector instructions of the unpacking hide behind the matrix instructions only in part (measured: the k loop of
//     the 64-row tile takes the sum, 16 MFMAs x 32 clk + 126 vector instructions x 4 clk per block and SIMD).  For batches that fill the chip
//     with 128 x 128 tiles the same code runs with four activation fragments per wave (MFR = 4): every unpacked weight
//     operand feeds four MFMAs, 64 MFMAs against 71 vector instructions per wave and block.
#include <type_traits>

#include "common.hpp"

namespace rmlx {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 128, kBlockK = 128, kThreads = 512;
constexpr int kUnroll = 4;                       // depth of the weight register ring; scales come per four blocks

struct K2Params {
  const uint32_t* w; const __half* s; const __half* b;
  const void* w_packed;  // tile-contiguous copy of w (PACKED builds), or null
  const __half* x;  // [M,K] row-major f16 (bf16 bits when XBF16)
  __half* out;
  uint32_t M, N, K, tiles_m, tiles_n;
  int32_t epi_kind, epi_dtype;
  const void* epi;
};

__device__ __forceinline__ uint32_t h2bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

struct DqConst { uint32_t m0, m1, k0, k1; };
// 8 Q4 values of one word -> f16 weights in slot order (k0,k4,k1,k5,k2,k6,k3,k7); exact int -> f16 through the
// magic numbers 1024 + q and 64 + q, then w = s*q + b in packed f16
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
// 8 Q8 values of two words -> f16 weights in natural order
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

// LDS slot (16 bytes) of activation unit (row R of the tile, segment seg = 8 consecutive k of the block).  Segment
// seg = 8 kh + 4 hh + ks is read by the waves of k half kh in k step ks, lane half hh; fragment R/32, lane row R%32:
// a contiguous 1 KB run per (fragment, kh, ks).  The xor keeps that run a permutation and spreads the 16 segments
// of a row, which one load instruction delivers to 16 neighbouring lanes, over all banks.
__device__ __forceinline__ uint32_t act_slot(uint32_t R, uint32_t seg) {
  return (((R >> 5) * 2 + (seg >> 3)) * 4 + (seg & 3)) * 64 + (((((seg >> 2) & 1) << 5) | (R & 31)) ^ seg);
}

// MFR: activation fragments of 32 rows per tile (2: 64 x 128 tiles; 4: 128 x 128 tiles, every unpacked weight operand
// then feeds four MFMAs)
// SBLDS: the tile's scales and biases wait in LDS (64-row tiles, group size 64, K <= 4096: a row's 128 bytes of either are
// one cache line, fetched once; read from global memory 16 bytes per four blocks, every read pulls the whole line
// through the CU's L1 again: measured 1.56 x the useful bytes between L2 and the CU).
template <int BITS, bool XBF16, int GS, int MFR, bool SBLDS = false, bool PACKED = false>
__global__ __launch_bounds__(kThreads) void qmm_k2_kernel(const K2Params p) {
  static_assert(!SBLDS || (GS == 64 && MFR <= 2), "scales in LDS: tiles of at most 64 rows, group size 64");
  constexpr int kTileM = 32 * MFR;
  constexpr int kChunkUnits = kTileM * 16;               // 16-byte units of one activation chunk (rows x 128 k): 512 / 1024 / 2048
  constexpr int kAL = kChunkUnits / kThreads;            // units per thread and chunk: 1 / 2 / 4
  constexpr int WV = BITS == 4 ? 1 : 2;                  // 16-byte weight loads per lane and block
  constexpr int kSbBytes = 4 * (kBlockK / GS) * 2;       // scales of one row and four blocks: 16 / 32 / 8 bytes
  constexpr int kSbVecs = kSbBytes > 16 ? 2 : 1;
  __shared__ u4 lds[4096];  // 64 KB: two activation stages of 16 / 32 KB; all of it for the final transposition

  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wn = wave & 3, kh = wave >> 2;
  const uint32_t r = lane & 31, hh = lane >> 5;

  // workgroup -> tile: ids go round-robin over the 8 XCDs (one L2 each); every XCD gets a compact block of tiles
  // (half of the row tiles x a quarter of the column tiles when those divide), so that what its L2 fetches is small
  uint32_t wg = blockIdx.x, mt, nt;
  const uint32_t total = p.tiles_m * p.tiles_n;
  if (total % 8 == 0 && p.tiles_m % 2 == 0 && p.tiles_n % 4 == 0) {
    const uint32_t xcd = wg % 8, local = wg / 8, bm = p.tiles_m / 2, bn = p.tiles_n / 4;
    mt = (xcd % 2) * bm + local % bm;
    nt = (xcd / 2) * bn + local / bm;
  } else {
    if (total % 8 == 0) wg = (wg % 8) * (total / 8) + wg / 8;
    mt = wg % p.tiles_m;
    nt = wg / p.tiles_m;
  }
  const uint32_t K = p.K, S = K / kBlockK, G = K / GS;
  const uint32_t row_lo = mt * kTileM;

  // ---- addresses: buffer resources (uniform base + byte range, in scalar registers) + one 32-bit byte offset per
  // thread; the per-block parts of an address are uniform and ride in the scalar offset operand.  Reads past a
  // resource's range return zero, which is what rows past M must contribute.
  auto make_rsrc = [](const void* base, uint64_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : bytes), 0x00020000);
  };
  const uint32_t row_words = K * BITS / 32;
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x + (uint64_t)row_lo * K, (uint64_t)(p.M - row_lo) * K * 2);
  // (PACKED: the tile's 128 rows x K as one run of (k block, column group, k half, load, lane) x 16 bytes)
  const __amdgpu_buffer_rsrc_t wr = PACKED
      ? make_rsrc(static_cast<const char*>(p.w_packed) + (uint64_t)nt * kTileN * row_words * 4, (uint64_t)kTileN * row_words * 4)
      : make_rsrc(p.w + (uint64_t)nt * kTileN * row_words, (uint64_t)kTileN * row_words * 4);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc(p.s + (uint64_t)nt * kTileN * G, (uint64_t)kTileN * G * 2);
  const __amdgpu_buffer_rsrc_t br = make_rsrc(p.b + (uint64_t)nt * kTileN * G, (uint64_t)kTileN * G * 2);
  // activations: unit q*512 + tid -> (tile row 32 q + tid/16, segment tid%16); 16 neighbouring lanes read one row's
  // 256 contiguous bytes
  const uint32_t seg = tid & 15, R0 = tid >> 4;
  uint32_t xoff[kAL];  // unit q: row R0 + 32 q (in the range-checked part of the address: rows past M read zero)
#pragma unroll
  for (int q = 0; q < kAL; ++q) xoff[q] = ((R0 + 32 * q) * K + seg * 8) * 2;
  const uint32_t lds_w0 = act_slot(R0, seg);     // unit q: + q * 512 slots
  // operand reads of k step ks (fragment i: + 512 slots, stage: + 1024 slots)
  uint32_t lds_r[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) lds_r[ks] = (kh * 4 + ks) * 64 + (((hh << 5) | r) ^ (8 * kh + 4 * hh + ks));
  // weights: row nt*128 + 32 wn + r; this lane's values of block it are k = 128 it + 64 kh + 32 hh .. + 31
  const uint32_t woff = PACKED ? ((wn * 2 + kh) * WV * 64 + lane) * 16
                               : ((32 * wn + r) * row_words) * 4 + (8 * kh + 4 * hh) * 4 * WV;
  const uint32_t soff = (32 * wn + r) * G * 2;

  f16v acc[MFR];
#pragma unroll
  for (int i = 0; i < MFR; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

  // activation chunks in flight (global -> registers -> LDS): two register sets (a chunk is requested two blocks before
  // it is written to LDS), or one where the second would not fit the register file (requested one block before)
  constexpr int kSets = (MFR == 4 && (BITS == 8 || GS == 32)) ? 1 : 2;
  u4 ra[kSets][kAL];
  u4 wq[kUnroll][WV];         // weights, four blocks ahead
  u4 s_cur[kSbVecs], b_cur[kSbVecs], s_nxt[kSbVecs], b_nxt[kSbVecs];  // scales / biases of four blocks

  auto to_slot_order = [&](u4 v) {
    if (XBF16) {  // bf16 activations: to f16 through f32 (exact for normal-range values)
      uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
        w[e] = h2bits((h2){(_Float16)lo, (_Float16)hi});
      }
      v = (u4){w[0], w[1], w[2], w[3]};
    }
    if (BITS != 4) return v;
    u4 o;  // halves (k0..k7) -> slots (k0,k4,k1,k5,k2,k6,k3,k7)
    o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
    o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
    o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
    o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    return o;
  };
  auto load_a = [&](uint32_t it, u4 (&dst)[kAL]) {
#pragma unroll
    for (int q = 0; q < kAL; ++q)
      dst[q] = __builtin_amdgcn_raw_buffer_load_b128(xr, xoff[q], it * (kBlockK * 2), 0);
  };
  auto store_a = [&](uint32_t stage, const u4 (&src)[kAL]) {
#pragma unroll
    for (int q = 0; q < kAL; ++q) lds[stage * kChunkUnits + q * 512 + lds_w0] = to_slot_order(src[q]);
  };
  auto load_w = [&](uint32_t it, int u) {
#pragma unroll
    for (int v = 0; v < WV; ++v)
      wq[u][v] = PACKED ? __builtin_amdgcn_raw_buffer_load_b128(wr, woff, it * (8192 * WV) + v * 1024, 0)
                        : __builtin_amdgcn_raw_buffer_load_b128(wr, woff, it * (16 * 4 * WV) + v * 16, 0);
  };
  // the scales / biases of blocks 4 blk .. 4 blk + 3 of this lane's row
  // (SBLDS: slot of (row, unit of four blocks) behind the two activation stages; the xor spreads the 32 rows of a wave
  // over the banks)
  auto sb_slot = [&](uint32_t which, uint32_t row, uint32_t unit) { return 2048 + which * 1024 + row * 8 + (unit ^ (row & 7)); };
  auto load_sb = [&](uint32_t blk, u4 (&ds)[kSbVecs], u4 (&db)[kSbVecs]) {
    if constexpr (SBLDS) {
      ds[0] = lds[sb_slot(0, 32 * wn + r, blk & 7)];
      db[0] = lds[sb_slot(1, 32 * wn + r, blk & 7)];
    } else if (GS == 128) {
      const u2 sv = __builtin_amdgcn_raw_buffer_load_b64(sr, soff, blk * 8, 0), bv = __builtin_amdgcn_raw_buffer_load_b64(br, soff, blk * 8, 0);
      ds[0] = (u4){sv.x, sv.y, 0u, 0u};
      db[0] = (u4){bv.x, bv.y, 0u, 0u};
    } else {
#pragma unroll
      for (int v = 0; v < kSbVecs; ++v) {
        ds[v] = __builtin_amdgcn_raw_buffer_load_b128(sr, soff, blk * kSbBytes + v * 16, 0);
        db[v] = __builtin_amdgcn_raw_buffer_load_b128(br, soff, blk * kSbBytes + v * 16, 0);
      }
    }
  };
  DqConst dq;
  dq.m0 = 0x000F000Fu; dq.m1 = 0x00F000F0u; dq.k0 = 0x64006400u; dq.k1 = 0x54005400u;
  asm volatile("" : "+s"(dq.m0), "+s"(dq.m1), "+v"(dq.k0), "+v"(dq.k1));
  // (scale, bias) pair of block slot u (u == kUnroll: block 0 of the next four).  This lane's 32 values of a block
  // lie in group (128 it + 64 kh + 32 hh) / GS: GS 64 -> half kh of word u; GS 32 -> half hh of word 2u + kh;
  // GS 128 -> half u%2 of word u/2.
  constexpr uint32_t kSelLo = 0x01000100u, kSelHi = 0x03020302u;
  const uint32_t sel_kh = kh ? kSelHi : kSelLo, sel_hh = hh ? kSelHi : kSelLo;
  auto word_of = [](const u4& v, int c) { return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w)); };
  auto scale_pair = [&](int u, h2& s2, h2& b2) {
    const u4 (&sv)[kSbVecs] = u < kUnroll ? s_cur : s_nxt;
    const u4 (&bv)[kSbVecs] = u < kUnroll ? b_cur : b_nxt;
    const int c = u % kUnroll;
    uint32_t sw, bw, sel;
    if (GS == 64) {
      sw = word_of(sv[0], c); bw = word_of(bv[0], c); sel = sel_kh;
    } else if (GS == 128) {
      sw = word_of(sv[0], c >> 1); bw = word_of(bv[0], c >> 1); sel = (c & 1) ? kSelHi : kSelLo;
    } else {  // word 2c + kh of the eight
      const u4& s4 = sv[(c >> 1) % kSbVecs];
      const u4& b4 = bv[(c >> 1) % kSbVecs];
      sw = kh ? word_of(s4, 2 * (c & 1) + 1) : word_of(s4, 2 * (c & 1));
      bw = kh ? word_of(b4, 2 * (c & 1) + 1) : word_of(b4, 2 * (c & 1));
      sel = sel_hh;
    }
    s2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(sw, sw, sel));
    b2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(bw, bw, sel));
  };
  // weight operand of k step ks of block slot u, given the block's (scale, bias)
  auto weight_operand = [&](int u, int ks, h2 s2, h2 b2) -> h8 {
    const int c = u % kUnroll;
    if (BITS == 4) return dequant_q4_word(word_of(wq[c][0], ks), s2, b2, dq);
    const u4& q = wq[c][(ks >> 1) % WV];
    return (ks & 1) ? dequant_q8_pair(q.z, q.w, s2, b2) : dequant_q8_pair(q.x, q.y, s2, b2);
  };
  auto read_b = [&](uint32_t stage, int i, int ks) -> h8 {
    return __builtin_bit_cast(h8, lds[stage * kChunkUnits + i * 512 + lds_r[ks]]);
  };

  // ---- prologue: chunks 0 and 1 in LDS, chunks 2 and 3 in the register sets, weights of blocks 0..3 ----------
  const uint32_t last = S - 1;
  auto clampi = [&](uint32_t it) { return it < last ? it : last; };
  load_a(0, ra[0]);
  if constexpr (kSets == 2) load_a(clampi(1), ra[kSets - 1]);
  if constexpr (SBLDS) {  // 128 rows x (scales, biases) x up to 8 units of 16 bytes: four pieces per thread, whole lines per row
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t piece = q * kThreads + tid, which = piece >> 10, row = (piece >> 3) & 127, unit = piece & 7;
      u4 v = (u4){0u, 0u, 0u, 0u};
      if (unit * 16 < G * 2) v = __builtin_amdgcn_raw_buffer_load_b128(which ? br : sr, row * G * 2 + unit * 16, 0, 0);
      lds[sb_slot(which, row, unit)] = v;
    }
  } else {
    load_sb(0, s_cur, b_cur);
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) load_w(u, u);  // (S >= 4)
  store_a(0, ra[0]);
  if constexpr (kSets == 2) {
    store_a(1, ra[1]);
    load_a(clampi(2), ra[0]);
    load_a(clampi(3), ra[1]);
  } else {
    load_a(clampi(1), ra[0]);
    store_a(1, ra[0]);
    load_a(clampi(2), ra[0]);
  }
  __syncthreads();
  if constexpr (SBLDS) load_sb(0, s_cur, b_cur);
  h8 bf[MFR][4];
#pragma unroll
  for (int i = 0; i < MFR; ++i)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bf[i][ks] = read_b(0, i, ks);
  __syncthreads();  // block 0 overwrites stage 0 with chunk 2: every wave must have taken its operands of chunk 0 first
  h2 s2, b2;
  scale_pair(0, s2, b2);
  h8 aw = weight_operand(0, 0, s2, b2), aw_nxt;

  // Block `it` (u = it % 4): its activation operands are already in bf[] (read during block it-1 from stage it%2,
  // which nothing reads any more); stage (it+1)%2 holds chunk it+1 and is read into bf[] as the slots come free;
  // chunk it+2 is written into stage it%2 from the register set that chunk it+4 is then loaded into.  Four k steps
  // of two MFMAs, each carrying its share of the other work and unpacking the next weight operand; one barrier per
  // block.  MAIN: blocks that still prefetch (all but the last four).  LOADSB: the block that fetches the scales of
  // the four blocks after the next four.
  auto block = [&](auto uc, auto mainc, uint32_t it) {
    constexpr int u = decltype(uc)::value;
    constexpr bool MAIN = decltype(mainc)::value;
    const uint32_t st_nxt = (u + 1) & 1, st_wr = u & 1;
    const bool writes = MAIN || it + 2 < S;  // (uniform)
    if (MAIN && u == 0) load_sb(it / kUnroll + 1, s_nxt, b_nxt);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int i = 0; i < MFR; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aw, bf[i][ks], acc[i], 0, 0, 0);
        bf[i][ks] = read_b(st_nxt, i, ks);  // the slot is free: next block's operand (past the last block: unused)
      }
      if (ks < 3) {
        aw_nxt = weight_operand(u, ks + 1, s2, b2);
      } else {
        scale_pair(u + 1, s2, b2);
        aw_nxt = weight_operand(u + 1, 0, s2, b2);
      }
      if (ks < kAL && writes) lds[st_wr * kChunkUnits + ks * 512 + lds_w0] = to_slot_order(ra[u % kSets][ks]);
      if (ks == (kAL > 3 ? kAL - 1 : 2)) {  // (the set's last unit has just been written)
        if constexpr (kSets == 2) { if (MAIN) load_a(it + 4, ra[u % 2]); }
        else if (it + 3 < S) load_a(it + 3, ra[0]);  // (uniform)
      }
      aw = aw_nxt;
      __builtin_amdgcn_sched_barrier(0);
    }
    if (MAIN) load_w(it + kUnroll, u);  // (every word of wq[u] has been unpacked)
    if (u == 3) {
#pragma unroll
      for (int v = 0; v < kSbVecs; ++v) { s_cur[v] = s_nxt[v]; b_cur[v] = b_nxt[v]; }
    }
    __syncthreads();
  };
  using std::integral_constant;
  uint32_t it0 = 0;
  for (; it0 + kUnroll < S; it0 += kUnroll) {
    block(integral_constant<int, 0>{}, integral_constant<bool, true>{}, it0);
    block(integral_constant<int, 1>{}, integral_constant<bool, true>{}, it0 + 1);
    block(integral_constant<int, 2>{}, integral_constant<bool, true>{}, it0 + 2);
    block(integral_constant<int, 3>{}, integral_constant<bool, true>{}, it0 + 3);
  }
  block(integral_constant<int, 0>{}, integral_constant<bool, false>{}, it0);
  block(integral_constant<int, 1>{}, integral_constant<bool, false>{}, it0 + 1);
  block(integral_constant<int, 2>{}, integral_constant<bool, false>{}, it0 + 2);
  block(integral_constant<int, 3>{}, integral_constant<bool, false>{}, it0 + 3);

  // ---- the two k halves -> one, and accumulator layout -> rows: through LDS ------------------------------------
  // A lane holds, of fragment i: activation row m = 32 i + r, weight rows 32 wn + 8 (e/4) + 4 hh + e%4.  Partial
  // [kh][m][32 groups of four weight rows], the group index xor-ed with m % 32 so that a wave's stores (32 rows at
  // a stride of 512 bytes) spread over the banks.
  // 64 rows (two fragments) per pass: 2 x 64 x 128 floats fill the 64 KB.
  float* red = reinterpret_cast<float*>(lds);
  constexpr int kFr = MFR >= 2 ? 2 : 1;   // fragments per pass: 64 rows (32 with one fragment) x 128 columns x two halves
  constexpr int kPassRows = 32 * kFr;
#pragma unroll
  for (int pass = 0; pass < MFR / kFr; ++pass) {
  if (pass > 0) __syncthreads();  // the previous pass has been read
#pragma unroll
  for (int i = 0; i < kFr; ++i) {
    const uint32_t m = 32 * i + r;
#pragma unroll
    for (int eg = 0; eg < 4; ++eg) {
      const uint32_t cg = 8 * wn + 2 * eg + hh;  // weight rows 4 cg .. 4 cg + 3 of the tile
      f4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = acc[kFr * pass + i][eg * 4 + e];
      *reinterpret_cast<f4*>(red + ((size_t)(kh * kPassRows + m) * 32 + (cg ^ (m & 31))) * 4) = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 2 * kFr; ++q) {  // rows x 32 groups = units of four outputs: four (two) per thread
    const uint32_t g = q * kThreads + tid, m = g >> 5, cgp = g & 31, cg = cgp ^ (m & 31);
    f4 v = *reinterpret_cast<const f4*>(red + ((size_t)m * 32 + cgp) * 4);
    v += *reinterpret_cast<const f4*>(red + ((size_t)(kPassRows + m) * 32 + cgp) * 4);
    const uint32_t row = row_lo + kPassRows * pass + m, col = nt * kTileN + 4 * cg;
    if (row < p.M) {
      const uint64_t o = (uint64_t)row * p.N + col;
      if (p.epi_kind != EPI_NONE) {  // residual add / SwiGLU gate in f32, one rounding (quantized.rs:3206-3246)
        f4 e;
        if (p.epi_dtype == RMLX_DTYPE_F32) {
          e = *reinterpret_cast<const f4*>(static_cast<const float*>(p.epi) + o);
        } else {
          const u2 eb = *reinterpret_cast<const u2*>(static_cast<const __half*>(p.epi) + o);
          const uint32_t ex = eb.x, ey = eb.y;
          const h2 e0 = __builtin_bit_cast(h2, ex), e1 = __builtin_bit_cast(h2, ey);
          e = (f4){(float)e0[0], (float)e0[1], (float)e1[0], (float)e1[1]};
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = p.epi_kind == EPI_RESIDUAL ? v[c] + e[c] : e[c] / (1.0f + __expf(-e[c])) * v[c];
      }
      const h2 lo = {(_Float16)v[0], (_Float16)v[1]};
      const h2 hi = {(_Float16)v[2], (_Float16)v[3]};
      *reinterpret_cast<u2*>(p.out + o) = (u2){h2bits(lo), h2bits(hi)};
    }
  }
  }
}

// One thread per 16-byte unit of the destination: unit = ((((nt * S + blk) * 4 + wn) * 2 + kh) * WV + v) * 64 + lane
// <- the 16 bytes that lane (row lane % 32, half lane / 32) of wave (wn, kh) loads as load v of k block blk of column tile nt.
__global__ __launch_bounds__(256) void gemm_repack_kernel(const uint32_t* __restrict__ w, uint32_t K, uint32_t bits, uint64_t units,
                                                          u4* __restrict__ dst) {
  const uint64_t unit = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (unit >= units) return;
  const uint32_t WV = bits == 4 ? 1 : 2, S = K / kBlockK, row_bytes = K * bits / 8;
  const uint32_t lane = unit & 63;
  uint64_t rest = unit >> 6;
  const uint32_t v = rest % WV; rest /= WV;
  const uint32_t kh = rest & 1, wn = (rest >> 1) & 3; rest >>= 3;
  const uint32_t blk = rest % S, nt = rest / S;
  const uint32_t row = nt * kTileN + 32 * wn + (lane & 31), hh = lane >> 5;
  const uint64_t src = (uint64_t)row * row_bytes + (uint64_t)blk * (64 * WV) + (8 * kh + 4 * hh) * 4 * WV + v * 16;
  dst[unit] = *reinterpret_cast<const u4*>(reinterpret_cast<const char*>(w) + src);
}

}  // namespace

size_t gemm_layout_bytes(size_t N, size_t K, uint32_t bits) {
  if (!(bits == 4 || bits == 8) || N == 0 || K == 0 || N % kTileN != 0 || K % (kBlockK * kUnroll) != 0) return 0;
  return N * K * bits / 8;
}

int32_t launch_gemm_repack(const uint32_t* w, uint32_t N, uint32_t K, uint32_t bits, void* dst, hipStream_t s) {
  const size_t bytes = gemm_layout_bytes(N, K, bits);
  if (bytes == 0) return fail(RMLX_INVALID_SHAPE, "gemm layout: N %% 128 == 0, K %% 512 == 0 and 4- or 8-bit weights required (N=%u K=%u bits=%u)", N, K, bits);
  const uint64_t units = bytes / 16;
  hipLaunchKernelGGL(gemm_repack_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s, w, K, bits, units, static_cast<u4*>(dst));
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

bool qmm_k2_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  return (group_size == 32 || group_size == 64 || group_size == 128) && (bits == 4 || bits == 8) && N > 0 && K > 0 &&
         N % kTileN == 0 && K % (kBlockK * kUnroll) == 0;
}

bool qmm_k2_tall_supported(uint32_t group_size, uint32_t bits, bool x_bf16) {
  // (8-bit weights at group size 32 / 64 with bf16 activations: that build would spill registers)
  return (bits == 4 || bits == 8) && (group_size == 32 || group_size == 64 || group_size == 128) &&
         !(bits == 8 && x_bf16 && group_size != 128);
}

int32_t launch_qmm_k2(const QmmArgs& a, uint32_t group_size, uint32_t tile_rows, hipStream_t s) {
  if (tile_rows != 64 && tile_rows != 32 && !(tile_rows == 128 && qmm_k2_tall_supported(group_size, a.bits, a.x_dtype == RMLX_DTYPE_BF16)))
    return fail(RMLX_INVALID_SHAPE, "qmm: no K-split kernel with %u-row tiles for bits=%u group_size=%u (%s activations)", tile_rows,
                a.bits, group_size, a.x_dtype == RMLX_DTYPE_BF16 ? "bf16" : "f16");
  if (!qmm_k2_supported(a.N, a.K, group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "qmm: unsupported shape N=%u K=%u bits=%u group_size=%u", a.N, a.K, a.bits, group_size);
  if (a.M == 0) return RMLX_OK;
  if (a.x_dtype != RMLX_DTYPE_F16 && a.x_dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_RUNTIME_ERROR, "qmm: f32 activations must be cast to f16 first");
  K2Params p{};
  p.w = a.w; p.s = a.s; p.b = a.b;
  p.w_packed = a.w_packed;
  p.x = static_cast<const __half*>(a.x);
  p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K;
  p.tiles_m = (a.M + tile_rows - 1) / tile_rows;
  p.tiles_n = a.N / kTileN;
  p.epi_kind = a.epi_kind; p.epi = a.epi; p.epi_dtype = a.epi_dtype;
  if ((uint64_t)p.tiles_m * p.tiles_n > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "qmm: grid too large");
  const dim3 grid(p.tiles_m * p.tiles_n), block(kThreads);
  const bool xb = a.x_dtype == RMLX_DTYPE_BF16, tall = tile_rows == 128;
  const bool sb_lds = group_size == 64 && !tall && a.K <= 4096;
  const bool low = tile_rows == 32;
  const bool packed = a.w_packed != nullptr;
  auto launch = [&](auto bits_c, auto gs_c, auto mfr_c) {
    constexpr int B = decltype(bits_c)::value, GSV = decltype(gs_c)::value, MFRV = decltype(mfr_c)::value;
    auto go = [&](auto xb_c, auto sb_c) {
      constexpr bool XB = decltype(xb_c)::value, SB = decltype(sb_c)::value;
      if constexpr (!(XB && MFRV == 4 && B == 8 && GSV != 128)) {
        if (packed) hipLaunchKernelGGL((qmm_k2_kernel<B, XB, GSV, MFRV, SB, true>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((qmm_k2_kernel<B, XB, GSV, MFRV, SB, false>), grid, block, 0, s, p);
      }
    };
    typedef std::true_type T;
    typedef std::false_type F;
    if constexpr (GSV == 64 && MFRV <= 2) {
      if (sb_lds) {
        if (xb) go(T{}, T{}); else go(F{}, T{});
        return;
      }
    }
    if (xb) go(T{}, F{}); else go(F{}, F{});
  };
  using std::integral_constant;
  typedef integral_constant<int, 2> Low;
  typedef integral_constant<int, 1> Flat;
  typedef integral_constant<int, 4> Tall;
  typedef integral_constant<int, 4> B4;
  typedef integral_constant<int, 8> B8;
  auto by_height = [&](auto bits_c, auto gs_c) {
    if (tall) launch(bits_c, gs_c, Tall{});
    else if (low) launch(bits_c, gs_c, Flat{});
    else launch(bits_c, gs_c, Low{});
  };
  auto by_group = [&](auto bits_c) {
    if (group_size == 64) by_height(bits_c, integral_constant<int, 64>{});
    else if (group_size == 128) by_height(bits_c, integral_constant<int, 128>{});
    else by_height(bits_c, integral_constant<int, 32>{});
  };
  if (a.bits == 4) by_group(B4{}); else by_group(B8{});
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
