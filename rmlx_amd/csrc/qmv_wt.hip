// Wave-per-tile streaming GEMV for 4-bit weights on gfx950: the expert projections of decode-sized MoE
// batches and gather_qmm over stacked weights (chunks of at most 8 or 16 rows of one expert), and dense
// matrices at group size 32 (chunks of 8 rows of the [M, K] activations).
//
// Replaces the reference's gather_qmv_fast_f16_q4 / moe_expert_matmul_q4
// (crates/rmlx-core/src/ops/quantized.rs:9752-9842, 10257-10370).
//
// The K-split kernel of qmv.hip lets eight waves share one 16-row weight tile and meet in a reduction
// through LDS after every tile: two barriers per tile, during which a workgroup has no loads in flight.
// Here a wave owns a whole tile (16 weight rows, all of K; fused gate / up: the same rows of both
// matrices) and walks it in passes of two or four 128-k slabs with the next pass already requested into a
// second register set - across tile boundaries too - so a wave always has loads in flight and never
// waits for another wave: after the activations are staged there is no barrier at all.
//   * The workgroup stages the chunk's activations once, for all of K, into one LDS image in the
//     operand order of the matrix instruction, together with the per (row, group) sums; every wave
//     reads its operands from that image.  Chunks of up to 16 rows keep two such images (rows 0-7 and
//     8-15) and multiply each unpacked weight operand against both, so an expert with 9 to 16 rows
//     still streams its weights once.
//   * Arithmetic is that of qmv.hip: 16x16x32 f16 matrix instructions with the weights as the B
//     operand, nibbles to f16 by mask-or, accumulator rows 0-7 / 8-15 carrying the two quantisation
//     groups of a slab, accumulators started from -sum(off*x), F += scale * c + bias * sum(x).
//   * Weight addresses are a buffer resource per matrix (the expert's base, in scalar registers), one
//     32-bit offset per lane and a wave-uniform offset per tile and slab.
#include <type_traits>

#include "common.hpp"
#include "q4_stream.hpp"

namespace rmlx {
namespace {

using namespace q4;

constexpr int kBlk = 33;   // 16-byte slots per (slab, j) block of an image: 4 k sub-blocks x 8 rows, then a slot of zeros

struct __attribute__((packed, aligned(4))) U2Unaligned { uint32_t v[2]; };

struct WtParams {
  const uint32_t* w0; const __half* s0; const __half* b0;  // tile set 0
  const uint32_t* w1; const __half* s1; const __half* b1;  // tile set 1 (fused gate / up only)
  const __half* x;
  const uint32_t* row_map;
  const uint32_t* chunk_tab;
  const uint32_t* n_chunks;
  void* out;
  uint32_t K, n_tiles, tiles_per_wg, ld_out, out_f32, M;
  uint32_t rows_per_expert;  // weight rows behind w0 (and behind w1) that one expert's buffer resource covers
  uint64_t estride_w, estride_s;
};

// RH = 8-row halves of a chunk (1: up to 8 rows, 2: up to 16); NW = waves per workgroup; DUAL = gate and up tiles with
// silu(g) * u written; TAB = rows come from a device chunk table; kPass = slabs per pass (one 16-byte load per lane,
// tile and slab; two register sets of a pass each are in flight or in use).
// GC = MFMA chains per slab: 1 for group size 64 (the 16 accumulator rows carry 8 activation rows x the slab's two
// groups), 2 for group size 32 (four groups per slab: chain c carries groups 2c and 2c + 1, so the matrix instructions
// and the operand reads double while the weights are still unpacked once).
template <int RH, int NW, bool DUAL, bool TAB, int kPass, int NS, int GC>
__global__ __launch_bounds__(NW * 64, NW == 8 && RH == 1 ? 4 : 1) void qmv_wt_kernel(WtParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TILES = DUAL ? 2 : 1;
  constexpr int NT = NW * 64;
  const uint32_t K = p.K, S = K >> 7, NP = S / kPass, upr = K >> 3;  // slabs, passes, 16-byte activation units per row
  const uint32_t img_half = S * 4 * kBlk * 16;                        // bytes of one 8-row image
  float* const sums_all = reinterpret_cast<float*>(smem + RH * img_half);  // [half][slab][chain][group of the chain][rows 0-3 / 4-7][-xoff x 4, xsum x 4]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4, par = g >> 1;

  // ---- which rows ------------------------------------------------------------------------
  uint32_t expert = 0, row0 = blockIdx.y * (8 * RH), rows;
  bool write_zeros = false;
  if (TAB) {
    if (p.n_chunks != nullptr && blockIdx.y >= *p.n_chunks) return;
    expert = p.chunk_tab[3 * blockIdx.y + 0];
    row0 = p.chunk_tab[3 * blockIdx.y + 1];
    rows = p.chunk_tab[3 * blockIdx.y + 2];
    write_zeros = (rows >> 31) != 0;
    rows &= 0x7FFFFFFFu;
  } else {
    rows = p.M - row0 < 8u * RH ? p.M - row0 : 8u * RH;
  }
  if (rows > 8u * RH) rows = 8u * RH;  // (the host builds chunks of at most that many rows)

  // ---- which tiles: wave w takes tiles first + w, first + w + NW, ... of the workgroup's range -------------
  const uint32_t first = blockIdx.x * p.tiles_per_wg;
  const uint32_t last = first + p.tiles_per_wg < p.n_tiles ? first + p.tiles_per_wg : p.n_tiles;
  const uint32_t my_tiles = first + wave < last ? (last - first - wave + NW - 1) / NW : 0u;
  const uint32_t n_steps = my_tiles * NP;

  // ---- addresses --------------------------------------------------------------------------
  const uint32_t row_bytes = K >> 1, gpr = (K >> 6) * GC;  // packed bytes and quantisation groups per weight row
  constexpr int kSbWords = kPass * GC;  // scale (or bias) words of a pass: two groups per word
  auto make_rsrc = [](const void* base, uint64_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : bytes), 0x00020000);
  };
  const uint64_t e_w = TAB ? expert * p.estride_w : 0, e_s = TAB ? expert * p.estride_s : 0;
  __amdgpu_buffer_rsrc_t wr[TILES];
  const __half* sb_base[TILES];  // scales for the lanes with even g, biases for those with odd g (exchanged at use)
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    wr[t] = make_rsrc((t == 0 ? p.w0 : p.w1) + e_w, (uint64_t)p.rows_per_expert * row_bytes);
    sb_base[t] = ((g & 1) ? (t == 0 ? p.b0 : p.b1) : (t == 0 ? p.s0 : p.s1)) + e_s + (uint64_t)n * gpr;
  }
  const uint32_t lane_woff = (uint32_t)n * row_bytes + (uint32_t)g * 16;

  struct Set {  // what one pass of one tile needs: 4 slabs of weights and their scales / biases, per tile slot
    u4 w[TILES][kPass];
    uint32_t sb[TILES][kSbWords];  // word it * GC + c: the two groups of chain c of slab `it` (scales or biases, by lane)
  };
  // the loads of pass `pass` of tile `tile` (wave-uniform): scales / biases first, the memory counter retires in order
  // Waves start at different passes of their tiles (and wrap around), so that the waves of the chip do not all read the
  // same column range of their rows at the same moment (measured: within 1 % of starting every tile at pass 0).
  const uint32_t skew = (wave * 5 + blockIdx.x * 3 + blockIdx.y) % NP;
  auto load_step = [&](uint32_t tile, uint32_t pass_i, Set& st) {
    const uint32_t pass = pass_i + skew < NP ? pass_i + skew : pass_i + skew - NP;
    const uint32_t tile_row = tile * 16;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const uint32_t* sp = reinterpret_cast<const uint32_t*>(sb_base[t] + (uint64_t)tile_row * gpr) + pass * kSbWords;
      if constexpr (kSbWords == 2) {  // (4-byte aligned is enough for the hardware)
        const U2Unaligned v = *reinterpret_cast<const U2Unaligned*>(sp);
        st.sb[t][0] = v.v[0]; st.sb[t][1] = v.v[1];
      } else {
#pragma unroll
        for (int q = 0; q < kSbWords / 4; ++q) {
          const U4Unaligned v = *reinterpret_cast<const U4Unaligned*>(sp + 4 * q);
          st.sb[t][4 * q] = v.v[0]; st.sb[t][4 * q + 1] = v.v[1]; st.sb[t][4 * q + 2] = v.v[2]; st.sb[t][4 * q + 3] = v.v[3];
        }
      }
    }
    const uint32_t soff = tile_row * row_bytes + pass * (kPass * 64);
#pragma unroll
    for (int it = 0; it < kPass; ++it)
#pragma unroll
      for (int t = 0; t < TILES; ++t) st.w[t][it] = __builtin_amdgcn_raw_buffer_load_b128(wr[t], lane_woff, soff + it * 64, 0);
  };

  // ---- 1. the chunk's activations -> LDS images in operand order (requested before the first weights: loads retire
  //         in order, and the activations are needed first) -----------------------------------------------------
  uint32_t srcs[8 * RH];  // source rows (wave-uniform)
#pragma unroll
  for (int m = 0; m < 8 * RH; ++m) {
    srcs[m] = row0 + m;
    if (TAB && p.row_map != nullptr && (uint32_t)m < rows) srcs[m] = p.row_map[row0 + m];
  }
  u4 xv[8 * RH];
#pragma unroll
  for (int m = 0; m < 8 * RH; ++m) {
    xv[m] = (u4){0u, 0u, 0u, 0u};
    if ((uint32_t)m < rows && (uint32_t)tid < upr) xv[m] = *reinterpret_cast<const u4*>(p.x + (uint64_t)srcs[m] * K + (uint32_t)tid * 8);
  }
  Set sets[NS];  // ring of register sets: one being multiplied, the others in flight
  uint32_t ld_tile = first + wave, ld_pass = 0;  // cursor of the next loads
  auto advance = [&](uint32_t& tile, uint32_t& pass) {
    if (++pass == NP) { pass = 0; tile += NW; }
  };
  // (the first pass only: the activations come first, and the in-order memory counter would make them wait for more)
  if (n_steps > 0) { load_step(ld_tile, ld_pass, sets[0]); advance(ld_tile, ld_pass); }
  if ((uint32_t)tid < upr) {
    // unit u = tid: k = 8 u .. 8 u + 7 -> slab u / 16, k sub-block (u / 4) % 4, product u % 4
    const uint32_t slab = (uint32_t)tid >> 4, gg = ((uint32_t)tid >> 2) & 3, j = (uint32_t)tid & 3;
    char* base = smem + ((slab * 4 + j) * kBlk + gg * 8) * 16;
#pragma unroll
    for (int m = 0; m < 8 * RH; ++m)
      *reinterpret_cast<u4*>(base + (m >> 3) * img_half + (m & 7) * 16) = permute_x8(xv[m]);
  }
  for (uint32_t z = tid; z < RH * S * 4; z += NT)  // the zero slot of every block
    *reinterpret_cast<u4*>(smem + (z / (S * 4)) * img_half + ((z % (S * 4)) * kBlk + 32) * 16) = (u4){0u, 0u, 0u, 0u};
  lds_barrier();

  // A-operand activity.  Group size 64: accumulator rows 0-7 take a slab's first group (k sub-blocks g < 2), rows 8-15
  // its second (g >= 2).  Group size 32: a k sub-block is a group; chain c gives rows 0-7 sub-block 2c and rows 8-15
  // sub-block 2c + 1.  The other lanes read the block's zero slot.
  uint32_t a_slot_off[GC];
#pragma unroll
  for (int c = 0; c < GC; ++c) {
    const bool a_active = GC == 1 ? (n < 8) == (g < 2) : g == 2 * c + (n >= 8 ? 1 : 0);
    a_slot_off[c] = (a_active ? (uint32_t)g * 8 + (n & 7) : 32u) * 16;
  }
  Q4Consts qc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(qc.m0), "+s"(qc.m1), "+v"(qc.k0), "+v"(qc.k1));

  // ---- 2. sums of the staged activations per (row, group), on the matrix unit: columns 0-7 of a constant B operand
  //         hold the unpack offsets (1024 / 64 by slot), columns 8-15 ones, so accumulator column 0 receives
  //         sum(off*x) of its rows and column 8 sum(x) -------------------------------------------------------------
  {
    const u4 bconst_bits = n < 8 ? (u4){0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u}
                                 : (u4){0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
    const h8 bconst = __builtin_bit_cast(h8, bconst_bits);
    for (uint32_t q = wave; q < RH * S; q += NW) {
      const uint32_t h = q / S, slab = q % S;
#pragma unroll
      for (int c = 0; c < GC; ++c) {
        f4 own = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const h8 av = *reinterpret_cast<const h8*>(smem + h * img_half + ((slab * 4 + j) * kBlk) * 16 + a_slot_off[c]);
          own = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bconst, own, 0, 0, 0);
        }
        float* sp = sums_all + (((q * GC + c) * 2 + par) * 2 + (g & 1)) * 8;
        if (n == 0) *reinterpret_cast<f4*>(sp) = -own;
        if (n == 8) *reinterpret_cast<f4*>(sp + 4) = own;
      }
    }
  }
  lds_barrier();
  if (n_steps == 0) return;

  // ---- 3. the wave's tiles, pass by pass -------------------------------------------------------------------------
  const uint32_t half_sel = par ? 0x07060302u : 0x05040100u;  // the lane's group of every (scale, scale) word
  auto half_at = [](const uint32_t (&o)[kSbWords / 2], int widx) -> float {
    const uint32_t wd = o[widx >> 1];
    const unsigned short hb = (widx & 1) ? (unsigned short)(wd >> 16) : (unsigned short)(wd & 0xFFFFu);
    return (float)__builtin_bit_cast(_Float16, hb);
  };
  f4 F[RH][TILES];
  uint32_t c_tile = first + wave, c_pass = 0;  // cursor of the pass being multiplied
  // H = 8-row halves that hold rows (wave-uniform: a chunk of at most 8 rows skips the second image)
  auto compute_halves = [&](const Set& st, auto hc) {
    constexpr int H = decltype(hc)::value;
    if (c_pass == 0) {
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int t = 0; t < TILES; ++t) F[h][t] = (f4){0.f, 0.f, 0.f, 0.f};
    }
    uint32_t sv[TILES][kSbWords / 2], bv[TILES][kSbWords / 2];  // the lane's group of every word, two words per register
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int q = 0; q < kSbWords / 2; ++q) {
        const uint32_t own = __builtin_amdgcn_perm(st.sb[t][2 * q + 1], st.sb[t][2 * q], half_sel), oth = swap16(own);
        sv[t][q] = (g & 1) ? oth : own;
        bv[t][q] = (g & 1) ? own : oth;
      }
    const uint32_t slab0 = (c_pass + skew < NP ? c_pass + skew : c_pass + skew - NP) * kPass;
#pragma unroll
    for (int it = 0; it < kPass; ++it) {
      const uint32_t slab = slab0 + it;
      f4 c[H][GC][TILES];
      f4 xsum[H][GC];
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int ch = 0; ch < GC; ++ch) {
          const float* sp = sums_all + ((((h * S + slab) * GC + ch) * 2 + par) * 2 + (g & 1)) * 8;
          const f4 negoff = *reinterpret_cast<const f4*>(sp);
          xsum[h][ch] = *reinterpret_cast<const f4*>(sp + 4);
#pragma unroll
          for (int t = 0; t < TILES; ++t) c[h][ch][t] = negoff;  // the chain ends in dot - sum(off*x)
        }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        h8 bw[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          const uint32_t wd = j == 0 ? st.w[t][it].x : (j == 1 ? st.w[t][it].y : (j == 2 ? st.w[t][it].z : st.w[t][it].w));
          bw[t] = unpack_q4_word(wd, qc);
        }
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
          for (int ch = 0; ch < GC; ++ch) {
            const h8 av = *reinterpret_cast<const h8*>(smem + h * img_half + ((slab * 4 + j) * kBlk) * 16 + a_slot_off[ch]);
#pragma unroll
            for (int t = 0; t < TILES; ++t) c[h][ch][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bw[t], c[h][ch][t], 0, 0, 0);
          }
      }
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int ch = 0; ch < GC; ++ch) {
          const float sc = half_at(sv[t], it * GC + ch), bi = half_at(bv[t], it * GC + ch);
#pragma unroll
          for (int h = 0; h < H; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) F[h][t][i] = fmaf(sc, c[h][ch][t][i], fmaf(bi, xsum[h][ch][i], F[h][t][i]));
        }
    }
    if (c_pass == NP - 1) {
      // the tile is complete: add the two group halves (lane ^ 32), lanes with g < 2 write rows 4g .. 4g+3, column n
      const uint32_t col = c_tile * 16 + n;
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v[TILES];
#pragma unroll
          for (int t = 0; t < TILES; ++t) v[t] = add_other_half(F[h][t][i]);
          float r = DUAL ? silu_f(v[0]) * v[TILES - 1] : v[0];
          if (write_zeros) r = 0.f;
          const uint32_t m = 8 * h + 4 * g + i;
          if (g < 2 && m < rows) {
            const uint64_t o = (uint64_t)(row0 + m) * p.ld_out + col;
            if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = r;
            else reinterpret_cast<__half*>(p.out)[o] = __float2half(r);
          }
        }
    }
    advance(c_tile, c_pass);
  };
  // (the fused gate / up kernel only: it runs eight waves and has the registers for both forms; in the plain 16-wave
  // kernel the second form spills)
  const bool one_half = RH == 2 && DUAL && rows <= 8;
  auto compute_step = [&](const Set& st) {
    if constexpr (RH == 2 && DUAL) {
      if (one_half) { compute_halves(st, std::integral_constant<int, 1>{}); return; }
    }
    compute_halves(st, std::integral_constant<int, RH>{});
  };

#pragma unroll
  for (int q = 1; q < NS - 1; ++q)
    if ((uint32_t)q < n_steps) { load_step(ld_tile, ld_pass, sets[q]); advance(ld_tile, ld_pass); }
  for (uint32_t i = 0; i < n_steps; i += NS) {
#pragma unroll
    for (int q = 0; q < NS; ++q) {
      if (i + q < n_steps) {
        if (i + q + NS - 1 < n_steps) { load_step(ld_tile, ld_pass, sets[(q + NS - 1) % NS]); advance(ld_tile, ld_pass); }
        compute_step(sets[q]);
      }
    }
  }
}

// ---- down projection with the weighted combine fused behind it, for decode-sized batches ----------------------------
// One workgroup per (token, 16-column tile): wave k multiplies the hidden row of the token's k-th assignment with that
// assignment's expert (a wave per (expert, tile), all of K, two register sets as above) and the eight results meet in
// LDS, where they are added as out[t] = sum_k w[t,k] * y_k in ascending k - the order and the f32 arithmetic of the
// separate combine kernel - and written as f16.  No intermediate [assignments, N] matrix, no combine launch.  An expert
// shared by two tokens is streamed once per token, which is why this form is for batches of a few tokens.
struct WcParams {
  const uint32_t* w; const __half* s; const __half* b;  // stacked weights, expert 0
  const __half* h;        // [assignments, K] f16, row a = assignment a (token a / top_k)
  const uint32_t* idx;    // [assignments] expert of every assignment (outside [0, n_experts): contributes nothing)
  const float* wts;       // [assignments] combine weights
  __half* out;            // [T, N]
  uint32_t K, N, top_k, n_experts;
  uint64_t estride_w, estride_s;
};

template <int kPass>
__global__ __launch_bounds__(512) void qmv_wt_combine_kernel(WcParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int kBlk1 = 5;  // slots per (slab, j) block of a one-row image: four k sub-blocks, then zeros
  const uint32_t K = p.K, S = K >> 7, NP = S / kPass;
  const uint32_t img_bytes = S * 4 * kBlk1 * 16, sums_bytes = S * 2 * 2 * sizeof(float);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4, par = g >> 1;
  char* const img = smem + wave * (img_bytes + sums_bytes);
  float* const sums = reinterpret_cast<float*>(img + img_bytes);           // [slab][group] = (-sum(off*x), sum(x))
  float* const red = reinterpret_cast<float*>(smem + 8 * (img_bytes + sums_bytes));  // [wave][column]
  const uint32_t t = blockIdx.y, tile = blockIdx.x, a = t * p.top_k + wave;
  uint32_t expert = 0xFFFFFFFFu;
  float cw = 0.f;
  if ((uint32_t)wave < p.top_k) {
    expert = p.idx[a];
    cw = p.wts[a];
  }
  const bool live = expert < p.n_experts;  // (wave-uniform)
  float mine = 0.f;
  if (live) {
    const uint32_t row_bytes = K >> 1, gpr = K >> 6, tile_row = tile * 16;
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(p.w + expert * p.estride_w), 0, (int)((uint64_t)p.N * row_bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : (uint64_t)p.N * row_bytes), 0x00020000);
    const __half* sb_base = ((g & 1) ? p.b : p.s) + expert * p.estride_s + (uint64_t)(tile_row + n) * gpr;
    const uint32_t lane_woff = (uint32_t)(tile_row + n) * row_bytes + (uint32_t)g * 16;
    struct Set { u4 w[kPass]; uint32_t sb[kPass]; };
    auto load_step = [&](uint32_t pass, Set& st) {
      const uint32_t* sp = reinterpret_cast<const uint32_t*>(sb_base) + pass * kPass;
      if constexpr (kPass == 4) {
        const U4Unaligned v = *reinterpret_cast<const U4Unaligned*>(sp);
        st.sb[0] = v.v[0]; st.sb[1] = v.v[1]; st.sb[2] = v.v[2]; st.sb[3] = v.v[3];
      } else {
        const U2Unaligned v = *reinterpret_cast<const U2Unaligned*>(sp);
        st.sb[0] = v.v[0]; st.sb[1] = v.v[1];
      }
#pragma unroll
      for (int it = 0; it < kPass; ++it) st.w[it] = __builtin_amdgcn_raw_buffer_load_b128(wr, lane_woff, pass * (kPass * 64) + it * 64, 0);
    };
    // the wave's activation row (requested first), then the first pass of weights
    constexpr int kMaxUnits = 8;  // K <= 4096: up to 8 units of 16 bytes per lane
    const u4* xg = reinterpret_cast<const u4*>(p.h + (uint64_t)a * K);
    u4 xv[kMaxUnits];
#pragma unroll
    for (int i = 0; i < kMaxUnits; ++i) {
      xv[i] = (u4){0u, 0u, 0u, 0u};
      if ((uint32_t)(lane + 64 * i) < (K >> 3)) xv[i] = xg[lane + 64 * i];
    }
    Set sa, sbuf;
    load_step(0, sa);
#pragma unroll
    for (int i = 0; i < kMaxUnits; ++i) {
      const uint32_t u = lane + 64 * i;
      if (u < (K >> 3)) {
        const uint32_t slab = u >> 4, gg = (u >> 2) & 3, j = u & 3;
        *reinterpret_cast<u4*>(img + ((slab * 4 + j) * kBlk1 + gg) * 16) = permute_x8(xv[i]);
      }
    }
    for (uint32_t z = lane; z < S * 4; z += 64) *reinterpret_cast<u4*>(img + (z * kBlk1 + 4) * 16) = (u4){0u, 0u, 0u, 0u};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (the image is private to the wave: no barrier)
    // accumulator row 0 takes a slab's first group (k sub-blocks g < 2), row 8 its second; the other lanes read zeros
    const bool a_active = (n == 0 && g < 2) || (n == 8 && g >= 2);
    const uint32_t a_slot_off = (a_active ? (uint32_t)g : 4u) * 16;
    Q4Consts qc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(qc.m0), "+s"(qc.m1), "+v"(qc.k0), "+v"(qc.k1));
    {
      const u4 bconst_bits = n < 8 ? (u4){0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u}
                                   : (u4){0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
      const h8 bconst = __builtin_bit_cast(h8, bconst_bits);
      for (uint32_t slab = 0; slab < S; ++slab) {
        f4 own = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const h8 av = *reinterpret_cast<const h8*>(img + ((slab * 4 + j) * kBlk1) * 16 + a_slot_off);
          own = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bconst, own, 0, 0, 0);
        }
        // accumulator row 0 (lanes g == 0) is the first group, row 8 (lanes g == 2) the second; column 0: sum(off*x), column 8: sum(x)
        if ((g & 1) == 0 && n == 0) sums[(slab * 2 + par) * 2] = -own.x;
        if ((g & 1) == 0 && n == 8) sums[(slab * 2 + par) * 2 + 1] = own.x;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const uint32_t half_sel = par ? 0x07060302u : 0x05040100u;
    float F = 0.f;  // row 0 / row 8 of the accumulator tile: lanes with g == 0 / g == 2, element 0
    auto compute_step = [&](uint32_t pass, const Set& st) {
      uint32_t sv[kPass / 2], bv[kPass / 2];
#pragma unroll
      for (int q = 0; q < kPass / 2; ++q) {
        const uint32_t own = __builtin_amdgcn_perm(st.sb[2 * q + 1], st.sb[2 * q], half_sel), oth = swap16(own);
        sv[q] = (g & 1) ? oth : own;
        bv[q] = (g & 1) ? own : oth;
      }
#pragma unroll
      for (int it = 0; it < kPass; ++it) {
        const uint32_t slab = pass * kPass + it;
        const float2 k2 = *reinterpret_cast<const float2*>(sums + (slab * 2 + par) * 2);
        f4 c = (f4){k2.x, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t wd = j == 0 ? st.w[it].x : (j == 1 ? st.w[it].y : (j == 2 ? st.w[it].z : st.w[it].w));
          const h8 av = *reinterpret_cast<const h8*>(img + ((slab * 4 + j) * kBlk1) * 16 + a_slot_off);
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, unpack_q4_word(wd, qc), c, 0, 0, 0);
        }
        const uint32_t swd = sv[it >> 1], bwd = bv[it >> 1];
        const float sc = (float)__builtin_bit_cast(_Float16, (unsigned short)((it & 1) ? swd >> 16 : swd & 0xFFFFu));
        const float bi = (float)__builtin_bit_cast(_Float16, (unsigned short)((it & 1) ? bwd >> 16 : bwd & 0xFFFFu));
        F = fmaf(sc, c.x, fmaf(bi, k2.y, F));
      }
    };
    for (uint32_t i = 0; i < NP; i += 2) {
      if (i + 1 < NP) load_step(i + 1, sbuf);
      compute_step(i, sa);
      if (i + 1 < NP) {
        if (i + 2 < NP) load_step(i + 2, sa);
        compute_step(i + 1, sbuf);
      }
    }
    // lanes with (g & 1) == 0 hold the row's two group halves (g = 0 and g = 2): lane ^ 32 is the other one
    mine = add_other_half((g & 1) == 0 ? F : 0.f);
  }
  if (g == 0) red[wave * 16 + n] = mine * cw;
  lds_barrier();
  if (tid < 16) {
    float acc = 0.f;
    for (uint32_t k = 0; k < p.top_k; ++k) acc += red[k * 16 + tid];  // ascending k, as the combine kernel adds
    p.out[(uint64_t)t * p.N + tile * 16 + tid] = __float2half(acc);
  }
}

template <int RH, int NW, bool DUAL, int kPass, int NS, int GC = 1>
int32_t launch_one(const WtParams& p, bool tab, dim3 grid, size_t lds_bytes, hipStream_t s) {
  auto go = [&](auto kernel) -> int32_t {
    static bool configured = false;  // (per instantiation; the attribute is idempotent, so a race only repeats the call)
    if (!configured) {
      RMLX_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds_bytes, s, p);
    return RMLX_OK;
  };
  if (tab) return go(qmv_wt_kernel<RH, NW, DUAL, true, kPass, NS, GC>);
  return go(qmv_wt_kernel<RH, NW, DUAL, false, kPass, NS, GC>);
}

}  // namespace

// bytes of LDS a workgroup needs: per 8-row half the image (33 slots of 16 bytes per (slab, product)) and the sums
static size_t wt_lds_bytes(uint32_t K, uint32_t group_size, uint32_t chunk_rows) {
  const size_t slabs = K >> 7, chains = group_size == 32 ? 2 : 1;
  return (size_t)(chunk_rows > 8 ? 2 : 1) * (slabs * 4 * kBlk * 16 + slabs * chains * 128);
}

bool qmv_wt_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t chunk_rows) {
  // one activation unit per thread while staging: K / 8 <= threads (8 waves: K <= 4096, 16 waves: K <= 8192);
  // group size 32 runs chunks of 8 rows only
  if (!(chunk_rows == 8 || (chunk_rows == 16 && group_size == 64))) return false;
  const uint32_t max_k = chunk_rows > 8 ? 8192u : 4096u;
  return (group_size == 64 || group_size == 32) && N % 16 == 0 && K % 512 == 0 && N > 0 && K > 0 && K <= max_k &&
         wt_lds_bytes(K, group_size, chunk_rows) <= 160 * 1024;
}

int32_t launch_qmv_wt(const QmvArgs& a, uint32_t chunk_rows, hipStream_t s) {
  const uint32_t gs = a.group_size == 0 ? 64 : a.group_size;
  if (!qmv_wt_supported(a.N, a.K, gs, chunk_rows))
    return fail(RMLX_INVALID_SHAPE, "qmv_wt: N %% 16, K %% 512, K <= %u and group size 64 (8-row chunks: or 32) required (N=%u K=%u group_size=%u)",
                chunk_rows > 8 ? 8192u : 4096u, a.N, a.K, gs);
  WtParams p{};
  p.w0 = a.w0; p.s0 = a.s0; p.b0 = a.b0;
  p.w1 = a.dual ? a.w1 : a.w0; p.s1 = a.dual ? a.s1 : a.s0; p.b1 = a.dual ? a.b1 : a.b0;
  p.x = a.x; p.row_map = a.row_map; p.chunk_tab = a.chunk_tab; p.n_chunks = a.n_chunks_dev;
  p.out = a.out; p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  p.K = a.K; p.ld_out = a.ld_out; p.M = a.M; p.out_f32 = a.out_f32;
  p.n_tiles = a.N / 16;
  p.rows_per_expert = a.N;
  const bool tab = a.chunk_tab != nullptr;
  const uint32_t chunks = tab ? a.max_chunks : (a.M + chunk_rows - 1) / chunk_rows;
  if (chunks == 0) return RMLX_OK;
  // 16-row chunks: the fused gate / up kernel needs more than the 128 registers of a 16-wave workgroup, so it runs 8
  // waves (its LDS images leave room for one workgroup per CU either way)
  const uint32_t rh = chunk_rows > 8 ? 2 : 1, nw = rh == 2 && !a.dual ? 16 : 8;
  const size_t lds = wt_lds_bytes(a.K, gs, chunk_rows);
  // tiles per wave: as many as leave about four workgroups per slot of the chip (a workgroup stages the chunk's
  // activations once for all of them)
  const uint64_t slots = (uint64_t)ctx().num_cus * (rh == 2 ? 1 : 2);  // resident workgroups
  uint32_t tpw = 1;
  for (uint32_t c : {4u, 3u, 2u})
    if ((uint64_t)chunks * ((p.n_tiles + nw * c - 1) / (nw * c)) >= 4 * slots) { tpw = c; break; }
  p.tiles_per_wg = nw * tpw;
  const dim3 grid((p.n_tiles + p.tiles_per_wg - 1) / p.tiles_per_wg, chunks);
  int32_t st;
  // (ring depths measured on the routed block at T = 32 / 128: a third set for the fused kernel 317 / 438 us against
  // 306 / 424 us with two; passes of two slabs in a ring of four or three for the plain kernel 263 / 261 us against 255 us
  // with passes of four in a ring of two.  The 16-row fused kernel runs one workgroup per CU either way and has the
  // registers for passes of four slabs: 329 against 370 us at T = 128, while two, three or four sets of two-slab passes
  // all take 370 to 375 us - the size of a pass matters, the depth of the ring does not)
  if (gs == 32) st = a.dual ? launch_one<1, 8, true, 2, 2, 2>(p, tab, grid, lds, s) : launch_one<1, 8, false, 2, 2, 2>(p, tab, grid, lds, s);
  else if (rh == 2) st = a.dual ? launch_one<2, 8, true, 4, 2>(p, tab, grid, lds, s) : launch_one<2, 16, false, 4, 2>(p, tab, grid, lds, s);
  else st = a.dual ? launch_one<1, 8, true, 2, 2>(p, tab, grid, lds, s) : launch_one<1, 8, false, 4, 2>(p, tab, grid, lds, s);
  RMLX_TRY(st);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

bool qmv_wt_combine_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t top_k) {
  return group_size == 64 && N % 16 == 0 && K % 512 == 0 && N > 0 && K > 0 && K <= 4096 && top_k >= 1 && top_k <= 8;
}

int32_t launch_qmv_wt_combine(const uint32_t* w, const __half* s, const __half* b, uint64_t expert_stride_w,
                              uint64_t expert_stride_s, uint32_t n_experts, const __half* h, const uint32_t* idx,
                              const float* wts, uint32_t T, uint32_t top_k, uint32_t N, uint32_t K, __half* out,
                              hipStream_t stream) {
  if (!qmv_wt_combine_supported(N, K, 64, top_k))
    return fail(RMLX_INVALID_SHAPE, "qmv_wt_combine: N %% 16, K %% 512, K <= 4096 and top_k <= 8 required (N=%u K=%u top_k=%u)", N, K, top_k);
  if (T == 0) return RMLX_OK;
  if (T > 65535) return fail(RMLX_INVALID_SHAPE, "qmv_wt_combine: at most 65535 tokens per launch (T=%u)", T);
  WcParams p{w, s, b, h, idx, wts, out, K, N, top_k, n_experts, expert_stride_w, expert_stride_s};
  const uint32_t S = K >> 7;
  const size_t lds = 8 * ((size_t)S * 4 * 5 * 16 + (size_t)S * 2 * 2 * sizeof(float)) + 8 * 16 * sizeof(float);
  static bool configured = false;
  if (!configured) {
    RMLX_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(qmv_wt_combine_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    configured = true;
  }
  hipLaunchKernelGGL(qmv_wt_combine_kernel<4>, dim3(N / 16, T), dim3(512), lds, stream, p);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
