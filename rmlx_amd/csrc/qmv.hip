// Streaming quantized GEMV family for gfx950: qmv (M <= 8 rows per pass), gather_qmm and the
// two MoE expert projections (fused gate/up + SwiGLU, down).
//
// Replaces the reference's affine_qmv_fast_f16_q4 / affine_qmv_batched_f16_q4 /
// gather_qmv_fast_f16_q4 (crates/rmlx-core/src/ops/quantized.rs:798-979, 9752-9842).
//
// Design (wave64, MFMA):
//   * A workgroup is 8 independent waves.  Wave w owns weight tile (w / KS) of the workgroup's
//     NT tiles of 16 rows and k-part (w % KS) of the pass, NT * KS = 8: K >= 4096 gives one tile
//     split 8 ways (512 k per wave and pass of 4096 k); smaller K gives several tiles per
//     workgroup (K = 1536: two tiles x four parts of 384 k), so a workgroup always streams a
//     sizeable block of weights.  Waves only meet in the final reduction.
//   * Every lane issues all of its 128-bit weight loads of a pass up front, after the few small
//     loads (activations, scales, biases): the memory counter retires in order, so the small
//     ones can be consumed while the bulk is still in flight.
//   * A "slab" is 16 rows x 128 k.  Lane (n = lane%16, g = lane/16) loads the 16 bytes holding
//     k in [32g, 32g+32) of row n; its four u32 words feed four v_mfma_f32_16x16x32_f16
//     (word j -> k = 32g + 8j + 0..7), weights as the B operand so that the accumulator lane
//     keeps column n.
//   * Nibbles are turned into f16 with mask-or only: (w & 0x000F000F) | 0x64006400 is the pair
//     (1024+q0, 1024+q4), (w & 0x00F000F0) | 0x54005400 is (64+q1, 64+q5).  The constant
//     offsets are removed exactly with -sum(off_k * x_k) per (row, group); the k order inside a
//     word (0,4,1,5,2,6,3,7) is matched by permuting x when it is staged into LDS.
//   * The two quantisation groups of a slab (group size 64) must be scaled separately.  With at
//     most 8 activation rows, accumulator rows 0-7 receive x restricted to the first group and
//     rows 8-15 the same x restricted to the second group (the other half of the A operand is
//     zero), so one accumulator tile yields both per-group integer dot products.  Each is then
//     folded into the f32 result with  acc += scale * (dot - sum(off*x)) + bias * sum(x).
//   * Each wave stages exactly the activations it consumes (wave-private LDS, no barrier).  The
//     per-(row, group) sums sum(x) and sum(off*x) come from the matrix unit too: one extra MFMA per
//     product against a constant operand (computed once per workgroup where one pass covers K).
//   * The kernel is bound by instruction issue before it is bound by memory (a wave moves 4 KB of
//     weights per tile): operand lanes whose rows are empty read a zero slot instead of being masked,
//     the unpacking constants sit in registers (and + or = one instruction), the two group halves
//     meet through v_permlane32_swap, and the operand reads of a tile are scheduled slab by slab
//     (low register count: up to three workgroups per CU).
//   * Barriers of the tile reduction wait for LDS traffic only, and a workgroup that walks several
//     tiles requests the next tile's weights as soon as the current accumulators have left for LDS.
#include "common.hpp"
#include "q4_stream.hpp"

namespace rmlx {
namespace {

using namespace q4;

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kSpwMax = 4;  // slabs (128 k) per wave per pass

// Field order matters: the first 16 dwords are preloaded into SGPRs at wave launch
// (-amdgpu-kernarg-preload-count), so everything the plain qmv path needs comes first.
struct KParams {
  const uint32_t* w0;
  const __half* s0;
  const __half* b0;
  const __half* x;
  void* out;
  uint32_t K, ld_out, M, out_f32;
  uint32_t ks;  // k-parts per pass (1, 2, 4 or 8); tiles per workgroup = 8 / ks
  uint32_t gs128;  // quantisation group size 128 instead of 64
  uint32_t tpw;  // consecutive tiles per workgroup (> 1 only when one pass covers K: the staged activations are reused)
  const uint32_t* w1;
  const __half* s1;
  const __half* b1;
  const uint32_t* row_map;
  const uint32_t* chunk_tab;
  const uint32_t* n_chunks;
  uint64_t estride_w, estride_s;
  uint32_t x_bf16;  // x holds bf16 bits: converted to f16 while the activations are staged
};



// MR = activation rows staged per pass (1, 2, 4 or 8); TILES = 1, or 2 (fused gate/up, or two
// 16-row tiles of one matrix sharing the staged activations: PAIR);
// TAB = rows come from a device chunk table (gather_qmm, MoE); SPW = slabs per wave and pass when
// every wave of every pass owns the same number (3 or 4: no guards, fewer registers, two
// workgroups per CU), 0 = decided at run time.
// REUSE != 0: one pass covers K, so the activations are staged once, before the tile loop; 2 = with fewer than
// 8 rows, the next tile's weights are loaded into a second register set while the current tile is multiplied
// (for workgroups that take several tiles; a workgroup with one tile keeps the registers for a third resident
// workgroup per CU);
// before the tile loop (their registers are free again when the weight loads start).
template <int MR, int TILES, bool TAB, int SPW, bool PAIR, int REUSE>
__global__ __launch_bounds__(kThreads, (REUSE != 0 && MR == 8 && TILES == 2) ? 4 : 1) void qmv_q4_kernel(KParams p) {
  static_assert(!REUSE || SPW != 0, "reuse needs a uniform slab count");
  static_assert(!PAIR || TILES == 2, "paired tiles need two tile slots");
  constexpr int kSlots = 4 * MR;                       // 16-byte activation slots per (slab, j) block ...
  constexpr int kBlk = kSlots + 1;                     // ... followed by one slot of zeros (read by the lanes whose operand rows are empty)
  constexpr int kXsWave = kSpwMax * 4 * kBlk * 16;     // bytes of activation image per wave
  __shared__ __attribute__((aligned(16))) char xs_all[kWaves * kXsWave];
  __shared__ float red[kWaves * TILES * 8 * 16];  // cross-wave reduction: [wave][tile][activation row][column]
  // Activation sums per (row, group) come from the matrix unit (see 2b).  With one pass over K they are computed
  // once, before the tile loop, and wait in LDS; otherwise every pass computes them beside its products.
  constexpr bool kPreSums = REUSE != 0;
  __shared__ __attribute__((aligned(16))) float sums_all[!kPreSums ? 4 : kWaves * kSpwMax * 2 * 8 * 2];  // [wave][group][row][-xoff, xsum]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (in a scalar register, with everything derived from it)
  const int n = lane & 15;   // weight row within the tile / accumulator column
  const int g = lane >> 4;   // k sub-block of the slab / accumulator row group
  const int par = g >> 1;    // which of the slab's two quantisation groups this lane scales
  char* xs = xs_all + wave * kXsWave;
  float* sums = sums_all + (!kPreSums ? 0 : wave * (kSpwMax * 2 * 8 * 2));

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

  // ---- which weights: tile tw of this workgroup, k-part kp of every pass --------------------
  const uint32_t K = p.K, KS = p.ks, NT = kWaves / KS;
  const uint32_t kp = wave % KS, tw = wave / KS;
  // group size 128 (p.gs128): one scale per slab, applied to both halves of it
  const uint32_t words_per_row = K >> 3, groups_per_row = p.gs128 ? K >> 7 : K >> 6, slabs_total = K >> 7;
  constexpr bool pair = PAIR;
  const uint32_t rows_per_slot = pair ? 32u : 16u;  // weight rows (of one matrix) per wave tile slot

  uint32_t srcs[MR];  // source rows of the activations (wave-uniform)
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    srcs[m] = row0 + m;
    if (TAB && p.row_map != nullptr && (uint32_t)m < rows) srcs[m] = p.row_map[row0 + m];
  }

  // A-operand activity: accumulator rows 0-7 take group 0 (g<2), rows 8-15 group 1 (g>=2).
  const int am = n & 7;
  const bool a_active = ((n < 8) == (g < 2)) && (am < MR);
  const int a_slot_off = (a_active ? g * MR + am : kSlots) * 16;  // the others read the block's zero slot
  if (lane < kSpwMax * 4) *reinterpret_cast<u4*>(xs + (lane * kBlk + kSlots) * 16) = (u4){0u, 0u, 0u, 0u};
  Q4Consts qc{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(qc.m0), "+s"(qc.m1), "+v"(qc.k0), "+v"(qc.k1));

  // constant B operand of the activation sums (see 2b)
  const u4 bconst_bits = n < 8 ? (u4){0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u}
                               : (u4){0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  const h8 bconst = __builtin_bit_cast(h8, bconst_bits);

  // activations of a pass: lane l of the wave loads 8 consecutive k of every row (slabs sl .. sl+my-1)
  auto load_x = [&](int sl, int my, u4 (&xv)[MR]) {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      xv[m] = (u4){0u, 0u, 0u, 0u};
      if ((uint32_t)m < rows && lane < my * 16)
        xv[m] = *reinterpret_cast<const u4*>(p.x + (uint64_t)srcs[m] * K + (uint32_t)(sl * 16 + lane) * 8);
    }
  };
  // this wave's activations -> its LDS image in operand order
  auto stage_x = [&](const u4 (&xv)[MR]) {
    const int ls = lane >> 4, gg = (lane >> 2) & 3, j = lane & 3;
    if (p.x_bf16) {  // (wave-uniform; the f16 path pays a scalar compare)
#pragma unroll
      for (int m = 0; m < MR; ++m)
        *reinterpret_cast<u4*>(xs + ((ls * 4 + j) * kBlk + gg * MR + m) * 16) = permute_x8(bf16x8_to_f16(xv[m]));
      return;
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
      *reinterpret_cast<u4*>(xs + ((ls * 4 + j) * kBlk + gg * MR + m) * 16) = permute_x8(xv[m]);
  };
  auto stage_sums = [&]() {
    if constexpr (kPreSums) {
      // sums of the staged activations, once for all tiles: accumulator row 4g+j of column 0 holds sum(off*x), of
      // column 8 sum(x) (see 2b); rows 0-7 are the activation rows of the slab's first group, rows 8-15 of its second
#pragma unroll
      for (int it = 0; it < SPW; ++it) {
        f4 own = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const h8 av = *reinterpret_cast<const h8*>(xs + ((it * 4 + j) * kBlk) * 16 + a_slot_off);
          own = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bconst, own, 0, 0, 0);
        }
        // per (slab, group, half of the rows): -sum(off*x) of the four rows, then their sum(x)
        float* sp = sums + ((it * 2 + par) * 8 + (g & 1) * 4) * 2;
        if (n == 0) *reinterpret_cast<f4*>(sp) = -own;
        if (n == 8) *reinterpret_cast<f4*>(sp + 4) = own;
      }
    }
  };

  // ---- tiles of this workgroup: consecutive, so it streams one contiguous block of weight rows.
  //      With one pass over K the activation image (and the sums) staged for the first tile serve
  //      all of them.
  const uint32_t ntiles = REUSE ? p.tpw : 1u;  // (without reuse the launcher gives every workgroup one tile)
  // every global load of one tile's slabs sl .. sl+my-1: scales / biases first (the memory counter retires in order)
  auto load_tile = [&](uint32_t wg_tile, int sl, int my, u4 (&sbv)[TILES], u4 (&wreg)[TILES][kSpwMax]) {
    const uint32_t tile_row = (wg_tile * NT + tw) * rows_per_slot;
    const u4* wrow[TILES];
    const __half* sbrow[TILES];
    // (the lane's part of the addresses is recomputed per tile on purpose: kept across the tile loop it costs
    // registers the 8-row kernels do not have)
    uint32_t lane_l = lane;
    asm volatile("" : "+v"(lane_l));
    const uint32_t n = lane_l & 15, g = lane_l >> 4;
  #pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const uint64_t e_w = TAB ? expert * p.estride_w : 0, e_s = TAB ? expert * p.estride_s : 0;
      const bool first = t == 0 || pair;                       // which matrix
      const uint32_t wr = tile_row + n + (pair ? 16 * t : 0);  // which row of it
      wrow[t] = reinterpret_cast<const u4*>((first ? p.w0 : p.w1) + e_w + (uint64_t)wr * words_per_row) + g;
      // scales live in the lanes with even g, biases in the lanes with odd g (exchanged later)
      const __half* sb = (g & 1) ? (first ? p.b0 : p.b1) : (first ? p.s0 : p.s1);
      sbrow[t] = sb + e_s + (uint64_t)wr * groups_per_row;
    }
    // sbv word `it` = (group 2*it, group 2*it+1) of slab sl+it: scales or biases, by lane
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      sbv[t] = (u4){0u, 0u, 0u, 0u};
      if (p.gs128) {  // four slabs = four halves; word `it` holds slab it's value twice
        const unsigned short* hp = reinterpret_cast<const unsigned short*>(sbrow[t]) + sl;
        const uint32_t h0 = my > 0 ? hp[0] : 0u, h1 = my > 1 ? hp[1] : 0u, h2 = my > 2 ? hp[2] : 0u, h3 = my > 3 ? hp[3] : 0u;
        sbv[t] = (u4){h0 | (h0 << 16), h1 | (h1 << 16), h2 | (h2 << 16), h3 | (h3 << 16)};
        continue;
      }
      const uint32_t* sp = reinterpret_cast<const uint32_t*>(sbrow[t]) + sl;
      if (my == kSpwMax) {  // 4 slabs: one 16-byte load (4-byte aligned is enough for the hardware)
        const U4Unaligned v = *reinterpret_cast<const U4Unaligned*>(sp);
        sbv[t] = (u4){v.v[0], v.v[1], v.v[2], v.v[3]};
      } else {
        if (my > 0) sbv[t].x = sp[0];
        if (my > 1) sbv[t].y = sp[1];
        if (my > 2) sbv[t].z = sp[2];
      }
    }
#pragma unroll
    for (int it = 0; it < kSpwMax; ++it) {
      if (it < my) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) wreg[t][it] = *(wrow[t] + (sl + it) * 4);
      }
    }
  };
  // The lane's half of every scale / bias word (the group `par` of each slab it multiplies), two slabs per register:
  // one byte permute per two slabs replaces a shift, a mask and a select per slab, the exchange between the lanes
  // that loaded scales and those that loaded biases moves two registers instead of four, and the halves are
  // consumed as f16 operands of mixed-precision fmas.
  const uint32_t half_sel = par ? 0x07060302u : 0x05040100u;
  auto pick_halves = [&](const u4& v, uint32_t (&sv)[2], uint32_t (&bv)[2]) {
    const uint32_t own0 = __builtin_amdgcn_perm(v.y, v.x, half_sel), own1 = __builtin_amdgcn_perm(v.w, v.z, half_sel);
    const uint32_t oth0 = swap16(own0), oth1 = swap16(own1);
    sv[0] = (g & 1) ? oth0 : own0; sv[1] = (g & 1) ? oth1 : own1;
    bv[0] = (g & 1) ? own0 : oth0; bv[1] = (g & 1) ? own1 : oth1;
  };
  auto half_at = [](const uint32_t (&o)[2], int it) -> float {
    const uint32_t wd = o[it >> 1];
    const unsigned short h = (it & 1) ? (unsigned short)(wd >> 16) : (unsigned short)(wd & 0xFFFFu);
    return (float)__builtin_bit_cast(_Float16, h);
  };
  // the tile's slabs against the staged activations: F += scale * (dot - sum(off*x)) + bias * sum(x)
  auto compute_tile = [&](int my, const u4 (&sbv)[TILES], const u4 (&wreg)[TILES][kSpwMax], f4 (&F)[TILES]) {
    // Slab by slab (few live registers).  The per (row, group) sums of the activations come from the matrix
    // unit: columns 0-7 of a constant B operand hold the unpack offsets (1024 for even k, 64 for odd k, in slot
    // order), columns 8-15 hold ones, so accumulator column n < 8 receives sum(off*x) and column n >= 8 sum(x)
    // of its rows; lane n^8 holds the other one.
    uint32_t sv[TILES][2], bv[TILES][2];
#pragma unroll
    for (int t = 0; t < TILES; ++t) pick_halves(sbv[t], sv[t], bv[t]);
    if constexpr (kPreSums) {
      // ---- one pass over K: the sums wait in LDS ----
#pragma unroll
      for (int it = 0; it < kSpwMax; ++it) {
        if (it < my) {
          // the accumulators start from -sum(off*x) of their rows, so the chain ends in dot - sum(off*x)
          const float* sp = sums + ((it * 2 + par) * 8 + (g & 1) * 4) * 2;
          const f4 negoff = *reinterpret_cast<const f4*>(sp);    // accumulator rows 4g .. 4g+3
          const f4 xsum = *reinterpret_cast<const f4*>(sp + 4);
          f4 c[TILES];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const h8 av = *reinterpret_cast<const h8*>(xs + ((it * 4 + j) * kBlk) * 16 + a_slot_off);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
              const uint32_t wd = j == 0 ? wreg[t][it].x : (j == 1 ? wreg[t][it].y : (j == 2 ? wreg[t][it].z : wreg[t][it].w));
              c[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, unpack_q4_word(wd, qc), j == 0 ? negoff : c[t], 0, 0, 0);
            }
          }
#pragma unroll
          for (int t = 0; t < TILES; ++t) {
            const float sc = half_at(sv[t], it), bi = half_at(bv[t], it);
#pragma unroll
            for (int i = 0; i < 4; ++i) F[t][i] = fmaf(sc, c[t][i], fmaf(bi, xsum[i], F[t][i]));
          }
          // (keeps the operand reads of later slabs from being hoisted above this one: they would cost the registers
          // that let a third workgroup share the CU)
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
      // ---- several passes over K: every pass computes the sums beside its products ----
#pragma unroll
      for (int it = 0; it < kSpwMax; ++it) {
        if (it < my) {
          f4 own = (f4){0.f, 0.f, 0.f, 0.f};
          f4 c[TILES];
#pragma unroll
          for (int t = 0; t < TILES; ++t) c[t] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const h8 av = *reinterpret_cast<const h8*>(xs + ((it * 4 + j) * kBlk) * 16 + a_slot_off);
            own = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bconst, own, 0, 0, 0);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
              const uint32_t wd = j == 0 ? wreg[t][it].x : (j == 1 ? wreg[t][it].y : (j == 2 ? wreg[t][it].z : wreg[t][it].w));
              c[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, unpack_q4_word(wd, qc), c[t], 0, 0, 0);
            }
          }
          const float o0 = swap8(own.x), o1 = swap8(own.y), o2 = swap8(own.z), o3 = swap8(own.w);
#pragma unroll
          for (int t = 0; t < TILES; ++t) {
            const float sc = half_at(sv[t], it), bi = half_at(bv[t], it);
            const float ce = n < 8 ? -sc : bi, co = n < 8 ? bi : -sc;
            F[t][0] = fmaf(sc, c[t][0], fmaf(ce, own.x, fmaf(co, o0, F[t][0])));
            F[t][1] = fmaf(sc, c[t][1], fmaf(ce, own.y, fmaf(co, o1, F[t][1])));
            F[t][2] = fmaf(sc, c[t][2], fmaf(ce, own.z, fmaf(co, o2, F[t][2])));
            F[t][3] = fmaf(sc, c[t][3], fmaf(ce, own.w, fmaf(co, o3, F[t][3])));
          }
        }
      }
    }
  };
  // ---- 4. reduce over the two group halves (lane + 32 holds the other one) and over the
  //         k-parts, write out.  In two steps, so that a tile loop can request the next tile's weights
  //         between them, when the accumulators are free again. ----------------------------------------
  auto reduce_halves = [&](f4 (&F)[TILES]) {
  lds_barrier();  // the previous tile's sums have been read
  // (index arithmetic of this part is kept inside the tile loop on purpose: hoisted out, it
  // costs registers for the whole kernel)
  uint32_t tid_t = tid;
  asm volatile("" : "+v"(tid_t));
  {
    const uint32_t lane_t = tid_t & 63, wave_t = tid_t >> 6, n_t = lane_t & 15, g_t = lane_t >> 4;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = add_other_half(F[t][i]);
        if (g_t < 2) red[((wave_t * TILES + t) * 8 + g_t * 4 + i) * 16 + n_t] = v;
      }
  }
  };
  auto reduce_parts_and_store = [&](uint32_t wg_tile) {
  lds_barrier();
  uint32_t tid_t = tid;
  asm volatile("" : "+v"(tid_t));
  for (uint32_t o = tid_t; o < NT * 128; o += kThreads) {
    const uint32_t otw = o >> 7, m = (o >> 4) & 7, nn = o & 15;
    if (m < rows) {
      float v[TILES];
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        float acc = 0.f;
        if (KS == 8) {  // (four reads in flight at a time instead of a chain of eight)
#pragma unroll
          for (uint32_t q = 0; q < 8; q += 4) {
            const float* rp = red + ((q * TILES + t) * 8 + m) * 16 + nn;
            const float r0 = rp[0], r1 = rp[TILES * 128], r2 = rp[2 * TILES * 128], r3 = rp[3 * TILES * 128];
            acc += (r0 + r1) + (r2 + r3);
          }
        } else {
          for (uint32_t q = 0; q < KS; ++q) acc += red[(((otw * KS + q) * TILES + t) * 8 + m) * 16 + nn];
        }
        v[t] = acc;
      }
      const uint64_t obase = (uint64_t)(row0 + m) * p.ld_out + (wg_tile * NT + otw) * rows_per_slot + nn;
      if (TILES == 2 && !pair) v[0] = silu_f(v[0]) * v[TILES - 1];
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        if (t == 0 || pair) {
          const float r = write_zeros ? 0.f : v[t];
          if (p.out_f32) reinterpret_cast<float*>(p.out)[obase + 16 * t] = r;
          else reinterpret_cast<__half*>(p.out)[obase + 16 * t] = __float2half(r);
        }
      }
    }
  }
  };
  auto finish_tile = [&](uint32_t wg_tile, f4 (&F)[TILES], bool) {
    reduce_halves(F);
    reduce_parts_and_store(wg_tile);
  };

  if constexpr (REUSE == 1 && MR < 8) {
    // one pass, one tile per workgroup (the launcher gives these kernels no more): straight-line code, which keeps
    // the registers low enough for a third resident workgroup per CU
    const int sl = (int)(kp * SPW);
    u4 sbv[TILES];
    u4 wreg[TILES][kSpwMax];
    {
      u4 xv[MR];
      load_x(sl, SPW, xv);
      load_tile(blockIdx.x, sl, SPW, sbv, wreg);
      stage_x(xv);
      stage_sums();
    }
    f4 F[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
    compute_tile(SPW, sbv, wreg, F);
    finish_tile(blockIdx.x, F, true);
  } else if constexpr (REUSE == 1) {
    // one pass: slabs kp*SPW .. of every tile; the activations and the first tile's weights are requested together.
    // One register set for the weights (eight rows: a second one would cost the second workgroup per CU, which
    // hides more latency than it; measured): the next tile's weights are requested as soon as the products of the
    // current tile have consumed the registers and the accumulators are on their way through LDS, and arrive while
    // the partial sums are added up and written.
    const int sl = (int)(kp * SPW);
    const uint32_t first = blockIdx.x * ntiles;
    u4 sbv[TILES];
    u4 wreg[TILES][kSpwMax];
    {
      u4 xv[MR];
      load_x(sl, SPW, xv);
      // (two tiles: their first weights do not fit beside the activations in the registers of four waves per SIMD)
      if constexpr (TILES == 1) load_tile(first, sl, SPW, sbv, wreg);
      stage_x(xv);
      if constexpr (TILES == 2) load_tile(first, sl, SPW, sbv, wreg);
      stage_sums();
    }
    for (uint32_t ti = 0; ti < ntiles; ++ti) {
      f4 F[TILES];
#pragma unroll
      for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
      compute_tile(SPW, sbv, wreg, F);
      reduce_halves(F);
      if (ti + 1 < ntiles) load_tile(first + ti + 1, sl, SPW, sbv, wreg);
      reduce_parts_and_store(first + ti);
    }
  } else if constexpr (REUSE == 2) {  // fewer rows, several tiles: the weights of the next tile are in flight while this one is multiplied
    const int sl = (int)(kp * SPW);
    u4 sbv_a[TILES], sbv_b[TILES];
    u4 wreg_a[TILES][kSpwMax], wreg_b[TILES][kSpwMax];
    const uint32_t first = blockIdx.x * ntiles;
    {
      u4 xv[MR];
      load_x(sl, SPW, xv);
      load_tile(first, sl, SPW, sbv_a, wreg_a);
      stage_x(xv);
      stage_sums();
    }
    for (uint32_t ti = 0; ti < ntiles; ti += 2) {
      f4 F[TILES];
      if (ti + 1 < ntiles) load_tile(first + ti + 1, sl, SPW, sbv_b, wreg_b);
#pragma unroll
      for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
      compute_tile(SPW, sbv_a, wreg_a, F);
      finish_tile(first + ti, F, ti == 0);
      if (ti + 1 < ntiles) {
        if (ti + 2 < ntiles) load_tile(first + ti + 2, sl, SPW, sbv_a, wreg_a);
#pragma unroll
        for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
        compute_tile(SPW, sbv_b, wreg_b, F);
        finish_tile(first + ti + 1, F, false);
      }
    }
  } else {
    const uint32_t wg_tile = blockIdx.x;
    f4 F[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) F[t] = (f4){0.f, 0.f, 0.f, 0.f};
    for (uint32_t slab0 = 0; slab0 < slabs_total; slab0 += KS * kSpwMax) {
      const uint32_t ns = slabs_total - slab0 < KS * kSpwMax ? slabs_total - slab0 : KS * kSpwMax;  // slabs of this pass
      const int spw = SPW ? SPW : (int)((ns + KS - 1) / KS);
      const int sl = (int)(slab0 + kp * spw);       // first slab of this wave
      int my_rt = (int)ns - (int)(kp * spw);
      my_rt = my_rt < 0 ? 0 : (my_rt > spw ? spw : my_rt);
      const int my = SPW ? SPW : my_rt;
      u4 xv[MR];
      load_x(sl, my, xv);
      u4 sbv[TILES];
      u4 wreg[TILES][kSpwMax];
      load_tile(wg_tile, sl, my, sbv, wreg);
      stage_x(xv);
      compute_tile(my, sbv, wreg, F);
    }
    finish_tile(wg_tile, F, true);
  }
}

template <int MR, int TILES, int SPW, bool PAIR>
void launch_s(const KParams& p, bool tab, dim3 grid, hipStream_t s) {
  if constexpr (SPW != 0) {
    if (p.K / 128 == p.ks * SPW) {  // one pass over K: the kernels that stage the activations once
      constexpr int kPipe = MR < 8 ? 2 : 1;
      if (p.tpw > 1) {
        if (tab) hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, true, SPW, PAIR, kPipe>), grid, dim3(kThreads), 0, s, p);
        else hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, false, SPW, PAIR, kPipe>), grid, dim3(kThreads), 0, s, p);
      } else {
        if (tab) hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, true, SPW, PAIR, 1>), grid, dim3(kThreads), 0, s, p);
        else hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, false, SPW, PAIR, 1>), grid, dim3(kThreads), 0, s, p);
      }
      return;
    }
  }
  if (tab) hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, true, SPW, PAIR, 0>), grid, dim3(kThreads), 0, s, p);
  else hipLaunchKernelGGL((qmv_q4_kernel<MR, TILES, false, SPW, PAIR, 0>), grid, dim3(kThreads), 0, s, p);
}

template <int MR, int TILES, bool PAIR = false>
void launch_t(const KParams& p, bool tab, dim3 grid, hipStream_t s) {
  // uniform slab count per wave and pass?
  const uint32_t slabs = p.K / 128, per_pass = p.ks * kSpwMax;
  int spw = 0;
  if (slabs % per_pass == 0) spw = 4;
  else if (slabs < per_pass && slabs % p.ks == 0 && slabs / p.ks == 3) spw = 3;
  if (spw == 4) launch_s<MR, TILES, 4, PAIR>(p, tab, grid, s);
  else if (spw == 3) launch_s<MR, TILES, 3, PAIR>(p, tab, grid, s);
  else launch_s<MR, TILES, 0, PAIR>(p, tab, grid, s);
}

__global__ void build_gather_chunks_kernel(const uint32_t* indices, uint32_t batch, uint32_t mpb,
                                           uint32_t n_experts, uint32_t chunk_rows, uint32_t* chunk_tab,
                                           uint32_t* n_chunks) {
  const uint32_t per = (mpb + chunk_rows - 1) / chunk_rows;
  const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= batch * per) return;
  if (c == 0 && n_chunks != nullptr) *n_chunks = batch * per;
  const uint32_t b = c / per, r = (c % per) * chunk_rows;
  uint32_t e = indices[b], rows = mpb - r < chunk_rows ? mpb - r : chunk_rows;
  if (e >= n_experts) { e = 0; rows |= 0x80000000u; }
  chunk_tab[3 * c + 0] = e;
  chunk_tab[3 * c + 1] = b * mpb + r;
  chunk_tab[3 * c + 2] = rows;
}

}  // namespace

int32_t launch_build_gather_chunks(const uint32_t* indices, uint32_t batch, uint32_t mpb, uint32_t n_experts,
                                   uint32_t chunk_rows, uint32_t* chunk_tab, uint32_t* n_chunks, hipStream_t s) {
  if (chunk_rows == 0) return fail(RMLX_RUNTIME_ERROR, "gather chunks: chunk_rows must be non-zero");
  const uint32_t n = batch * ((mpb + chunk_rows - 1) / chunk_rows);
  if (n == 0) return RMLX_OK;
  hipLaunchKernelGGL(build_gather_chunks_kernel, dim3((n + 255) / 256), dim3(256), 0, s, indices, batch, mpb,
                     n_experts, chunk_rows, chunk_tab, n_chunks);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}


// K in whole slabs of 128: a wave takes up to four slabs per pass, the last part of a pass may be shorter or empty.
bool qmv_q4_supported(uint32_t N, uint32_t K, uint32_t group_size) {
  return (group_size == 64 || group_size == 128) && N % 16 == 0 && K % 128 == 0 && N > 0 && K > 0;
}

int32_t launch_qmv_q4(const QmvArgs& a, hipStream_t s) {
  if (!qmv_q4_supported(a.N, a.K, 64)) return fail(RMLX_INVALID_SHAPE, "qmv_q4: N %% 16 and K %% 128 required (N=%u K=%u)", a.N, a.K);
  KParams p{};
  p.w0 = a.w0; p.s0 = a.s0; p.b0 = a.b0;
  p.w1 = a.dual ? a.w1 : a.w0; p.s1 = a.dual ? a.s1 : a.s0; p.b1 = a.dual ? a.b1 : a.b0;
  p.x = a.x; p.row_map = a.row_map; p.chunk_tab = a.chunk_tab; p.n_chunks = a.n_chunks_dev;
  p.out = a.out; p.estride_w = a.expert_stride_w; p.estride_s = a.expert_stride_s;
  p.K = a.K; p.ld_out = a.ld_out; p.M = a.M; p.out_f32 = a.out_f32;
  p.gs128 = a.group_size == 128 ? 1u : 0u;
  p.x_bf16 = a.x_bf16 ? 1u : 0u;
  const bool tab = a.chunk_tab != nullptr;
  uint32_t chunks = tab ? a.max_chunks : (a.M + 7) / 8;
  if (chunks == 0) return RMLX_OK;
  // k-parts per pass: 8 for K >= 4096; for smaller K the fewest parts of at most 4 slabs each,
  // the remaining waves take further 16-row tiles (as long as N divides)
  uint32_t ks = 8;
  const uint32_t slabs = a.K / 128;
  if (slabs < 32) {
    ks = 1;
    while (ks * kSpwMax < slabs) ks *= 2;
    while (ks < 8 && a.N % (16 * (8 / ks)) != 0) ks *= 2;
  }
  p.ks = ks;
  int mr = a.mr;
  if (mr == 0) mr = tab ? 8 : (a.M >= 5 ? 8 : (a.M >= 3 ? 4 : (a.M == 2 ? 2 : 1)));
  // With 8 rows every wave takes two tiles (rows r and r+16) for the same staged activations when
  // that still gives every CU a workgroup: the activation traffic and staging work per
  // weight byte halve.
  const uint32_t nt = 8 / ks;
  const bool pair = !a.dual && mr == 8 && a.N % (32 * nt) == 0 &&
                    (uint64_t)(a.N / (32 * nt)) * chunks >= 1ull * (uint32_t)ctx().num_cus;
  // Tiles per workgroup: with one pass over K a workgroup keeps its staged activations for several
  // consecutive tiles (staging 8 rows costs as many bytes as the two tiles it serves), as long as
  // every CU still gets two workgroups.
  const uint32_t tiles_x = a.N / (16 * nt * (pair ? 2 : 1));
  uint32_t tpw = 1;
  const bool uniform_single_pass = slabs == ks * kSpwMax || slabs == ks * 3;  // the kernels with a fixed slab count
  if (uniform_single_pass) {
    // With a chunk table, consecutive chunks often belong to one expert (more than 8 rows): a grid
    // width that is a multiple of the 8 XCDs puts their workgroups for the same tiles on one XCD,
    // next to each other in time, so the second chunk finds the weights in that L2.
    static const uint32_t cand[] = {8, 6, 4, 3, 2};
    for (int pass = tab ? 0 : 1; pass < 2 && tpw == 1; ++pass)
      for (uint32_t c : cand)
        if (tiles_x % c == 0 && (pass == 1 || (tiles_x / c) % 8 == 0) &&
            (uint64_t)(tiles_x / c) * chunks >= 2ull * (uint32_t)ctx().num_cus) { tpw = c; break; }
  }
  p.tpw = tpw;
  dim3 grid(tiles_x / tpw, chunks);
  if (pair) {
    launch_t<8, 2, true>(p, tab, grid, s);
  } else if (a.dual) {
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
