// Quantized GEMM for gfx950, batches that fill the chip only with small tiles (M from about 20 to 150 rows at N = 4096):
// 32 x 64 tiles with K split four ways inside the workgroup.
//
// Replaces the reference's affine_qmm_steel4sg_splitk_q4 + steel_splitk_reduce and affine_qmm_nax_q4 at M = 128
// (crates/rmlx-core/src/ops/quantized.rs:4572-4786, 6927-7103, 3331-3565).
//
// With few activation rows a launch is as long as one workgroup's k loop: a dependent chain of loads, LDS traffic and a
// barrier per 128-wide k block, which no amount of idle matrix units shortens.  The register-weights GEMM (qmm_rw.hip)
// walks all of K in one wave per SIMD at M = 128 (32 blocks at K = 4096), or splits K over workgroups and pays a second
// launch for the reduction.  Here the split sits inside the workgroup:
//   * Tile = 32 activation rows x 64 weight rows; eight waves = 2 column groups (32 weight rows each) x 4 quarters of K.
//     Wave (cg, kq) multiplies its 32 weight rows by the 32 activation rows over the k blocks kq*S/4 .. (kq+1)*S/4 - 1:
//     a quarter of the k loop, eight 32x32x16 MFMAs per block in two independent accumulators.
//   * Every quarter has its own two-stage LDS ring of activation chunks (32 rows x 128 k), staged by the quarter's two
//     waves: global -> registers (four sets, requested five blocks ahead) -> LDS in the operand order of qmm_k2.hip
//     (slot order of the nibble unpacking, xor-swizzled).  Weights go 2 x 16 bytes per lane and block straight into a
//     register ring four blocks deep and are dequantised word by word into the MFMA operand; scales and biases ride along
//     as one word per row and block.
//   * One barrier per block that waits for LDS traffic only (the loads requested ahead stay in flight).
//   * At the end the four quarters meet in LDS (32 KB of f32 partial sums, added in quarter order: deterministic) and the
//     store applies the fused epilogue.  No workspace, no second launch.
#include <type_traits>

#include "common.hpp"
#include "q4_stream.hpp"

namespace rmlx {
namespace {

using q4::u4;
using q4::f4;
using q4::h8;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int kTileM = 32, kTileN = 64, kBlockK = 128, kThreads = 512, kRing = 4;

struct K4Params {
  const uint32_t* w; const __half* s; const __half* b;
  const void* w_packed;  // tile-contiguous copy of w (PACKED builds; the layout of qmm_k2.hip), or null
  const __half* x;  // [M,K] row-major f16 (bf16 bits when XBF16)
  __half* out;
  uint32_t M, N, K, tiles_m, tiles_n;
  int32_t epi_kind, epi_dtype;
  const void* epi;
};

__device__ __forceinline__ uint32_t h2bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// 8 Q4 values of one word -> f16 weights in slot order (k0,k4,k1,k5,k2,k6,k3,k7): exact int -> f16 through the magic
// numbers 1024 + q and 64 + q, then w = s*q + b in packed f16
__device__ __forceinline__ h8 dequant_word(uint32_t w, h2 s2, h2 b2, const q4::Q4Consts& c) {
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

// LDS slot (16 bytes) of activation unit (row R < 32 of the tile, segment seg = 8 consecutive k of the block) inside a
// stage of 512 slots.  Segment seg = 8 kh + 4 hh + ks is read in k step (kh, ks) by lane half hh: a contiguous 1 KB run
// per (kh, ks), which the xor keeps a permutation while spreading the 16 segments of a row over all banks.
__device__ __forceinline__ uint32_t act_slot(uint32_t R, uint32_t seg) {
  return ((seg >> 3) * 4 + (seg & 3)) * 64 + (((((seg >> 2) & 1) << 5) | R) ^ seg);
}

template <bool XBF16, bool PACKED>
__global__ __launch_bounds__(kThreads) void qmm_k4_kernel(const K4Params p) {
  __shared__ u4 lds[4096];  // 64 KB: four quarters x two stages x 8 KB; the first 32 KB again for the final reduction

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), cg = wave & 1, kq = wave >> 1;
  const uint32_t r = lane & 31, hh = lane >> 5;

  // workgroup -> tile: ids go round-robin over the 8 XCDs (one L2 each); every XCD gets a compact block of tiles
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
  const uint32_t K = p.K, S = K / kBlockK, Sq = S / 4, G = K / 64;
  const uint32_t row_lo = mt * kTileM;
  const uint32_t blk0 = kq * Sq;  // first k block of this wave's quarter

  // addresses: buffer resources (uniform base + byte range) + one 32-bit byte offset per thread; the per-block part is
  // uniform and rides in the scalar offset operand.  Reads past a resource's range return zero (rows past M).
  auto make_rsrc = [](const void* base, uint64_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : bytes), 0x00020000);
  };
  const uint32_t row_bytes = K / 2;
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x + (uint64_t)row_lo * K, (uint64_t)(p.M - row_lo) * K * 2);
  // (PACKED: this tile is half of a 128-row tile of the packed layout - column groups 2 (nt % 2) + cg - whose k blocks are
  // runs of 8 KB: (column group, k half, lane) x 16 bytes)
  const __amdgpu_buffer_rsrc_t wr = PACKED
      ? make_rsrc(static_cast<const char*>(p.w_packed) + (uint64_t)(nt >> 1) * 128 * row_bytes, (uint64_t)128 * row_bytes)
      : make_rsrc(p.w + (uint64_t)nt * kTileN * (row_bytes / 4), (uint64_t)kTileN * row_bytes);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc(p.s + (uint64_t)nt * kTileN * G, (uint64_t)kTileN * G * 2);
  const __amdgpu_buffer_rsrc_t br = make_rsrc(p.b + (uint64_t)nt * kTileN * G, (uint64_t)kTileN * G * 2);
  // activations: the quarter's 128 threads stage its chunk: unit q*128 + qt -> (row 8 q + qt/16, segment qt%16)
  const uint32_t qt = cg * 64 + lane, seg = qt & 15, R0 = qt >> 4;
  uint32_t xoff[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) xoff[q] = ((R0 + 8 * q) * K + seg * 8) * 2;
  const uint32_t lds_q = kq * 1024;                // this quarter's two stages (512 slots each)
  uint32_t lds_wq[4];                              // unit q: row R0 + 8 q
#pragma unroll
  for (int q = 0; q < 4; ++q) lds_wq[q] = act_slot(R0 + 8 * q, seg);
  // operand reads of k step (kh, ks)
  uint32_t lds_r[2][4];
#pragma unroll
  for (int kh = 0; kh < 2; ++kh)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) lds_r[kh][ks] = (kh * 4 + ks) * 64 + (((hh << 5) | r) ^ (8 * kh + 4 * hh + ks));
  // weights: row nt*64 + 32 cg + r; this lane's values of a block are words 8 kh + 4 hh .. + 3 of the row's 16
  const uint32_t woff = PACKED ? (((2 * (nt & 1) + cg) * 2) * 64 + lane) * 16 : (32 * cg + r) * row_bytes + hh * 16;
  const uint32_t soff = (32 * cg + r) * G * 2;

  f16v acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

  u4 ra[kRing][4];      // activation chunks in flight (global -> registers -> LDS): requested five blocks ahead
  u4 wq[kRing][2];      // weights, four blocks ahead: [slot][k half]
  u4 s_cur, b_cur, s_nxt, b_nxt;  // (scale, scale) and (bias, bias) words of four blocks: word u = block it0 + u

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
    return q4::permute_x8(v);
  };
  auto load_a = [&](uint32_t it, u4 (&dst)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) dst[q] = __builtin_amdgcn_raw_buffer_load_b128(xr, xoff[q], (blk0 + it) * (kBlockK * 2), 0);
  };
  auto store_a = [&](uint32_t stage, const u4 (&src)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) lds[lds_q + stage * 512 + lds_wq[q]] = to_slot_order(src[q]);
  };
  // scales and biases of the four blocks it0 .. it0 + 3: 16 bytes per row (a word per block and row would touch the same
  // 32 cache lines once per block, and the lines of a workgroup's 64 rows x 4 quarters x 2 do not stay in the CU's L1)
  auto load_sb = [&](uint32_t it0, u4& ds, u4& db) {
    ds = __builtin_amdgcn_raw_buffer_load_b128(sr, soff, (blk0 + it0) * 4, 0);
    db = __builtin_amdgcn_raw_buffer_load_b128(br, soff, (blk0 + it0) * 4, 0);
  };
  // weights of the two blocks it, it + 1 (it even) into ring slots u, u + 1: the four loads cover the lane's 4 x 16 bytes
  // of one 128-byte line per row and are issued back to back, so the line comes up from L2 once (requested a block
  // apart, the second half found the line evicted again: the workgroup's 256 weight rows and its activation chunks
  // together exceed the CU's L1)
  auto load_w2 = [&](uint32_t it, int u) {
    const uint32_t blk = blk0 + it;
    if (PACKED) {
      wq[u][0] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 8192, 0);
      wq[u][1] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 8192 + 1024, 0);
      wq[u + 1][0] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 8192 + 8192, 0);
      wq[u + 1][1] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 8192 + 9216, 0);
    } else {
      wq[u][0] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 64, 0);
      wq[u][1] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 64 + 32, 0);
      wq[u + 1][0] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 64 + 64, 0);
      wq[u + 1][1] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, blk * 64 + 96, 0);
    }
  };
  q4::Q4Consts dq{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(dq.m0), "+s"(dq.m1), "+v"(dq.k0), "+v"(dq.k1));
  auto word_of = [](const u4& v, int c) { return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w)); };

  // ---- prologue: chunk 0 in LDS, chunks 1 and 2 in the register sets, weights of blocks 0..3 requested ---------------
  // (a quarter has a multiple of four blocks.  Every load is issued unconditionally, with the block index clamped to the
  // quarter's last block where it would run past it: the counts behind every s_waitcnt are then exact, whereas loads under
  // a condition make the compiler wait for all of them, the ones requested ahead included)
  const uint32_t last = Sq - 1;
  auto clampi = [&](uint32_t it) { return it < last ? it : last; };
  // (requested in the order the loop requests them - the chunk five blocks ahead, then the weights four blocks ahead - so
  // that the loop is entered with the same queue of outstanding loads as every later round leaves behind.  The memory
  // counter retires in order: a chunk that is requested before the weights of the same age never waits for them.)
  // (sched_barrier: the compiler's scheduler otherwise regroups the loads, and the wait counts follow its order)
  auto pin = [] { __builtin_amdgcn_sched_barrier(0); };
  load_sb(0, s_cur, b_cur); pin();
  load_a(0, ra[0]); pin();
  load_a(1, ra[1]); pin();
  load_a(2, ra[2]); pin();
  load_w2(0, 0); pin();
  load_a(3, ra[3]); pin();
  store_a(0, ra[0]); pin();
  load_a(clampi(4), ra[0]); pin();
  load_w2(2, 2); pin();
  q4::lds_barrier();

  // Block `it` (ring slot u = it % 4): chunk it sits in stage it % 2; chunk it + 1 goes from its register set into the other
  // stage (nobody reads that one any more: the barrier behind block it - 1), and the set takes chunk it + 5.
  auto block = [&](auto uc, uint32_t it) {
    constexpr int u = decltype(uc)::value;
    constexpr uint32_t st = u & 1, st_nxt = (u + 1) & 1;
    constexpr int set = (u + 1) % kRing;
    store_a(st_nxt, ra[set]);  // (behind the last block: a stage nobody reads any more)
    pin();
    load_a(clampi(it + 5), ra[set]);
    pin();
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      const uint32_t sel = kh ? 0x03020302u : 0x01000100u;
      const uint32_t swd = word_of(s_cur, u), bwd = word_of(b_cur, u);
      const h2 s2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(swd, swd, sel));
      const h2 b2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(bwd, bwd, sel));
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const h8 bf = __builtin_bit_cast(h8, lds[lds_q + st * 512 + lds_r[kh][ks]]);
        const h8 aw = dequant_word(word_of(wq[u][kh], ks), s2, b2, dq);
        acc[kh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aw, bf, acc[kh], 0, 0, 0);
      }
    }
    pin();
    if constexpr (u & 1) {  // (both blocks of the pair are consumed)
      load_w2(clampi(it + kRing - 1), u - 1);
      pin();
    }
    q4::lds_barrier();
  };
  using std::integral_constant;
  for (uint32_t it0 = 0; it0 < Sq; it0 += kRing) {
    load_sb(clampi(it0 + kRing) & ~3u, s_nxt, b_nxt); pin();  // (the next four blocks' scales; past the end: the last four again)
    block(integral_constant<int, 0>{}, it0);
    block(integral_constant<int, 1>{}, it0 + 1);
    block(integral_constant<int, 2>{}, it0 + 2);
    block(integral_constant<int, 3>{}, it0 + 3);
    s_cur = s_nxt; b_cur = b_nxt;
  }

  // ---- the four quarters -> one, and accumulator layout -> rows: through LDS -------------------------------------------
  // A lane holds activation row m = r and weight rows 32 cg + 8 (e/4) + 4 hh + e%4.  Partial [kq][m][16 groups of four
  // weight rows], the group index xor-ed with m % 16 so that a wave's stores (32 rows at a stride of 256 bytes) spread
  // over the banks.  (The last barrier of the k loop has passed: nobody reads a stage any more.)
  float* red = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int eg = 0; eg < 4; ++eg) {
    const uint32_t grp = 8 * cg + 2 * eg + hh;  // weight rows 4 grp .. 4 grp + 3 of the tile
    f4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = acc[0][eg * 4 + e] + acc[1][eg * 4 + e];
    *reinterpret_cast<f4*>(red + ((size_t)(kq * kTileM + r) * 16 + (grp ^ (r & 15))) * 4) = v;
  }
  q4::lds_barrier();
  {  // 32 rows x 16 groups = 512 units of four outputs: one per thread
    const uint32_t m = tid >> 4, gp = tid & 15, grp = gp ^ (m & 15);
    f4 v = *reinterpret_cast<const f4*>(red + ((size_t)m * 16 + gp) * 4);
#pragma unroll
    for (int q = 1; q < 4; ++q) v += *reinterpret_cast<const f4*>(red + ((size_t)(q * kTileM + m) * 16 + gp) * 4);
    const uint32_t row = row_lo + m, col = nt * kTileN + 4 * grp;
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

}  // namespace

bool qmm_k4_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits) {
  // (four quarters of a multiple of four 128-wide blocks each; 4-bit weights at group size 64)
  return group_size == 64 && bits == 4 && N > 0 && K > 0 && N % kTileN == 0 && K % (4 * kRing * kBlockK) == 0;
}

int32_t launch_qmm_k4(const QmmArgs& a, uint32_t group_size, hipStream_t s) {
  if (!qmm_k4_supported(a.N, a.K, group_size, a.bits))
    return fail(RMLX_INVALID_SHAPE, "qmm: the 32 x 64 K-split kernel takes 4-bit weights at group size 64 with N %% 64 == 0 and K %% 2048 == 0 "
                                    "(N=%u K=%u bits=%u group_size=%u)", a.N, a.K, a.bits, group_size);
  if (a.M == 0) return RMLX_OK;
  if (a.x_dtype != RMLX_DTYPE_F16 && a.x_dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_RUNTIME_ERROR, "qmm: f32 activations must be cast to f16 first");
  K4Params p{};
  p.w = a.w; p.s = a.s; p.b = a.b;
  p.w_packed = a.N % 128 == 0 ? a.w_packed : nullptr;
  p.x = static_cast<const __half*>(a.x);
  p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K;
  p.tiles_m = (a.M + kTileM - 1) / kTileM;
  p.tiles_n = a.N / kTileN;
  p.epi_kind = a.epi_kind; p.epi = a.epi; p.epi_dtype = a.epi_dtype;
  if ((uint64_t)p.tiles_m * p.tiles_n > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "qmm: grid too large");
  const dim3 grid(p.tiles_m * p.tiles_n), block(kThreads);
  const bool xb = a.x_dtype == RMLX_DTYPE_BF16;
  if (p.w_packed != nullptr) {
    if (xb) hipLaunchKernelGGL((qmm_k4_kernel<true, true>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((qmm_k4_kernel<false, true>), grid, block, 0, s, p);
  } else {
    if (xb) hipLaunchKernelGGL((qmm_k4_kernel<true, false>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((qmm_k4_kernel<false, false>), grid, block, 0, s, p);
  }
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
