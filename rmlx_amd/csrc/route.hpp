// Routing of one token by one wave, shared by the routing kernels and by the expert projection that routes its own
// token (moe_topk_route_f32, crates/rmlx-core/src/ops/topk_route.rs:212-359).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace rmlx {
namespace route {

// ---- wave-wide reductions on DPP (lane ^ 1, lane ^ 2, the other quad of 8, the other 8 of 16), one
//      swizzle (lane ^ 16) and two readlanes: a fraction of the latency of six LDS shuffles ------------
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float swz16_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
__device__ __forceinline__ float readlane_f32(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f32<0xB1>(v));
  v = fmaxf(v, dpp_f32<0x4E>(v));
  v = fmaxf(v, dpp_f32<0x141>(v));
  v = fmaxf(v, dpp_f32<0x140>(v));
  v = fmaxf(v, swz16_f32(v));
  return fmaxf(readlane_f32(v, 0), readlane_f32(v, 32));
}
__device__ __forceinline__ float wave_add(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  v += swz16_f32(v);
  return readlane_f32(v, 0) + readlane_f32(v, 32);
}
__device__ __forceinline__ uint32_t max_u32(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max_u32(v, dpp_u32<0xB1>(v));
  v = max_u32(v, dpp_u32<0x4E>(v));
  v = max_u32(v, dpp_u32<0x141>(v));
  v = max_u32(v, dpp_u32<0x140>(v));
  v = max_u32(v, (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F));
  return max_u32((uint32_t)__builtin_amdgcn_readlane((int)v, 0), (uint32_t)__builtin_amdgcn_readlane((int)v, 32));
}

// ---- routing: one wave per token -----------------------------------------------------------
// exp(x) for x <= 0 from plain f32 multiplies and adds, each rounded once (no fused multiply-add, no
// hardware transcendental): the same sequence of IEEE operations gives the same bits on any machine, so a
// CPU restatement reproduces the softmax values -- and with them the ties the ranking sees -- exactly.
// Cody-Waite reduction x = n ln2 + r, degree-5 polynomial for (e^r - 1 - r) / r^2, scale by 2^n.  Arguments
// below -80 give 0, which keeps every softmax value (at least e^-80 / 256) a normal number.
__device__ __forceinline__ float exp_neg_exact(float x) {
#pragma clang fp contract(off)
  if (x < -80.0f) return 0.0f;
  const float n = __builtin_rintf(x * 1.44269504f);
  float r = x - n * 0.693359375f;
  r = r - n * -2.12194440e-4f;
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  p = p * (r * r);
  p = p + r;
  p = p + 1.0f;
  return p * __uint_as_float((uint32_t)((int)n + 127) << 23);
}

// Each lane owns experts lane, lane+64, lane+128, lane+192 (E <= 256).  Ranking follows the reference:
// the f32 softmax value exp(l - max) * (1 / sum) with strict >, so equal values (two logits that collapse
// after exp, an underflowing tail) go to the lower expert index (topk_route.rs:283-300).  The sum runs over the
// four values of a lane in ascending order and then over the lanes as a balanced pairwise tree.
// The keys of a token's experts, one wave: lane l receives the keys of experts l, l + 64, l + 128, l + 192.  A key is
// the bits of the expert's non-negative softmax value (order-preserving; -0 counted as +0) plus one, zero for an expert
// index past E.
__device__ __forceinline__ void token_keys(const float* __restrict__ logits, const float* __restrict__ bias, uint32_t E,
                                           uint32_t row, uint32_t lane, uint32_t (&key)[4]) {
  const float NEG_INF = -__builtin_inff();
  float v[4], sm[4];
  float mx = NEG_INF;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t e = lane + 64 * j;
    v[j] = NEG_INF;
    if (e < E) {
      v[j] = logits[(size_t)row * E + e];
      if (bias != nullptr) v[j] += bias[e];
    }
    mx = fmaxf(mx, v[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    sm[j] = (lane + 64 * j < E) ? exp_neg_exact(v[j] - mx) : 0.f;
    sum += sm[j];
  }
  sum = wave_add(sum);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int j = 0; j < 4; ++j) key[j] = lane + 64 * j < E ? __float_as_uint(sm[j] * inv + 0.0f) + 1u : 0u;
}

// Lane k < K leaves with the k-th pick in `my_idx` (0xFFFFFFFF: none left) and its weight in `my_w`.
__device__ __forceinline__ void token_picks(const float* __restrict__ logits, const float* __restrict__ bias, uint32_t E,
                                            uint32_t K, int renorm, uint32_t row, uint32_t lane, uint32_t& my_idx_out,
                                            float& my_w_out) {
  uint32_t key[4];
  token_keys(logits, bias, E, row, lane, key);
  // A round: the wave maximum of the keys, then the lowest expert index that holds it -- slots in ascending j, inside a
  // slot the lowest lane of the ballot; a slot that is taken gets key zero.  Lane k keeps the k-th pick (no register arrays
  // indexed by the round counter).
  float my_w = 0.f;
  uint32_t my_idx = 0xFFFFFFFFu;
  for (uint32_t k = 0; k < K; ++k) {
    const uint32_t top = wave_max_u32(max_u32(max_u32(key[0], key[1]), max_u32(key[2], key[3])));  // uniform
    uint32_t bi = 0xFFFFFFFFu;
    if (top != 0) {
#pragma unroll
      for (int j = 3; j >= 0; --j) {
        const uint64_t holders = __builtin_amdgcn_ballot_w64(key[j] == top);
        if (holders != 0) bi = (uint32_t)__builtin_ctzll(holders) + 64u * j;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (bi == lane + 64 * j) key[j] = 0u;
    if (lane == k) {
      my_idx = bi;
      my_w = top != 0 ? __uint_as_float(top - 1u) : 0.f;
    }
  }
  float scale = 1.0f;
  if (renorm) {
    // sum of the K picks in pick order (lanes 0 .. K-1), the order a serial loop would add them in
    float ws = 0.f;
    for (uint32_t k = 0; k < K; ++k) ws += readlane_f32(my_w, (int)k);
    scale = ws > 0.f ? 1.0f / ws : 0.f;
  }
  my_idx_out = my_idx;
  my_w_out = my_w * scale;
}

// The same picks and weights by a whole workgroup (blockDim.x = 256, 512 or 1024): the first wave makes the
// keys, then every thread counts, for one expert and a share of the others, how many rank before it (larger key, or the
// same key and a lower index): an expert's rank is its place in the sequence of repeated arg-max rounds above, found
// without the rounds' serial chain.  Results in workgroup memory: out_idx[k], out_w[k] for k < K (0xFFFFFFFF / 0 where
// fewer than K experts exist); every thread may read them after the call.  `ws` is workspace of 2 * 256 words.
__device__ __forceinline__ void token_picks_workgroup(const float* __restrict__ logits, const float* __restrict__ bias,
                                                      uint32_t E, uint32_t K, int renorm, uint32_t row, uint32_t* ws,
                                                      uint32_t* out_idx, float* out_w) {
  uint32_t* keys = ws;         // [256]
  uint32_t* rank = ws + 256;   // [256]
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x;
  if (wave == 0) {
    uint32_t key[4];
    token_keys(logits, bias, E, row, lane, key);
#pragma unroll
    for (int j = 0; j < 4; ++j) { keys[lane + 64 * j] = key[j]; rank[lane + 64 * j] = 0u; }
    if (lane < 8) { out_idx[lane] = 0xFFFFFFFFu; out_w[lane] = 0.f; }
  }
  __syncthreads();
  // thread -> (expert i, part): the slots 0 .. ep - 1 (ep = 64, 128 or 256 covers E) are split between the parts of an
  // expert, four keys per LDS read (a wave reads one address: a broadcast)
  uint32_t ep = 64;
  while (ep < E) ep <<= 1;
  const uint32_t parts = nthreads / ep, per = ep / parts;
  if (tid < ep * parts) {
    const uint32_t i = tid & (ep - 1), part = tid / ep, mine = keys[i];
    uint32_t before = 0;
    for (uint32_t j = part * per; j < (part + 1) * per; j += 4) {
      const uint4 k4 = *reinterpret_cast<const uint4*>(keys + j);
      before += (k4.x > mine || (k4.x == mine && j + 0 < i)) ? 1u : 0u;
      before += (k4.y > mine || (k4.y == mine && j + 1 < i)) ? 1u : 0u;
      before += (k4.z > mine || (k4.z == mine && j + 2 < i)) ? 1u : 0u;
      before += (k4.w > mine || (k4.w == mine && j + 3 < i)) ? 1u : 0u;
    }
    if (mine != 0u && before != 0u) atomicAdd(&rank[i], before);
  }
  __syncthreads();
  if (tid < 256) {
    const uint32_t mine = keys[tid], r = rank[tid];
    if (mine != 0u && r < K) { out_idx[r] = tid; out_w[r] = __uint_as_float(mine - 1u); }
  }
  __syncthreads();
  if (renorm) {
    // sum of the K picks in pick order, the order a serial loop would add them in (every thread computes the same)
    float wsum = 0.f;
    for (uint32_t k = 0; k < K; ++k) wsum += out_w[k];
    const float scale = wsum > 0.f ? 1.0f / wsum : 0.f;
    __syncthreads();
    if (tid < K) out_w[tid] = out_w[tid] * scale;
    __syncthreads();
  }
}

}  // namespace route
}  // namespace rmlx
