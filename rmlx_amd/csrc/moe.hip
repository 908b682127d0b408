// MoE routing and data-movement kernels for gfx950.
//
//   topk_route_kernel   -- moe_topk_route_f32 (crates/rmlx-core/src/ops/topk_route.rs:212-359)
//   moe_sort_kernel     -- histogram + exclusive scan (moe_prefix_scan_u32, topk_route.rs:373-388)
//                          + the stable token->expert grouping the reference builds on the host
//                          (crates/rmlx-nn/src/moe.rs:1439-1447), done on the device
//   index_gather / scatter_weighted_add / silu_gate / combine
//                       -- crates/rmlx-core/src/ops/moe_kernels.rs:46-223, ops/silu.rs:142-166
#include "common.hpp"
#include "route.hpp"

namespace rmlx {
namespace {

constexpr int kMaxExperts = 1024;  // LDS histogram capacity of the sort kernel

// ---- routing: one wave per token (route.hpp) --------------------------------------------------
// (`lds_idx`: optional copy of the picks in workgroup memory, for a sort fused behind the routing)
__device__ __forceinline__ void route_token(const float* __restrict__ logits, const float* __restrict__ bias,
                                            uint32_t E, uint32_t K, int renorm, uint32_t* __restrict__ out_idx,
                                            float* __restrict__ out_w, uint32_t row, uint32_t lane,
                                            uint32_t* lds_idx) {
  uint32_t my_idx;
  float my_w;
  route::token_picks(logits, bias, E, K, renorm, row, lane, my_idx, my_w);
  if (lane < K) {
    out_idx[(size_t)row * K + lane] = my_idx;
    out_w[(size_t)row * K + lane] = my_w;
    if (lds_idx != nullptr) lds_idx[row * K + lane] = my_idx;
  }
}

__global__ __launch_bounds__(64) void topk_route_kernel(const float* __restrict__ logits,
                                                        const float* __restrict__ bias, uint32_t E,
                                                        uint32_t K, int renorm, uint32_t* __restrict__ out_idx,
                                                        float* __restrict__ out_w) {
  route_token(logits, bias, E, K, renorm, out_idx, out_w, blockIdx.x, threadIdx.x, nullptr);
}

// ---- histogram + scan + stable counting sort, one workgroup --------------------------------
// Deterministic by construction.  Offsets and the chunk table come from block-wide exclusive scans
// of the per-expert counts.  Placement walks the assignments in blocks of 1024: every wave ranks
// its 64 consecutive assignments among themselves (lane l counts the lanes below it with the same
// expert) and leaves its count per expert in LDS; thread e turns the 16 counts of expert e into an
// exclusive prefix over the waves; position = running cursor of the expert + prefix of the wave +
// rank in the wave, so ids of one expert keep their original order (numpy.argsort(kind="stable")).
// Four barriers per block of 1024 ids.
__device__ __forceinline__ uint32_t block_exclusive_scan_1024(uint32_t v, uint32_t* wave_tot, uint32_t* total) {
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t t = __shfl_up(inc, o, 64);
    if ((int)lane >= o) inc += t;
  }
  __syncthreads();  // wave_tot may still be read by a previous scan
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  uint32_t base = 0, all = 0;
  for (uint32_t w = 0; w < 16; ++w) {
    const uint32_t t = wave_tot[w];
    if (w < wave) base += t;
    all += t;
  }
  *total = all;
  return base + inc - v;
}

__global__ __launch_bounds__(1024) void moe_sort_kernel(const uint32_t* __restrict__ idx, uint32_t n_assign,
                                                        uint32_t E, uint32_t top_k, uint32_t* __restrict__ sorted,
                                                        uint32_t* __restrict__ sorted_tok,
                                                        uint32_t* __restrict__ inv, uint32_t* __restrict__ counts,
                                                        uint32_t* __restrict__ offsets,
                                                        uint32_t* __restrict__ chunk_tab,
                                                        uint32_t* __restrict__ n_chunks, uint32_t chunk_rows,
                                                        uint32_t* __restrict__ split_tab, uint32_t* __restrict__ split_n,
                                                        uint32_t split_cap) {
  __shared__ uint32_t cnt[kMaxExperts];
  __shared__ uint32_t cur[kMaxExperts];  // running cursor of every expert
  __shared__ uint32_t wave_tot[16];
  __shared__ uint16_t wcnt[16][kMaxExperts];  // placement: per (wave, expert) counts of a block of 1024 ids
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  cnt[tid] = 0;  // kMaxExperts == blockDim.x
#pragma unroll
  for (int w = 0; w < 16; ++w) wcnt[w][tid] = 0;
  __syncthreads();
  for (uint32_t i = tid; i < n_assign; i += 1024) {
    const uint32_t e = idx[i];
    if (e < E) atomicAdd(&cnt[e], 1u);
  }
  __syncthreads();
  // thread e owns expert e: offsets, counts, its chunks of at most chunk_rows rows
  const uint32_t my_cnt = tid < E ? cnt[tid] : 0u;
  uint32_t total_rows, total_chunks;
  const uint32_t my_off = block_exclusive_scan_1024(my_cnt, wave_tot, &total_rows);
  const uint32_t my_chunks = (my_cnt + chunk_rows - 1) / chunk_rows;
  const uint32_t my_chunk0 = block_exclusive_scan_1024(my_chunks, wave_tot, &total_chunks);
  cur[tid] = my_off;
  if (tid < E) {
    if (offsets != nullptr) offsets[tid] = my_off;
    if (counts != nullptr) counts[tid] = my_cnt;
    if (chunk_tab != nullptr) {
      for (uint32_t c = 0; c < my_chunks; ++c) {
        chunk_tab[3 * (my_chunk0 + c) + 0] = tid;
        chunk_tab[3 * (my_chunk0 + c) + 1] = my_off + chunk_rows * c;
        chunk_tab[3 * (my_chunk0 + c) + 2] = my_cnt - chunk_rows * c < chunk_rows ? my_cnt - chunk_rows * c : chunk_rows;
      }
    }
  }
  if (tid == 0) {
    if (offsets != nullptr) offsets[E] = total_rows;
    if (n_chunks != nullptr) *n_chunks = total_chunks;
  }
  // A second pair of tables that splits the experts by their row count: up to 8 rows -> one chunk in the first table
  // (split_cap entries), more -> chunks of at most 16 rows in the second (behind the first); split_n = the two lengths.
  if (split_tab != nullptr) {
    uint32_t n_small, n_big;
    const uint32_t small = my_cnt >= 1 && my_cnt <= 8 ? 1u : 0u, big = my_cnt > 8 ? (my_cnt + 15) / 16 : 0u;
    const uint32_t small0 = block_exclusive_scan_1024(small, wave_tot, &n_small);
    const uint32_t big0 = block_exclusive_scan_1024(big, wave_tot, &n_big);
    if (small) {
      split_tab[3 * small0 + 0] = tid;
      split_tab[3 * small0 + 1] = my_off;
      split_tab[3 * small0 + 2] = my_cnt;
    }
    uint32_t* bt = split_tab + 3 * (size_t)split_cap;
    for (uint32_t c = 0; c < big; ++c) {
      bt[3 * (big0 + c) + 0] = tid;
      bt[3 * (big0 + c) + 1] = my_off + 16 * c;
      bt[3 * (big0 + c) + 2] = my_cnt - 16 * c < 16 ? my_cnt - 16 * c : 16;
    }
    if (tid == 0) { split_n[0] = n_small; split_n[1] = n_big; }
  }
  if (sorted == nullptr) return;

  const int e_bits = 32 - __builtin_clz(E | 1u);  // bits that tell valid expert ids apart
  const uint64_t lanes_below = (1ull << lane) - 1ull;
  uint32_t e_next = tid < n_assign ? idx[tid] : 0xFFFFFFFFu;
  for (uint32_t base = 0; base < n_assign; base += 1024) {
    const uint32_t e = e_next;
    e_next = base + 1024 + tid < n_assign ? idx[base + 1024 + tid] : 0xFFFFFFFFu;  // in flight during this block
    const bool valid = e < E;
    // rank among the wave's 64 assignments, and how many of them share the expert: the lanes holding the same
    // expert are the intersection, over the bits of the id, of the lanes that agree with this one on that bit
    uint64_t peers = __ballot(valid);
    for (int bit = 0; bit < e_bits; ++bit) {
      const uint64_t set = __ballot((e >> bit) & 1u);
      peers &= ((e >> bit) & 1u) ? set : ~set;
    }
    const uint32_t rank = (uint32_t)__popcll(peers & lanes_below), same_total = (uint32_t)__popcll(peers);
    // assignments of (wave, expert) in this block -> exclusive prefix over the waves, per expert
    if (valid && rank + 1 == same_total) wcnt[wave][e] = (uint16_t)same_total;
    __syncthreads();
    uint32_t run = 0;
    if (tid < E) {
#pragma unroll
      for (int w = 0; w < 16; ++w) {
        const uint32_t c = wcnt[w][tid];
        wcnt[w][tid] = (uint16_t)run;
        run += c;
      }
    }
    __syncthreads();
    if (valid) {
      const uint32_t pos = cur[e] + wcnt[wave][e] + rank;
      sorted[pos] = base + tid;
      if (sorted_tok != nullptr) sorted_tok[pos] = (base + tid) / top_k;
      if (inv != nullptr) inv[base + tid] = pos;
    } else if (inv != nullptr && base + tid < n_assign) {
      inv[base + tid] = 0xFFFFFFFFu;  // an expert id outside [0, E): the combine step skips the assignment
    }
    __syncthreads();
    // thread t owns column t of wcnt and cur[t]: cursor forward, column cleared for the next block
    cur[tid] += run;
#pragma unroll
    for (int w = 0; w < 16; ++w) wcnt[w][tid] = 0;
    __syncthreads();
  }
}

// At most 64 assignments (decode-sized batches): one wave, no barriers.  Lane i owns assignment i; ranks,
// offsets and chunk positions are counted with readlane loops over the other lanes.  Same outputs as above.
__device__ __forceinline__ void sort_small(uint32_t lane, uint32_t n, uint32_t e, uint32_t E, uint32_t top_k,
                                           uint32_t* __restrict__ sorted, uint32_t* __restrict__ sorted_tok,
                                           uint32_t* __restrict__ inv, uint32_t* __restrict__ counts,
                                           uint32_t* __restrict__ offsets, uint32_t* __restrict__ chunk_tab,
                                           uint32_t* __restrict__ n_chunks) {
  const bool valid = e < E;  // (lanes past the n assignments hold an invalid expert)
  uint32_t rank = 0, same = 0, less = 0, n_valid = 0;
  for (int j = 0; j < (int)n; ++j) {
    const uint32_t ej = (uint32_t)__builtin_amdgcn_readlane((int)e, j);
    if (ej >= E) continue;  // uniform
    ++n_valid;
    same += ej == e ? 1u : 0u;
    rank += (ej == e && j < (int)lane) ? 1u : 0u;
    less += ej < e ? 1u : 0u;
  }
  const uint32_t pos = less + rank;
  if (valid && sorted != nullptr) {
    sorted[pos] = lane;
    if (sorted_tok != nullptr) sorted_tok[pos] = lane / top_k;
    if (inv != nullptr) inv[lane] = pos;
  }
  if (!valid && lane < n && inv != nullptr) inv[lane] = 0xFFFFFFFFu;  // skipped by the combine step
  // the first assignment of every expert writes the expert's chunks; chunks of lower experts come first
  const bool leader = valid && rank == 0;
  const uint32_t my_chunks = leader ? (same + 7) / 8 : 0u;
  uint32_t chunks_before = 0, total_chunks = 0;
  for (int j = 0; j < (int)n; ++j) {
    const uint32_t cj = (uint32_t)__builtin_amdgcn_readlane((int)my_chunks, j);
    if (cj == 0) continue;  // uniform
    const uint32_t ej = (uint32_t)__builtin_amdgcn_readlane((int)e, j);
    total_chunks += cj;
    chunks_before += ej < e ? cj : 0u;
  }
  if (leader && chunk_tab != nullptr) {
    for (uint32_t c = 0; c < my_chunks; ++c) {
      chunk_tab[3 * (chunks_before + c) + 0] = e;
      chunk_tab[3 * (chunks_before + c) + 1] = less + 8 * c;
      chunk_tab[3 * (chunks_before + c) + 2] = same - 8 * c < 8u ? same - 8 * c : 8u;
    }
  }
  if (lane == 0 && n_chunks != nullptr) *n_chunks = total_chunks;
  if (counts != nullptr || offsets != nullptr) {
    for (uint32_t ee = lane; ee < E; ee += 64) {
      uint32_t c = 0, o = 0;
      for (int j = 0; j < 64; ++j) {
        const uint32_t ej = (uint32_t)__builtin_amdgcn_readlane((int)e, j);
        c += ej == ee ? 1u : 0u;
        o += ej < ee ? 1u : 0u;
      }
      if (counts != nullptr) counts[ee] = c;
      if (offsets != nullptr) offsets[ee] = o;
    }
    if (lane == 0 && offsets != nullptr) offsets[E] = n_valid;
  }
}

__global__ __launch_bounds__(64) void moe_sort_small_kernel(const uint32_t* __restrict__ idx, uint32_t n_assign,
                                                            uint32_t E, uint32_t top_k, uint32_t* __restrict__ sorted,
                                                            uint32_t* __restrict__ sorted_tok,
                                                            uint32_t* __restrict__ inv, uint32_t* __restrict__ counts,
                                                            uint32_t* __restrict__ offsets,
                                                            uint32_t* __restrict__ chunk_tab,
                                                            uint32_t* __restrict__ n_chunks) {
  const uint32_t lane = threadIdx.x;
  sort_small(lane, n_assign, lane < n_assign ? idx[lane] : 0xFFFFFFFFu, E, top_k, sorted, sorted_tok, inv, counts, offsets,
             chunk_tab, n_chunks);
}

// Routing and grouping of a decode-sized batch in one launch: at most 8 tokens and 64 assignments.  Wave t
// routes token t and leaves its picks in workgroup memory; after the barrier wave 0 sorts them.
__global__ __launch_bounds__(512) void route_sort_small_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ bias, uint32_t T, uint32_t E,
                                                               uint32_t K, int renorm, uint32_t* __restrict__ out_idx,
                                                               float* __restrict__ out_w, uint32_t* __restrict__ sorted,
                                                               uint32_t* __restrict__ sorted_tok,
                                                               uint32_t* __restrict__ inv,
                                                               uint32_t* __restrict__ chunk_tab,
                                                               uint32_t* __restrict__ n_chunks) {
  __shared__ uint32_t picks[64];
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave < T) route_token(logits, bias, E, K, renorm, out_idx, out_w, wave, lane, picks);
  __syncthreads();
  if (wave == 0)
    sort_small(lane, T * K, lane < T * K ? picks[lane] : 0xFFFFFFFFu, E, K, sorted, sorted_tok, inv, nullptr, nullptr,
               chunk_tab, n_chunks);
}

__global__ void index_gather_kernel(const __half* __restrict__ src, uint32_t d, const uint32_t* __restrict__ idx,
                                    uint32_t src_rows, __half* __restrict__ dst) {
  const uint32_t i = blockIdx.x;
  const uint32_t r = idx[i];
  for (uint32_t c = threadIdx.x; c < d; c += blockDim.x)
    dst[(size_t)i * d + c] = r < src_rows ? src[(size_t)r * d + c] : __float2half(0.f);
}

// One workgroup per destination row: assignments are visited in ascending order, so the f32
// sum of a row is reproducible.
__global__ void scatter_weighted_add_kernel(const __half* __restrict__ src, uint32_t n, uint32_t d,
                                            const uint32_t* __restrict__ tok, const float* __restrict__ w,
                                            __half* __restrict__ dst) {
  const uint32_t t = blockIdx.x;
  for (uint32_t c = threadIdx.x; c < d; c += blockDim.x) {
    float acc = __half2float(dst[(size_t)t * d + c]);
    for (uint32_t i = 0; i < n; ++i)
      if (tok[i] == t) acc += w[i] * __half2float(src[(size_t)i * d + c]);
    dst[(size_t)t * d + c] = __float2half(acc);
  }
}

__global__ void silu_gate_kernel(const __half* __restrict__ g, const __half* __restrict__ u,
                                 __half* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const float x = __half2float(g[i]);
    out[i] = __float2half(x / (1.0f + __expf(-x)) * __half2float(u[i]));
  }
}

// out[r, c] = silu(g[r*ld + c]) * u[r*ld + c]: gate and up halves of one [rows, ld] matrix
__global__ void silu_gate_strided_kernel(const __half* __restrict__ g, const __half* __restrict__ u, uint32_t ld,
                                         __half* __restrict__ out, uint32_t rows, uint32_t cols) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x, n = (size_t)rows * cols;
  for (; i < n; i += stride) {
    const size_t r = i / cols, c = i % cols;
    const float x = __half2float(g[r * ld + c]);
    out[i] = __float2half(x / (1.0f + __expf(-x)) * __half2float(u[r * ld + c]));
  }
}

// assignments in their own order: token of assignment a is a / top_k, its position is a
__global__ void identity_positions_kernel(uint32_t* __restrict__ tok, uint32_t* __restrict__ inv, uint32_t n, uint32_t top_k) {
  const uint32_t a = blockIdx.x * blockDim.x + threadIdx.x;
  if (a < n) {
    tok[a] = a / top_k;
    inv[a] = a;
  }
}

// out[t,:] = sum_k w[t*K+k] * y[inv[t*K+k],:], k ascending, f32.  grid = (T, column blocks of 1024):
// every thread owns four columns, loads its rows of all top_k experts first and sums in order.
// Assignments whose position is not below n_rows (the grouping kernels mark an expert id outside
// [0, E) that way) contribute nothing.
// (YT: the expert outputs as f32, or as f16 where the projection left them so)
__device__ __forceinline__ float4 load_four(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load_four(const __half* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  const float2 lo = __half22float2(*reinterpret_cast<const __half2*>(&r.x)), hi = __half22float2(*reinterpret_cast<const __half2*>(&r.y));
  return make_float4(lo.x, lo.y, hi.x, hi.y);
}
template <typename YT>
__global__ __launch_bounds__(256) void moe_combine_kernel(const YT* __restrict__ y,
                                                          const uint32_t* __restrict__ inv,
                                                          const float* __restrict__ weights, uint32_t top_k,
                                                          uint32_t D, uint32_t n_rows, __half* __restrict__ out) {
  const uint32_t t = blockIdx.x;
  const uint32_t c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= D) return;
  float w[8];
  float4 v[8];
#pragma unroll
  for (uint32_t k = 0; k < 8; ++k) {
    w[k] = 0.f;
    v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (k < top_k) {
      const uint32_t pos = inv[(size_t)t * top_k + k];
      if (pos < n_rows) {
        w[k] = weights[(size_t)t * top_k + k];
        v[k] = load_four(y + (size_t)pos * D + c);
      }
    }
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (uint32_t k = 0; k < 8; ++k) {
    if (k < top_k) { acc.x += w[k] * v[k].x; acc.y += w[k] * v[k].y; acc.z += w[k] * v[k].z; acc.w += w[k] * v[k].w; }
  }
  const __half2 lo = __floats2half2_rn(acc.x, acc.y), hi = __floats2half2_rn(acc.z, acc.w);
  uint2 o;
  o.x = *reinterpret_cast<const uint32_t*>(&lo);
  o.y = *reinterpret_cast<const uint32_t*>(&hi);
  *reinterpret_cast<uint2*>(out + (size_t)t * D + c) = o;
}

// The same sum over f16 rows in assignment order (no grouping: row t*K+k is pick k of token t): out[t,:] = sum_k
// w[t*K+k] * y[t*K+k,:], k ascending, f32; an assignment whose expert id lies outside [0, E) contributes nothing.
__global__ __launch_bounds__(256) void moe_combine_rows_f16_kernel(const __half* __restrict__ y,
                                                                   const uint32_t* __restrict__ idx,
                                                                   const float* __restrict__ weights, uint32_t top_k,
                                                                   uint32_t D, uint32_t E, __half* __restrict__ out) {
  const uint32_t t = blockIdx.x;
  const uint32_t c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= D) return;
  float w[8];
  uint2 v[8];
#pragma unroll
  for (uint32_t k = 0; k < 8; ++k) {
    w[k] = 0.f;
    v[k] = make_uint2(0u, 0u);
    if (k < top_k) {
      const size_t a = (size_t)t * top_k + k;
      if (idx[a] < E) {
        w[k] = weights[a];
        v[k] = *reinterpret_cast<const uint2*>(y + a * D + c);
      }
    }
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (uint32_t k = 0; k < 8; ++k) {
    if (k < top_k) {
      const float2 lo = __half22float2(*reinterpret_cast<const __half2*>(&v[k].x)), hi = __half22float2(*reinterpret_cast<const __half2*>(&v[k].y));
      acc.x += w[k] * lo.x; acc.y += w[k] * lo.y; acc.z += w[k] * hi.x; acc.w += w[k] * hi.y;
    }
  }
  const __half2 lo = __floats2half2_rn(acc.x, acc.y), hi = __floats2half2_rn(acc.z, acc.w);
  uint2 o;
  o.x = *reinterpret_cast<const uint32_t*>(&lo);
  o.y = *reinterpret_cast<const uint32_t*>(&hi);
  *reinterpret_cast<uint2*>(out + (size_t)t * D + c) = o;
}

}  // namespace

int32_t launch_topk_route(const float* logits, const float* bias, uint32_t T, uint32_t E, uint32_t K,
                          int renorm, uint32_t* idx, float* w, uint32_t* counts, uint32_t* offsets,
                          hipStream_t s) {
  if (T > 0) {
    hipLaunchKernelGGL(topk_route_kernel, dim3(T), dim3(64), 0, s, logits, bias, E, K, renorm, idx, w);
    RMLX_HIP_CHECK(hipGetLastError());
  }
  if ((counts != nullptr || offsets != nullptr) && T * K <= 64 && E <= (uint32_t)kMaxExperts) {
    hipLaunchKernelGGL(moe_sort_small_kernel, dim3(1), dim3(64), 0, s, idx, T * K, E, K, (uint32_t*)nullptr,
                       (uint32_t*)nullptr, (uint32_t*)nullptr, counts, offsets, (uint32_t*)nullptr,
                       (uint32_t*)nullptr);
    RMLX_HIP_CHECK(hipGetLastError());
  } else if (counts != nullptr || offsets != nullptr) {
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, s, idx, T * K, E, K, (uint32_t*)nullptr,
                       (uint32_t*)nullptr, (uint32_t*)nullptr, counts, offsets, (uint32_t*)nullptr,
                       (uint32_t*)nullptr, 8u, (uint32_t*)nullptr, (uint32_t*)nullptr, 0u);
    RMLX_HIP_CHECK(hipGetLastError());
  }
  return RMLX_OK;
}

bool route_sort_fusable(uint32_t T, uint32_t E, uint32_t K) {
  return T >= 1 && T <= 8 && T * K <= 64 && E <= 256 && K >= 1 && K <= 8;
}

int32_t launch_route_sort_small(const float* logits, const float* bias, uint32_t T, uint32_t E, uint32_t K,
                                int renorm, uint32_t* idx, float* w, uint32_t* sorted, uint32_t* sorted_tok,
                                uint32_t* inv, uint32_t* chunk_tab, uint32_t* n_chunks, hipStream_t s) {
  if (!route_sort_fusable(T, E, K)) return fail(RMLX_RUNTIME_ERROR, "route_sort_small: T=%u E=%u K=%u not supported", T, E, K);
  hipLaunchKernelGGL(route_sort_small_kernel, dim3(1), dim3(64 * T), 0, s, logits, bias, T, E, K, renorm, idx, w, sorted,
                     sorted_tok, inv, chunk_tab, n_chunks);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_moe_sort(const uint32_t* idx, uint32_t n_assign, uint32_t E, uint32_t top_k, uint32_t* sorted,
                        uint32_t* sorted_tok, uint32_t* inv, uint32_t* counts, uint32_t* offsets,
                        uint32_t* chunk_tab, uint32_t* n_chunks, uint32_t chunk_rows, hipStream_t s, uint32_t* split_tab,
                        uint32_t* split_n, uint32_t split_cap) {
  if (E > (uint32_t)kMaxExperts)
    return fail(RMLX_INVALID_SHAPE, "moe_sort: n_experts (%u) exceeds maximum %d", E, kMaxExperts);
  if (chunk_rows == 0) return fail(RMLX_RUNTIME_ERROR, "moe_sort: chunk_rows must be non-zero");
  if (n_assign <= 64 && chunk_rows == 8 && split_tab == nullptr)  // the one-wave kernel writes chunks of 8 rows
    hipLaunchKernelGGL(moe_sort_small_kernel, dim3(1), dim3(64), 0, s, idx, n_assign, E, top_k ? top_k : 1u, sorted,
                       sorted_tok, inv, counts, offsets, chunk_tab, n_chunks);
  else
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, s, idx, n_assign, E, top_k ? top_k : 1u, sorted,
                       sorted_tok, inv, counts, offsets, chunk_tab, n_chunks, chunk_rows, split_tab, split_n, split_cap);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_index_gather(const __half* src, uint32_t d, const uint32_t* idx, uint32_t n, uint32_t src_rows,
                            __half* dst, hipStream_t s) {
  if (n == 0 || d == 0) return RMLX_OK;
  hipLaunchKernelGGL(index_gather_kernel, dim3(n), dim3(256), 0, s, src, d, idx, src_rows, dst);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_scatter_weighted_add(const __half* src, uint32_t n, uint32_t d, const uint32_t* tok,
                                    const float* w, __half* dst, uint32_t dst_rows, hipStream_t s) {
  if (n == 0 || d == 0 || dst_rows == 0) return RMLX_OK;
  hipLaunchKernelGGL(scatter_weighted_add_kernel, dim3(dst_rows), dim3(256), 0, s, src, n, d, tok, w, dst);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_silu_gate(const __half* g, const __half* u, __half* out, size_t n, hipStream_t s) {
  if (n == 0) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(silu_gate_kernel, dim3((unsigned)blocks), dim3(256), 0, s, g, u, out, n);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_silu_gate_strided(const __half* g, const __half* u, uint32_t ld, __half* out, uint32_t rows,
                                 uint32_t cols, hipStream_t s) {
  const size_t n = (size_t)rows * cols;
  if (n == 0) return RMLX_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(silu_gate_strided_kernel, dim3((unsigned)blocks), dim3(256), 0, s, g, u, ld, out, rows, cols);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_identity_positions(uint32_t* tok, uint32_t* inv, uint32_t n, uint32_t top_k, hipStream_t s) {
  if (n == 0) return RMLX_OK;
  hipLaunchKernelGGL(identity_positions_kernel, dim3((n + 255) / 256), dim3(256), 0, s, tok, inv, n, top_k);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_moe_combine(const float* y, const uint32_t* inv, const float* weights, uint32_t T, uint32_t top_k,
                           uint32_t D, __half* out, hipStream_t s) {
  if (T == 0) return RMLX_OK;
  if (top_k > 8 || D % 4 != 0) return fail(RMLX_INVALID_SHAPE, "moe_combine: top_k <= 8 and D %% 4 == 0 required (top_k=%u D=%u)", top_k, D);
  hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(T, (D + 1023) / 1024), dim3(256), 0, s, y, inv, weights, top_k, D, T * top_k, out);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

// The same over f16 expert outputs (the products are summed in f32 as above).
int32_t launch_moe_combine_f16(const __half* y, const uint32_t* inv, const float* weights, uint32_t T, uint32_t top_k,
                               uint32_t D, __half* out, hipStream_t s) {
  if (T == 0) return RMLX_OK;
  if (top_k > 8 || D % 4 != 0) return fail(RMLX_INVALID_SHAPE, "moe_combine: top_k <= 8 and D %% 4 == 0 required (top_k=%u D=%u)", top_k, D);
  hipLaunchKernelGGL(moe_combine_kernel<__half>, dim3(T, (D + 1023) / 1024), dim3(256), 0, s, y, inv, weights, top_k, D, T * top_k, out);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

int32_t launch_moe_combine_rows_f16(const __half* y, const uint32_t* idx, const float* weights, uint32_t T, uint32_t top_k,
                                    uint32_t D, uint32_t E, __half* out, hipStream_t s) {
  if (T == 0) return RMLX_OK;
  if (top_k > 8 || D % 4 != 0) return fail(RMLX_INVALID_SHAPE, "moe_combine: top_k <= 8 and D %% 4 == 0 required (top_k=%u D=%u)", top_k, D);
  hipLaunchKernelGGL(moe_combine_rows_f16_kernel, dim3(T, (D + 1023) / 1024), dim3(256), 0, s, y, idx, weights, top_k, D, E, out);
  RMLX_HIP_CHECK(hipGetLastError());
  return RMLX_OK;
}

}  // namespace rmlx
