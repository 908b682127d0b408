// Internal definitions shared by the host-side entry points and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/rmlx_hip.h"

namespace rmlx {

// ---- error channel ---------------------------------------------------------------------
std::string& last_error();
int32_t fail(int32_t code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define RMLX_HIP_CHECK(expr)                                                                  \
  do {                                                                                        \
    hipError_t _e = (expr);                                                                   \
    if (_e != hipSuccess)                                                                     \
      return ::rmlx::fail(RMLX_RUNTIME_ERROR, "%s failed: %s (%s:%d)", #expr,                \
                          hipGetErrorString(_e), __FILE__, __LINE__);                         \
  } while (0)

#define RMLX_TRY(expr)                 \
  do {                                 \
    int32_t _s = (expr);               \
    if (_s != RMLX_OK) return _s;      \
  } while (0)

// `checked_u32` of the reference (crates/rmlx-core/src/ops/mod.rs:71-74).
int32_t checked_u32(size_t v, const char* name, uint32_t* out);

inline size_t dtype_size(int32_t dt) {
  switch (dt) {
    case RMLX_DTYPE_F32: case RMLX_DTYPE_U32: return 4;
    case RMLX_DTYPE_F16: case RMLX_DTYPE_BF16: return 2;
    case RMLX_DTYPE_U8: return 1;
    default: return 0;
  }
}
const char* dtype_name(int32_t dt);
inline size_t numel(const rmlx_array* a) {
  size_t n = 1;
  for (int i = 0; i < a->ndim; ++i) n *= a->shape[i];
  return n;
}

struct DeviceCtx {
  bool ready = false;
  int device = -1;
  int num_cus = 0;
};
DeviceCtx& ctx();
int32_t require_init();

// Finishes a call: synchronous when the caller passed no stream.
int32_t finish(hipStream_t stream);

// Stream-ordered scratch from a per-stream pool (see api.cpp).  Used for dtype casts, the
// re-laid-out activations of the GEMM and the MoE intermediates; the f16 qmv path needs none.
// A caller-provided block that scratch is carved from instead of the pool (entry points that must not allocate).
struct Arena {
  char* base = nullptr;
  size_t capacity = 0, used = 0;
};

struct Scratch {
  void* ptr = nullptr;
  size_t size = 0;
  hipStream_t stream = nullptr;
  bool pooled = false;
  int32_t alloc(size_t bytes, hipStream_t s, Arena* arena = nullptr);
  void release();
  ~Scratch() { release(); }
};

}  // namespace rmlx

// Opaque handle behind rmlx_qweight.
struct rmlx_qweight {
  const uint32_t* w;
  const __half* s;
  const __half* b;
  uint32_t group_size;
  uint32_t bits;
  size_t out_features;  // N (per expert)
  size_t in_features;   // K
  size_t n_experts;     // 1 for a plain linear weight
  // stacked expert weights: average rows per expert from which the expert projections run on the grouped MFMA GEMM
  // instead of the streaming GEMV (read from the gate weight of a block; 0 = never)
  uint32_t expert_gemm_min_rows = 10;
  // stacked expert weights: which streaming kernel runs decode-sized batches (read from the gate weight of a block):
  // 0 = the library's choice, 1 = K split over the waves of a workgroup (qmv.hip), 2 = a wave per tile (qmv_wt.hip)
  uint32_t expert_stream_kernel = 0;
  // optional second copy of the weights in the tile-contiguous order of the K-split GEMMs (rmlx_hip_qweight_set_gemm_layout;
  // the caller owns the buffer); null = none
  const void* gemm_packed = nullptr;
};

namespace rmlx {

// ---- kernel launchers (one translation unit per family) ------------------------------------

// Activation cast to f16 (f32 / bf16 -> f16) or bf16 -> kept; n elements.
int32_t launch_cast_to_f16(const void* src, int32_t src_dtype, __half* dst, size_t n, hipStream_t s);
int32_t launch_cast_f16_to_f32(const __half* src, float* dst, size_t n, hipStream_t s);

// Portable scalar kernel: any bits in {2,3,4,6,8}, any group size; x f16 [M,K] -> out f16 [M,N].
// Optional per-row expert lookup (gather): W/S/B of row-batch b start at expert indices[b].
struct GenericArgs {
  const uint32_t* w; const __half* s; const __half* b;
  const __half* x; __half* out;
  const uint32_t* indices;  // nullable; one expert per `rows_per_index` consecutive x rows
  uint32_t rows_per_index;
  uint32_t M, N, K, group_size, bits, n_experts;
};
int32_t launch_generic(const GenericArgs& a, hipStream_t s);

// Streaming GEMV family (qmv, gather_qmm, MoE expert projections).  Rows are processed in
// chunks of at most 8; `chunk_tab` on the device lists (expert, first row position, row count)
// triples (bit 31 of the count: write zeros instead of computing).
struct QmvArgs {
  const uint32_t* w0; const __half* s0; const __half* b0;  // tile set 0
  const uint32_t* w1; const __half* s1; const __half* b1;  // tile set 1 (fused gate/up only)
  uint32_t N;                // weight rows per expert covered by this launch (multiple of 16)
  uint32_t K;                // multiple of 512
  uint64_t expert_stride_w;  // u32 words per expert
  uint64_t expert_stride_s;  // halves per expert
  const __half* x;           // [x_rows, K] f16
  const uint32_t* row_map;   // nullable: source row of position p is row_map[p]
  void* out;                 // f16 [positions, ld_out] (f32 when out_f32)
  uint32_t ld_out;
  int out_f32;
  int dual;                  // 1: out = silu(tile0 . x) * (tile1 . x)
  const uint32_t* chunk_tab; // nullable -> expert 0, rows [0,M) in chunks of 8
  const uint32_t* n_chunks_dev;  // nullable -> every chunk of the grid is valid
  uint32_t max_chunks;       // grid.y when chunk_tab != null
  uint32_t M;                // used when chunk_tab == null
  uint32_t mr;               // rows staged per chunk (1,2,4,8); 0 -> derive from M
  uint32_t group_size;       // 64 (also when 0) or 128
  // launch_qmv_m1_gate_up without an index list only: the workgroups rank their own token's experts from f32 logits
  // [T, n_experts] (+ optional bias) and also write the picks and normalised weights to route_idx_out / route_w_out
  const float* route_logits; const float* route_bias; uint32_t* route_idx_out; float* route_w_out;
  int32_t route_renorm;
  int32_t x_bf16;  // launch_qmv_m1_gate_up and launch_qmv_q4: x holds bf16 bits, converted to f16 while they are staged
};
int32_t launch_qmv_q4(const QmvArgs& a, hipStream_t s);
bool qmv_q4_supported(uint32_t N, uint32_t K, uint32_t group_size);
// Gate / up projection of single rows through chosen experts (qmv_m1.hip): position a = activation row a / top_k (x, no
// row map) through expert idx[a] (idx == null: pick a % top_k of the ranking the kernel makes itself, see route_logits) of the two stacked matrices of `a` (w0 / w1, expert strides), out[a, :] = silu(gate) * up
// in f16 [assignments, N]; 4- or 8-bit weights, the shapes of the single-row GEMV.  chunk_tab / M / mr of `a` are not used.
bool qmv_m1_gate_up_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
// gather_qmm with one activation row per index on the single-row kernel (qmv_m1.hip): x [batch, K] f16, idx [batch]
// (outside [0, n_experts): zeros), stacked 4- or 8-bit weights with strides in u32 words / halves, out [batch, N] f16;
// the shapes qmv_m1_supported(N, K, group_size, bits) takes
int32_t launch_qmv_m1_gather(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                             uint32_t n_experts, const __half* x, const uint32_t* idx, uint32_t batch, __half* out, uint32_t N,
                             uint32_t K, uint32_t group_size, uint32_t bits, hipStream_t stream,
                             uint32_t rows_per_index = 1);  // batch rows; rows_per_index consecutive rows share idx[row / rows_per_index]
int32_t launch_qmv_m1_gate_up(const QmvArgs& a, uint32_t bits, const uint32_t* idx, uint32_t assignments, uint32_t top_k,
                              uint32_t n_experts, hipStream_t stream);
// Down projection of a few tokens with the weighted combine behind it on the single-row layout (qmv_m1.hip): h
// [T * top_k, K] f16 in assignment order, out[t] = sum_k wts[t, k] * (h[t * top_k + k] . W[idx[t * top_k + k]]^T) in ascending
// k, f16 [T, N]; 8-bit weights, K at most two wave-wide chunks (2048), N % 4 == 0
bool qmv_m1_down_combine_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, uint32_t top_k);
int32_t launch_qmv_m1_down_combine(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                                   uint32_t n_experts, const __half* h, const uint32_t* idx, const float* wts, uint32_t T,
                                   uint32_t top_k, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, __half* out,
                                   hipStream_t stream);
// Wave-per-tile streaming GEMV (qmv_wt.hip): the same arguments; chunks of at most chunk_rows (8 or 16) rows, a wave owns
// a 16-row weight tile over all of K (no cross-wave reduction), group size 64, K <= 4096 (16-row chunks: 8192)
bool qmv_wt_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t chunk_rows);
int32_t launch_qmv_wt(const QmvArgs& a, uint32_t chunk_rows, hipStream_t s);
// Down projection of a few tokens with the weighted combine fused behind it (qmv_wt.hip): h [T * top_k, K] f16 in
// assignment order, out[t] = sum_k wts[t, k] * (h[t * top_k + k] . W[idx[t * top_k + k]]^T) in ascending k, f16 [T, N];
// 4-bit weights, group size 64, K <= 4096
bool qmv_wt_combine_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t top_k);
int32_t launch_qmv_wt_combine(const uint32_t* w, const __half* s, const __half* b, uint64_t expert_stride_w,
                              uint64_t expert_stride_s, uint32_t n_experts, const __half* h, const uint32_t* idx,
                              const float* wts, uint32_t T, uint32_t top_k, uint32_t N, uint32_t K, __half* out,
                              hipStream_t stream);
// 8-bit streaming GEMV (qmv_q8.hip): f16 activations [M,K], chunks of 16 rows, group size 64 or 128.
bool qmv_q8_supported(uint32_t N, uint32_t K, uint32_t group_size);
int32_t launch_qmv_q8(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream,
                      int32_t x_bf16 = 0);  // 1: x holds bf16 bits, converted in registers
// chunk-table mode for the expert projections (expert strides in u32 words / halves as for the 4-bit kernel)
int32_t launch_qmv_q8_tab(const QmvArgs& a, hipStream_t stream);
// Single-row GEMV (qmv_m1.hip): 4- or 8-bit weights, group size 32 / 64 / 128, f16 activations; M rows are
// passes of up to four rows over the weights (grid.y); the store epilogue (EPI_*) is fused.
bool qmv_m1_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
int32_t launch_qmv_m1(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits, int epi_kind, const void* epi,
                      int32_t epi_dtype, const __half* norm_w, const float* inv_rms, hipStream_t stream,
                      int32_t x_bf16 = 0);  // 1: x holds bf16 bits, 2: f32 values; converted while staged (M <= 2 in one pass, no norm prologue)
bool qmv_m1_fuses_norm(uint32_t M, uint32_t K, uint32_t bits);
// Single-row GEMV for 2-bit weights (qmv_q2.hip): group size 32 / 64 / 128, f16 activations, one activation row per
// pass over the weights (grid.y = M), f16 out
bool qmv_q2_supported(uint32_t N, uint32_t K, uint32_t group_size);
int32_t launch_qmv_q2(const uint32_t* w, const __half* s, const __half* b, const __half* x, __half* out, uint32_t M,
                      uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream);
// The same with a weight matrix per output row (qmv_q2.hip): row m = activation row m / x_div of x through expert idx[m]
// of stacked 2-bit weights (outside [0, n_experts): zeros), out [batch, N] f16
int32_t launch_qmv_q2_gather(const uint32_t* w, const __half* s, const __half* b, uint64_t estride_w, uint64_t estride_s,
                             uint32_t n_experts, const __half* x, uint32_t x_div, const uint32_t* idx, uint32_t batch, __half* out,
                             uint32_t N, uint32_t K, uint32_t group_size, hipStream_t stream);
// dst[m,k] = (half(x[m,k]) * half(inv_rms[m])) * norm_w[k], each product rounded to f16 (the RMSNorm prologue as a separate pass)
int32_t launch_norm_rows(const void* x, int32_t x_dtype, const __half* norm_w, const float* inv_rms, uint32_t M,
                         uint32_t K, __half* dst, hipStream_t s);
// chunk table for gather_qmm: batch b owns rows [b*mpb, (b+1)*mpb) and expert indices[b]; chunks of at most
// chunk_rows rows (an index out of range sets bit 31 of the count: zeros are written); n_chunks (nullable)
// receives the table's length
int32_t launch_build_gather_chunks(const uint32_t* indices, uint32_t batch, uint32_t mpb, uint32_t n_experts,
                                   uint32_t chunk_rows, uint32_t* chunk_tab, uint32_t* n_chunks, hipStream_t s);

struct QmmArgs {
  const uint32_t* w; const __half* s; const __half* b;
  const void* x;      // [M,K] row-major, f16 / bf16 / f32 (cast fused into the re-layout pass)
  int32_t x_dtype;
  __half* out;        // [M,N]
  uint32_t M, N, K, bits;
  void* workspace;    // qmm_workspace_bytes(M, K[, N]) bytes of device scratch (fragment-major activations[, partial sums])
  int bf16_mfma;      // 1: bf16 activations x Q8 weights on the bf16 MFMA (weights rounded to bf16)
  // fused store epilogue (register-weights GEMM; the single-row GEMV takes the same three values): 0 none, 1 out = acc + e, 2 out = silu(e) * acc
  int epi_kind;
  const void* epi;    // [M,N] f16 or f32
  int32_t epi_dtype;
  const void* w_packed = nullptr;  // K-split GEMMs: the weights in their tile-contiguous order (gemm_layout_bytes), or null
  uint32_t group_size = 64;        // LDS-staged GEMM (the other GEMMs take it as a launch argument)
  bool workspace_has_partials = false;  // LDS-staged GEMM: the workspace was sized with N, so a launch of few tiles may split K
};
enum { EPI_NONE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2 };
// out[i] = out[i] + e[i]  /  silu(e[i]) * out[i], in place on f16 out (kernels without a fused epilogue)
int32_t launch_epilogue(__half* out, int kind, const void* e, int32_t e_dtype, size_t n, hipStream_t s);
size_t qmm_workspace_bytes(uint32_t M, uint32_t K, uint32_t N = 0);
// split-K partial sums of the register-weights GEMM (0 when the launch is not split); pass the buffer in QmmArgs::workspace
size_t qmm_rw_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
// 16 x 16 fragments per workgroup (tile rows / 16 x tile columns / 16) of the tile the launcher would pick; 0 = not supported
uint32_t qmm_rw_tile_work(uint32_t M, uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
bool qmm_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
int32_t launch_qmm(const QmmArgs& a, hipStream_t s);
// Register-weights GEMM (qmm_rw.hip): f16 activations only, no workspace.
bool qmm_rw_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
int32_t launch_qmm_rw(const QmmArgs& a, uint32_t group_size, hipStream_t s);
// K-split GEMM (qmm_k2.hip) for prefill-sized batches: 64 x 128 or 128 x 128 tiles (tile_rows), 32x32x16 MFMAs, the two
// halves of a workgroup split K; f16 / bf16 activations, no workspace, fused store epilogue.  The 128-row tile is built
// for every format whose kernel fits the register file (all but 8-bit weights at group size 32 / 64 with bf16 activations).
bool qmm_k2_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
bool qmm_k2_tall_supported(uint32_t group_size, uint32_t bits, bool x_bf16);
int32_t launch_qmm_k2(const QmmArgs& a, uint32_t group_size, uint32_t tile_rows, hipStream_t s);
// Tile-contiguous copy of a weight matrix for the K-split GEMMs: per (128 weight rows, 128-wide k block) the bytes in the
// order the waves load them, so that every wave instruction reads 1 KB of consecutive memory instead of 32 bytes of each
// of 32 rows.  0 bytes = the shape has no such layout (N % 128, K % 512, 4- or 8-bit).
size_t gemm_layout_bytes(size_t N, size_t K, uint32_t bits);
int32_t launch_gemm_repack(const uint32_t* w, uint32_t N, uint32_t K, uint32_t bits, void* dst, hipStream_t s);
// 32 x 64 tiles with K split four ways inside the workgroup (qmm_k4.hip): 4-bit weights, group size 64, K % 2048 == 0
bool qmm_k4_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
int32_t launch_qmm_k4(const QmmArgs& a, uint32_t group_size, hipStream_t s);
// Grouped form of the same GEMM for the expert projections of batches with many rows per expert: every
// row tile (kGroupedTileRows rows of one expert) takes its expert and rows from a device table of
// (expert, first row position, row count) triples (bit 31 of the count: write zeros instead of computing;
// not for a pair); `n_tiles_dev` holds the table's length.  With a second
// weight (w1 / s1 / b1: the up projection) the store writes silu(x Wg^T) * (x Wu^T).
constexpr uint32_t kGroupedTileRows = 64;
struct GroupedQmmArgs {
  const uint32_t* w; const __half* s; const __half* b;     // expert 0 of the (gate) weight
  const uint32_t* w1; const __half* s1; const __half* b1;  // expert 0 of the up weight, or null
  uint32_t N, K, bits;       // output columns (of a pair: columns of the product), input features
  uint32_t group_size;       // 32, 64 or 128
  uint64_t expert_stride_w;  // u32 words per expert
  uint64_t expert_stride_s;  // halves per expert
  const __half* x;           // [x_rows, K] f16
  const uint32_t* row_map;   // nullable: source row of position p is row_map[p]
  void* out;                 // f16 [positions, N] (f32 when out_f32; not for a pair)
  int out_f32;
  const uint32_t* tile_tab; const uint32_t* n_tiles_dev;
  uint32_t max_tiles;        // row tiles the grid covers (>= *n_tiles_dev)
  uint32_t tile_rows;        // rows per tile the table was built for: 32 or kGroupedTileRows
};
bool qmm_rw_grouped_supported(uint32_t N, uint32_t K, uint32_t group_size, uint32_t bits);
int32_t launch_qmm_rw_grouped(const GroupedQmmArgs& a, hipStream_t s);
// The LDS-staged GEMM over the same kind of table (tile_rows == 64, one weight, f16 output; shapes: qmm_supported)
size_t qmm_grouped_workspace_bytes(uint32_t max_tiles, uint32_t K, uint32_t tile_rows = 64);
int32_t launch_qmm_grouped(const GroupedQmmArgs& a, void* workspace, hipStream_t s);

// MoE helpers
int32_t launch_topk_route(const float* logits, const float* bias, uint32_t T, uint32_t E, uint32_t K,
                          int renorm, uint32_t* idx, float* w, uint32_t* counts, uint32_t* offsets,
                          hipStream_t s);
// Stable counting sort; also emits the chunk table used by the GEMV family
// (chunk_tab: 3 u32 per chunk; n_chunks: 1 u32).  chunk_tab / n_chunks may be null.
// sorted_tok (nullable): token of each sorted position, sorted[p] / top_k.
int32_t launch_moe_sort(const uint32_t* idx, uint32_t n_assign, uint32_t E, uint32_t top_k, uint32_t* sorted,
                        uint32_t* sorted_tok, uint32_t* inv, uint32_t* counts, uint32_t* offsets,
                        uint32_t* chunk_tab, uint32_t* n_chunks, uint32_t chunk_rows, hipStream_t s,
                        // (nullable) a second pair of tables that splits the experts by their row count: up to 8 rows -> one
                        // chunk in split_tab[0 .. 3 * split_cap), more -> chunks of at most 16 rows behind it; split_n[2]: lengths
                        uint32_t* split_tab = nullptr, uint32_t* split_n = nullptr, uint32_t split_cap = 0);
// Decode-sized batches (at most 8 tokens, 64 assignments): routing and grouping in one launch.
bool route_sort_fusable(uint32_t T, uint32_t E, uint32_t K);
int32_t launch_route_sort_small(const float* logits, const float* bias, uint32_t T, uint32_t E, uint32_t K,
                                int renorm, uint32_t* idx, float* w, uint32_t* sorted, uint32_t* sorted_tok,
                                uint32_t* inv, uint32_t* chunk_tab, uint32_t* n_chunks, hipStream_t s);
int32_t launch_index_gather(const __half* src, uint32_t d, const uint32_t* idx, uint32_t n, uint32_t src_rows,
                            __half* dst, hipStream_t s);
int32_t launch_scatter_weighted_add(const __half* src, uint32_t n, uint32_t d, const uint32_t* tok,
                                    const float* w, __half* dst, uint32_t dst_rows, hipStream_t s);
int32_t launch_silu_gate(const __half* g, const __half* u, __half* out, size_t n, hipStream_t s);
// out[r, c] = silu(g[r*ld + c]) * u[r*ld + c]
int32_t launch_silu_gate_strided(const __half* g, const __half* u, uint32_t ld, __half* out, uint32_t rows,
                                 uint32_t cols, hipStream_t s);
// tok[a] = a / top_k, inv[a] = a  (assignments kept in their own order)
int32_t launch_identity_positions(uint32_t* tok, uint32_t* inv, uint32_t n, uint32_t top_k, hipStream_t s);
// out[t,:] = sum_k w[t*K+k] * y[inv[t*K+k],:]  (y f32 rows at sorted positions)
int32_t launch_moe_combine(const float* y, const uint32_t* inv, const float* weights, uint32_t T,
                           uint32_t top_k, uint32_t D, __half* out, hipStream_t s);
int32_t launch_moe_combine_f16(const __half* y, const uint32_t* inv, const float* weights, uint32_t T, uint32_t top_k,
                               uint32_t D, __half* out, hipStream_t s);
// The same over f16 rows in assignment order (row t * top_k + k is pick k of token t); idx: the assignments' experts
// (outside [0, E): skipped)
int32_t launch_moe_combine_rows_f16(const __half* y, const uint32_t* idx, const float* weights, uint32_t T, uint32_t top_k,
                                    uint32_t D, uint32_t E, __half* out, hipStream_t s);
int32_t launch_add_bias_rows(__half* out, const __half* bias, uint32_t M, uint32_t N, hipStream_t s);
int32_t launch_awq_dequant(const uint32_t* qweight, const uint32_t* qzeros, const float* scales, float* out,
                           uint32_t rows, uint32_t cols, uint32_t group_size, hipStream_t s);
int32_t launch_gptq_dequant(const uint32_t* qweight, const uint32_t* qzeros, const float* scales,
                            const int32_t* g_idx, float* out, uint32_t in_features, uint32_t out_features,
                            uint32_t group_size, uint32_t num_groups, hipStream_t s);
int32_t launch_check_indices(const uint32_t* idx, uint32_t n, uint32_t limit, uint32_t* flag, hipStream_t s);

}  // namespace rmlx
