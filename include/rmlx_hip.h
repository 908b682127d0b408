/*
 * rmlx_hip.h -- C ABI of the MI355X (gfx950) quantized-matmul engine.
 *
 * Drop-in boundary for the quantized-matmul hot path of RMLX (`rmlx_core::ops::quantized`,
 * `ops::topk_route`, `ops::moe_kernels`, and the `rmlx-nn` callers `QuantizedLinear`,
 * `ExpertGroup::grouped_forward`, `MoeLayer::forward_grouped`).  A Rust `extern "C"` crate
 * binds exactly these symbols in place of the rmlx-metal dispatch for this path; every entry
 * point names the reference interface it replaces (paths relative to the reference checkout).
 *
 * Conventions (they mirror the reference's):
 *   - every pointer named `*_dev`, every `rmlx_array::data` and every weight buffer is a DEVICE
 *     pointer owned by the caller; no function takes ownership of caller memory;
 *   - outputs are caller-allocated (the caller plays the role of `Array::uninit`,
 *     crates/rmlx-core/src/array.rs:238); every output of a matmul is f16, row-major;
 *   - functions return 0 on success, RMLX_INVALID_SHAPE / RMLX_NOT_FOUND (the two
 *     `KernelError` variants used on this path, crates/rmlx-core/src/kernels/mod.rs:29-42) or
 *     RMLX_RUNTIME_ERROR for a failing HIP call; the message is kept per thread and read
 *     with rmlx_hip_last_error();
 *   - `stream == NULL` means synchronous: the call returns after the GPU has finished
 *     (`ExecMode::Sync`, crates/rmlx-core/src/ops/mod.rs:182-206).  With a stream the work is
 *     only enqueued (the `_into_cb` twins, crates/rmlx-core/src/ops/quantized.rs:7797-7802)
 *     and the caller synchronises;
 *   - all sizes are checked to fit in u32 (`checked_u32`, crates/rmlx-core/src/ops/mod.rs:71-74).
 */
#ifndef RMLX_HIP_H
#define RMLX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with hidden visibility: the functions declared here are its whole dynamic symbol table. */
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default)
#endif

/* ---- status / dtype ------------------------------------------------------------------ */

enum {
  RMLX_OK = 0,
  RMLX_INVALID_SHAPE = 1, /* KernelError::InvalidShape */
  RMLX_NOT_FOUND = 2,     /* KernelError::NotFound     */
  RMLX_RUNTIME_ERROR = 3  /* a HIP runtime call failed */
};

/* Subset of `DType` (crates/rmlx-core/src/dtype.rs:34-52) that appears on this path. */
enum {
  RMLX_DTYPE_F32 = 0,
  RMLX_DTYPE_F16 = 1,
  RMLX_DTYPE_BF16 = 2,
  RMLX_DTYPE_U32 = 3,
  RMLX_DTYPE_U8 = 4
};

/* View of an `Array` (crates/rmlx-core/src/array.rs:137-144): `data` already includes the
 * array's byte offset; the array must be row-contiguous. */
typedef struct rmlx_array {
  void* data;
  int32_t dtype;
  int32_t ndim;
  size_t shape[4];
} rmlx_array;

typedef void* rmlx_stream;            /* a hipStream_t */
typedef void* rmlx_event;             /* a hipEvent_t  */
typedef struct rmlx_qweight rmlx_qweight; /* `QuantizedWeight`, opaque */

/* Message of the last failing call on this thread ("" if none). */
const char* rmlx_hip_last_error(void);

/* ---- runtime shim (replaces the rmlx-metal device/queue/buffer calls this path makes) ---- */

/* Select `device`, verify it is a gfx950 part and load the kernels.  Fails loudly (no CPU
 * fallback exists in this library). */
int32_t rmlx_hip_init(int32_t device);
/* Fills: [0] compute units, [1] wavefront size, [2] LDS bytes per workgroup, [3] total
 * global memory in MiB, [4] max engine clock kHz, [5] memory clock kHz, [6] bus width bits,
 * [7] L2 bytes. */
int32_t rmlx_hip_device_info(int64_t out[8]);
int32_t rmlx_hip_malloc(void** dev_ptr, size_t bytes);
int32_t rmlx_hip_free(void* dev_ptr);
int32_t rmlx_hip_memset(void* dev_ptr, int32_t value, size_t bytes, rmlx_stream stream);
int32_t rmlx_hip_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, rmlx_stream stream);
int32_t rmlx_hip_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, rmlx_stream stream);
int32_t rmlx_hip_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, rmlx_stream stream);
int32_t rmlx_hip_stream_create(rmlx_stream* out);
int32_t rmlx_hip_stream_sync(rmlx_stream stream);
/* Synchronises the stream, hands its idle scratch blocks back to the driver and destroys it. */
int32_t rmlx_hip_stream_destroy(rmlx_stream stream);
/* The library keeps the scratch blocks of a stream (dtype casts, split-K partial sums, MoE intermediates) for
 * the next call on that stream, so steady-state calls do not allocate.  This synchronises the stream (NULL = the
 * default stream of synchronous calls) and frees its idle blocks, e.g. after one unusually large batch.  The
 * counterpart of the reference's thread-local array pool going out of scope (crates/rmlx-core/src/array.rs:33-47). */
int32_t rmlx_hip_trim_pool(rmlx_stream stream);
/* Number of device allocations (hipMalloc) the library's scratch pool has made in this process so far.  It does not
 * move across a call that took everything from blocks the pool already held, or across rmlx_hip_moe_forward_noalloc;
 * a caller that is about to capture a graph can check just that.  (No counterpart in the reference.) */
uint64_t rmlx_hip_scratch_allocations(void);
/* Recording and replaying a train of calls (the counterpart of encoding several `_into_cb` calls into one command
 * buffer and committing it, crates/rmlx-core/src/ops/quantized.rs:7797-7802): between graph_begin and graph_end
 * every call on `stream` is recorded instead of run; graph_launch replays the recording on a stream.  Only calls
 * that neither allocate nor synchronise may be recorded (the f16 qmv / qmm paths, rmlx_hip_moe_forward_noalloc; a
 * pooled call whose scratch the stream's pool already holds), and the buffers they name must stay alive. */
typedef void* rmlx_graph;             /* a hipGraphExec_t */
int32_t rmlx_hip_graph_begin(rmlx_stream stream);
int32_t rmlx_hip_graph_end(rmlx_stream stream, rmlx_graph* out);
int32_t rmlx_hip_graph_launch(rmlx_graph graph, rmlx_stream stream);
int32_t rmlx_hip_graph_destroy(rmlx_graph graph);
int32_t rmlx_hip_event_create(rmlx_event* out);
int32_t rmlx_hip_event_record(rmlx_event ev, rmlx_stream stream);
int32_t rmlx_hip_event_sync(rmlx_event ev);
int32_t rmlx_hip_event_elapsed_ms(rmlx_event start, rmlx_event stop, float* ms);
int32_t rmlx_hip_event_destroy(rmlx_event ev);

/* ---- QuantizedWeight ------------------------------------------------------------------
 * `QuantizedWeight::new` (crates/rmlx-core/src/ops/quantized.rs:97-160).  MLX affine layout:
 * weights u32 [out_features, in_features*bits/32] (value i of a row in word i/(32/bits) at
 * bit bits*(i%(32/bits))), scales and biases f16 [out_features, in_features/group_size],
 * w = scale*q + bias.  Same validation and messages: bits in {2,3,4,6,8}, group_size in
 * {32,64,128}, in_features % group_size == 0, the three byte lengths large enough.
 * `n_experts` > 1 declares the stacked layout [n_experts, out_features, ...] that
 * `gather_qmm` / `gather_qmv_fast_f16_q4` consume (quantized.rs:9279-9290, 9605-9620);
 * pass 1 for a plain linear weight. */
int32_t rmlx_hip_qweight_create(const void* weights_dev, size_t weights_bytes,
                                const void* scales_dev, size_t scales_bytes,
                                const void* biases_dev, size_t biases_bytes,
                                uint32_t group_size, uint32_t bits,
                                size_t out_features, size_t in_features, size_t n_experts,
                                rmlx_qweight** out);
int32_t rmlx_hip_qweight_destroy(rmlx_qweight* qw);

/* ---- qmv: `affine_quantized_matmul` (quantized.rs:1309-1411) ----------------------------
 * vec: 1-D (or any shape) with numel == in_features, f16 / f32 (bf16 also accepted and used
 * natively); out: f16 [out_features].  Q4 and Q8. */
int32_t rmlx_hip_affine_quantized_matmul(const rmlx_qweight* qw, const rmlx_array* vec,
                                         void* out_f16_dev, size_t out_bytes, rmlx_stream stream);

/* ---- qmm: `affine_quantized_matmul_batched` (quantized.rs:7149-7782) -----------------------
 * x: 2-D [M, in_features], f16 / f32 / bf16; out: f16 [M, out_features].  Chooses the kernel
 * by M (the reference's dispatch ladder, re-tuned for this chip): the single-row streaming
 * GEMV for M <= 2, the multi-row streaming MFMA GEMV for small M, the MFMA GEMM (weights
 * dequantised in registers, or staged through LDS) above, and the portable kernel for bit
 * widths and shapes none of those takes. */
int32_t rmlx_hip_affine_quantized_matmul_batched(const rmlx_qweight* qw, const rmlx_array* x,
                                                 void* out_f16_dev, size_t out_bytes,
                                                 rmlx_stream stream);

/* Same contract as the batched entry point but forces one kernel family (the reference
 * exposes its kernels individually too, e.g. `affine_qmv_batched_f16_q4` quantized.rs:1675,
 * `affine_quantized_matmul_nax` :8517).  kernel: 0 = auto, 1 = streaming GEMV (qmv: the
 * single-row kernel where it applies -- M <= 2, or M <= 16 at group size 32, of which the automatic choice keeps M <= 4
 * where the MFMA GEMM takes the shape -- else the multi-row one),
 * 2 = MFMA GEMM (qmm, f16 MFMA; bf16 activations are converted, which is exact for
 * normal-range values; the register-weights kernel when K % 512 == 0 (group size 64: K % 128 == 0, K >= 512), else the
 * LDS-staged one: K % 64 == 0),
 * 3 = portable scalar kernel (any bits/group size the type admits),
 * 4 = LDS-staged MFMA GEMM on the bf16 matrix instruction (Q8 weights and bf16 activations
 * only; weights are rounded to bf16, so its error is about four times that of kernel 2),
 * 5 = LDS-staged MFMA GEMM (f16 MFMA, every group size, K % 64 == 0, K >= 256),
 * 6 = multi-row streaming GEMV also for a single row (group sizes 64 and 128; 4-bit weights at group size 32 with
 * K % 512 == 0 and K <= 4096 on the wave-per-tile form, which the automatic choice takes for 3 to 8 rows over matrices
 * of 24576 rows or more),
 * 7 = K-split MFMA GEMM (64 x 128 tiles, 32x32x16 MFMAs; N % 128 == 0, K % 512 == 0; what kernel 2 resolves to
 * when that grid is one round over most of the chip), 8 = the register-weights GEMM whatever the shape,
 * 9 = the K-split MFMA GEMM with 128 x 128 tiles (not for 8-bit weights at group size 32 / 64 with bf16 activations; what
 * kernel 2 resolves to when those tiles make 0.55 rounds over the chip or more), 10 = the K-split MFMA GEMM with 32 x 128
 * tiles (what kernel 2 resolves to when those tiles make at most one round over the chip and the register-weights GEMM
 * would need more than one round of its 32 x 64 tiles; K <= 4096), 11 = the MFMA GEMM with 32 x 64 tiles and K split four
 * ways inside the workgroup (4-bit weights at group size 64, N % 64 == 0, K % 2048 == 0). */
int32_t rmlx_hip_qmm_select(const rmlx_qweight* qw, const rmlx_array* x, int32_t kernel,
                            void* out_f16_dev, size_t out_bytes, rmlx_stream stream);

/* Fused store epilogues of the batched matmul (`qmm_add_residual_into_cb` quantized.rs:8227-8340,
 * `qmm_swiglu_into_cb` :8345-8452): out = x @ dequant(W)^T + residual, resp.
 * out = silu(gate_result) * (x @ dequant(W)^T).  residual / gate_result: [M, out_features],
 * Float16 or Float32 (the reference's are Float32), same validation message as the reference
 * ("... shape must be [M, N]"); out is f16.  Evaluated in f32 on the accumulator with one rounding
 * in the GEMM kernel; after the GEMV / portable kernels as a separate elementwise pass.  Unlike the
 * reference (Q4, M > 32 only) every shape the batched entry point takes is accepted. */
int32_t rmlx_hip_qmm_add_residual(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* residual,
                                  void* out_f16_dev, size_t out_bytes, rmlx_stream stream);
int32_t rmlx_hip_qmm_swiglu(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* gate_result,
                            void* out_f16_dev, size_t out_bytes, rmlx_stream stream);

/* RMSNorm prologue of the reference's Q4 MMA kernel (`has_norm`, function constant 203: quantized.rs:2955-2992, A loader
 * :3070-3095; no host entry point of the reference sets it): the activations are normalised on the way in,
 * x'[m,k] = (half(x[m,k]) * half(inv_rms[m])) * norm_weight[k], each product rounded to f16, and out = x' @ dequant(W)^T.
 * x: [M, in_features] f16 / f32 / bf16; norm_weight: f16 [in_features]; inv_rms: f32 [M] (the caller's 1/rms of each row).
 * Fused into the single-row GEMV (M <= 2); a separate elementwise pass in front of the other kernels. */
int32_t rmlx_hip_qmm_norm(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* norm_weight,
                          const rmlx_array* inv_rms, void* out_f16_dev, size_t out_bytes, rmlx_stream stream);

/* Encode `count` batched matmuls back to back on `stream` with no synchronisation in between:
 * the `_into_cb` usage of the reference, which encodes every QMM of a decoder stack into one
 * command buffer (`affine_quantized_matmul_batched_into_cb`, quantized.rs:7797-7802;
 * crates/rmlx-core/benches/qmm_pipeline_bench.rs:249-304).  Matmul i multiplies x by
 * qws[i % n_qw] and writes outs[i % n_out] (each f16 [M, out_features], out_bytes long).
 * All weights must have the same shape.  stream == NULL synchronises once at the end. */
int32_t rmlx_hip_qmm_encode_many(const rmlx_qweight* const* qws, size_t n_qw, const rmlx_array* x,
                                 void* const* outs_f16_dev, size_t n_out, size_t out_bytes,
                                 size_t count, int32_t kernel, rmlx_stream stream);

/* ---- `QuantizedLinear::forward` / `Linear::forward` call shape ------------------------------
 * (crates/rmlx-nn/src/quantized_linear.rs:153-201, crates/rmlx-nn/src/linear.rs:98-191)
 * x 1-D [in] is treated as [1,in]; 2-D [batch,in] -> [batch,out]; other ranks are rejected;
 * batch == 1 takes the qmv path.  `bias_f16_dev` (nullable, [out]) is the broadcast bias
 * `Linear` adds. */
int32_t rmlx_hip_quantized_linear_forward(const rmlx_qweight* qw, const rmlx_array* x,
                                          const void* bias_f16_dev, void* out_f16_dev,
                                          size_t out_bytes, rmlx_stream stream);

/* ---- gather_qmm (quantized.rs:9404-9599) and gather_qmv_fast_f16_q4 (:10061-10236) ---------
 * out[b] = x[b] @ dequant(W[indices[b]])^T.  x: [batch, m_per_batch, k] f16 or f32;
 * w/s/b: stacked [n_experts, n, ...] buffers with their byte lengths; indices: u32 [batch];
 * out: f16 [batch, m_per_batch, n].  Validation as the reference (non-zero dims, even k,
 * k % group_size, buffer lengths, indices dtype/length, every index < n_experts; batch == 0
 * returns an empty result).  The index range check reads the indices back and therefore
 * only runs when stream == NULL; with a stream, rows whose index is out of range are
 * written as zeros. */
int32_t rmlx_hip_gather_qmm(const rmlx_array* x, const void* w_packed_dev, size_t w_bytes,
                            const void* scales_dev, size_t scales_bytes,
                            const void* biases_dev, size_t biases_bytes,
                            const rmlx_array* indices, size_t batch, size_t m_per_batch,
                            size_t n, size_t k, size_t n_experts, uint32_t group_size,
                            void* out_f16_dev, size_t out_bytes, rmlx_stream stream);
/* The same with the kernel family forced (the reference exposes `gather_qmm` and `gather_qmv_fast_f16_q4`
 * separately, quantized.rs:9404, 10061).  kernel: 0 = auto (one row per entry: the single-row GEMV with a weight
 * matrix per activation row, N % 8 == 0, K % 32 == 0, K <= 28672; streaming GEMV up to 8 rows per entry; grouped MFMA
 * GEMM from 9 rows on where it takes the shape: N % 128 == 0, K % 512 == 0, at group sizes 32 / 64 also K % 128 == 0
 * from 512 on; the portable kernel for every other shape), 1 = streaming GEMV (group size 64 / 128, N % 16 == 0,
 * K % 128 == 0), 2 = grouped MFMA GEMM,
 * 3 = portable kernel. */
int32_t rmlx_hip_gather_qmm_select(const rmlx_array* x, const void* w_packed_dev, size_t w_bytes,
                                   const void* scales_dev, size_t scales_bytes,
                                   const void* biases_dev, size_t biases_bytes,
                                   const rmlx_array* indices, size_t batch, size_t m_per_batch,
                                   size_t n, size_t k, size_t n_experts, uint32_t group_size,
                                   int32_t kernel, void* out_f16_dev, size_t out_bytes,
                                   rmlx_stream stream);

/* ---- gpu_topk_route (crates/rmlx-core/src/ops/topk_route.rs:433-650) -----------------------
 * gate_logits [T,E] f32 or f16 -> expert_indices u32 [T*K] (descending, ties to the lower
 * index), expert_weights f32 [T*K] (softmax, renormalised over the K picks unless
 * renormalize == 0), expert_counts u32 [E], dispatch_offsets u32 [E+1].  1 <= K <= 8,
 * K <= E <= 256; expert_bias (nullable) is 1-D [E] f32 or f16. */
int32_t rmlx_hip_topk_route(const rmlx_array* gate_logits, size_t top_k,
                            const rmlx_array* expert_bias, int32_t renormalize,
                            uint32_t* expert_indices_dev, float* expert_weights_dev,
                            uint32_t* expert_counts_dev, uint32_t* dispatch_offsets_dev,
                            rmlx_stream stream);

/* ---- token -> expert grouping (crates/rmlx-nn/src/moe.rs:1439-1447) --------------------------
 * On-device replacement of the host-side `expert_dispatch` build: a stable counting sort of
 * the flat assignment ids (tok*K + k) by expert.  sorted_assign u32 [n_assign]: segment
 * [offsets[e], offsets[e+1]) lists the ids routed to expert e in ascending order;
 * offsets u32 [n_experts+1]. */
int32_t rmlx_hip_moe_sort(const uint32_t* expert_indices_dev, size_t n_assign, size_t n_experts,
                          uint32_t* sorted_assign_dev, uint32_t* offsets_dev, rmlx_stream stream);

/* ---- index_gather / scatter_weighted_add (crates/rmlx-core/src/ops/moe_kernels.rs:239-363) --
 * dst[i,:] = src[idx[i],:]            (f16 rows of width d)
 * dst[tok[i],:] += w[i] * src[i,:]    (f32 accumulation, deterministic: assignments of a
 *                                      token are added in ascending i) */
int32_t rmlx_hip_index_gather(const void* src_f16_dev, size_t src_rows, size_t d,
                              const uint32_t* idx_dev, size_t n, void* dst_f16_dev,
                              rmlx_stream stream);
int32_t rmlx_hip_scatter_weighted_add(const void* src_f16_dev, size_t n, size_t d,
                                      const uint32_t* tok_dev, const float* w_dev,
                                      void* dst_f16_dev, size_t dst_rows, rmlx_stream stream);

/* ---- silu_gate (crates/rmlx-core/src/ops/silu.rs:142-166) -----------------------------------
 * out = silu(gate_in) * up_in, f16, sigmoid evaluated in f32. */
int32_t rmlx_hip_silu_gate(const void* gate_in_f16_dev, const void* up_in_f16_dev,
                           void* out_f16_dev, size_t numel, rmlx_stream stream);

/* ---- ExpertGroup::grouped_forward (crates/rmlx-nn/src/expert_group.rs:308-533) --------------
 * Literal contract: `n_items` (expert_idx, input [batch_i, D]) pairs, inputs packed one
 * after another in x ([sum batch_i, D] f16); out receives the per-item outputs in the same
 * packing.  Per item: y = (silu(x Wg^T) * (x Wu^T)) Wd^T with stacked expert weights (the streaming kernels
 * take 4-bit weights with group size 64 or 128 and dimensions in multiples of 512, and 8-bit weights with group size 64
 * and dimensions in multiples of 256; batches with many rows per expert take the grouped MFMA GEMM, see
 * rmlx_hip_qweight_set_expert_gemm_min_rows; every other 2- / 4- / 8-bit weight the type admits runs the same block
 * on the portable kernels)
 * gate/up [E, I, D] and down [E, D, I].  `up` may be NULL when `gate` holds the fused
 * [E, 2I, D] layout (gate rows first).  expert_idx and batch_sizes are HOST arrays.
 * Validation as the reference: idx < E, n_items == 0 -> nothing to do. */
int32_t rmlx_hip_expert_group_grouped_forward(const rmlx_qweight* gate, const rmlx_qweight* up,
                                              const rmlx_qweight* down, size_t n_items,
                                              const uint32_t* expert_idx_host,
                                              const uint32_t* batch_sizes_host,
                                              const rmlx_array* x, void* out_f16_dev,
                                              size_t out_bytes, rmlx_stream stream);

/* ---- MoeLayer::forward_grouped (crates/rmlx-nn/src/moe.rs:1391-1508) ------------------------
 * The whole routed-expert block with no host round trip:
 * route (given) -> on-device sort -> gate/up gather_qmm + SwiGLU -> down gather_qmm ->
 * f32 weighted combine -> f16 out [T, D].  expert_indices / expert_weights are the [T*K]
 * outputs of rmlx_hip_topk_route (device). */
int32_t rmlx_hip_moe_forward_grouped(const rmlx_qweight* gate, const rmlx_qweight* up,
                                     const rmlx_qweight* down, const rmlx_array* x,
                                     const uint32_t* expert_indices_dev,
                                     const float* expert_weights_dev, size_t top_k,
                                     void* out_f16_dev, size_t out_bytes, rmlx_stream stream);

/* Kernel choice of the expert projections (ExpertGroup and the MoeLayer entry points): batches with at least
 * `min_rows` rows per expert on average (rows / num_experts; for ExpertGroup rows / n_items) multiply with the
 * grouped MFMA GEMM -- row tiles of 16, 32 or 64 rows of one expert, weights dequantised in registers; 4- / 8-bit,
 * group sizes 32 / 64 / 128 (one for the three projections), hidden and intermediate dimensions in multiples of
 * 512 -- smaller ones with the streaming GEMV, which reads an expert's weights once per 8 rows (8-bit experts
 * switch at an eighth of `min_rows`, at least 1).  0 = never the GEMM; the default (10) is the measured crossover.
 * The value lives in the handle of the stacked GATE weight and applies to the calls that pass that handle: there
 * is no process-wide state.  Set it before other threads use the handle.  The counterpart of choosing a
 * `MoeStrategy` for a layer in the reference (crates/rmlx-nn/src/moe.rs:515-541).  Returns the previous value. */
uint32_t rmlx_hip_qweight_set_expert_gemm_min_rows(rmlx_qweight* gate_qw, uint32_t min_rows);
/* Optional second copy of a weight matrix in the order the K-split MFMA GEMMs (kernels 7, 9, 10, 11) load it: per 128
 * weight rows and 128-wide k block the 8 KB (8-bit: 16 KB) of the tile as consecutive 1 KB wave loads, instead of 32 bytes
 * of each of 32 rows per load.  The MLX layout stays the input and stays in use by every other kernel; the caller owns
 * `dst_dev` (`rmlx_hip_qweight_gemm_layout_bytes(qw)` bytes = the size of the weight buffer, 16-byte aligned; 0 = the
 * weight has no such layout: 4- or 8-bit, out_features % 128 == 0, in_features % 512 == 0, one expert) and keeps it
 * alive while the handle uses it; `dst_dev == NULL` drops it again.  The copy is made on `stream` (NULL: before the call
 * returns).  Results are bit-identical with and without it.  The counterpart of the reference repacking weights at load
 * time (crates/rmlx-nn/src/safetensors_loader.rs:562-628).  Set it before other threads use the handle. */
size_t rmlx_hip_qweight_gemm_layout_bytes(const rmlx_qweight* qw);
int32_t rmlx_hip_qweight_set_gemm_layout(rmlx_qweight* qw, void* dst_dev, size_t dst_bytes, rmlx_stream stream);
/* Which streaming kernel runs the expert projections of decode-sized batches (below the grouped GEMM's threshold) of a
 * block whose gate weight is `qw`: 1 = K split over the waves of a workgroup, chunks of 8 rows, 2 = a wave per 16-row
 * weight tile, chunks of 8 rows, 3 = a wave per tile, chunks of 16 rows, 4 = kernel 1 for the gate / up projection and
 * kernel 2 for the down projection (4-bit weights, group size 64; other weights keep kernel 1), 5 = as 4 with the gate / up
 * projection in two launches, the experts split by their row count: up to 8 rows on kernel 1, more on kernel 3, so every
 * expert is streamed once whatever the largest row count, 0 = the library's choice (4; 5 from 6 rows per expert on
 * average).  Kernel 3 streams an expert with 9 to 16 rows once instead of twice and is the fastest of the four from 7 rows
 * per expert on average - as long as no expert of the batch has more than 16 rows, so it is for callers whose router bounds
 * that.  Returns the previous value; the tests use it to check that the kernels agree.  (No counterpart in the reference, which has one kernel for this: gather_qmv_fast_f16_q4,
 * crates/rmlx-core/src/ops/quantized.rs:9752-9842.) */
uint32_t rmlx_hip_qweight_set_expert_stream_kernel(rmlx_qweight* qw, uint32_t kind);

/* Routing + the block above in one call: gate_logits [T,E] (the router's output). */
int32_t rmlx_hip_moe_forward(const rmlx_qweight* gate, const rmlx_qweight* up,
                             const rmlx_qweight* down, const rmlx_array* x,
                             const rmlx_array* gate_logits, size_t top_k,
                             const rmlx_array* expert_bias, void* out_f16_dev, size_t out_bytes,
                             rmlx_stream stream);

/* rmlx_hip_moe_forward for callers that cannot allocate: code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels and the same
 * result as rmlx_hip_moe_forward, but every intermediate (routing output, grouping tables, hidden activations,
 * per-assignment expert outputs, dtype casts) is carved from a workspace of 8 MiB that is part of the library's
 * device code (one copy per GPU, held until the process ends; rmlx_hip_init resolves its address), so the call
 * makes no hipMalloc / hipFree and touches no pool.  Limits: batches whose intermediates exceed the workspace
 * (about seq_len * top_k * (4 * hidden + 2 * intermediate + 36) bytes: 53 tokens at top-8, hidden 4096,
 * intermediate 1536; 2-bit experts: seq_len * top_k * (2 * hidden + 6 * intermediate)) are rejected with InvalidShape;
 * expert weights that only the portable kernels take are rejected with NotFound.  Every call on a GPU uses the same workspace: calls that
 * overlap on one GPU (two streams, two threads) race; consecutive calls on one stream are ordered. */
int32_t rmlx_hip_moe_forward_noalloc(const rmlx_qweight* gate, const rmlx_qweight* up,
                                     const rmlx_qweight* down, const rmlx_array* x,
                                     const rmlx_array* gate_logits, size_t top_k,
                                     const rmlx_array* expert_bias, void* out_f16_dev, size_t out_bytes,
                                     rmlx_stream stream);

/* ---- AWQ / GPTQ INT4 dequantisation to f32 -----------------------------------------------------
 * `awq_dequant` (quantized.rs:2269-2383, kernel :707-733): qweight u32 [rows, cols/8] packed along
 * the columns, qzeros u32 [rows/group_size, cols/8], scales f32 [rows/group_size, cols];
 * out f32 [rows, cols] = scales[g, col] * (nibble(qweight, col % 8) - nibble(qzeros, col % 8)), g = row / group_size.
 * `gptq_dequant` (quantized.rs:2407-2590, kernel :749-783): qweight u32 [in_features/8, out_features]
 * packed along the rows, qzeros u32 [num_groups, out_features/8], scales f32 [num_groups, out_features],
 * g_idx (nullable) i32 [in_features]; out f32 [in_features, out_features] =
 * scales[g, col] * (nibble(qweight, row % 8) - (nibble(qzeros, col % 8) + 1)), g = g_idx[row] or row / group_size.
 * With g_idx, num_groups is what the scales buffer holds (scales_bytes / 4 / out_features), as in the
 * reference; unlike the reference, a row whose g_idx lies outside [0, num_groups) is written as zeros
 * instead of reading out of bounds.  Validation and messages as the reference (pack-factor multiples,
 * group_size > 0, divisibility, the buffer lengths). */
int32_t rmlx_hip_awq_dequant(const void* qweight_dev, size_t qweight_bytes, const void* qzeros_dev,
                             size_t qzeros_bytes, const void* scales_f32_dev, size_t scales_bytes,
                             size_t rows, size_t cols, size_t group_size, void* out_f32_dev,
                             size_t out_bytes, rmlx_stream stream);
int32_t rmlx_hip_gptq_dequant(const void* qweight_dev, size_t qweight_bytes, const void* qzeros_dev,
                              size_t qzeros_bytes, const void* scales_f32_dev, size_t scales_bytes,
                              const int32_t* g_idx_dev, size_t g_idx_bytes, size_t in_features,
                              size_t out_features, size_t group_size, void* out_f32_dev,
                              size_t out_bytes, rmlx_stream stream);

/* ---- machine floors (measurement aid; no counterpart in the reference) ---------------------------------
 * `count` back-to-back launches, on `stream`, of a kernel that does nothing but one thing, so that a benchmark
 * can time them with the same events as the matmul kernels:
 *   RMLX_FLOOR_EMPTY          an empty kernel (launch cost);
 *   RMLX_FLOOR_READ2/4/8      a plain streaming read of `bytes` bytes with 16-byte non-temporal loads, 2 / 4 / 8
 *                             loads in flight per lane, 512-thread workgroups; launch i reads copy i % n_src of
 *                             the n_src consecutive copies at src_dev (cycle more than the caches hold);
 *   RMLX_FLOOR_MFMA           `iters` rounds of 16 independent v_mfma_f32_16x16x32_f16 per wave, 8 waves per
 *                             workgroup, `bytes` workgroups (0 = two per CU): 8 * 16 * 16384 * iters flop each;
 *   RMLX_FLOOR_MFMA_VALU      the same loop with n_src (2, 4, 6 or 8) and-or vector instructions behind every MFMA:
 *                             the matrix rate left while the vector ALU unpacks beside it;
 *   RMLX_FLOOR_LDS            `iters` rounds of eight conflict-free 16-byte LDS reads per lane, n_src (8 or 16)
 *                             waves per workgroup, `bytes` workgroups (0 = one per CU): waves * 64 * 128 * iters
 *                             bytes each;
 *   RMLX_FLOOR_L2_READ        n_src workgroups (0 = two per CU) of 512 threads each read iters * 32 KB from a source
 *                             of `bytes` bytes (a power of two, small enough to stay in one L2) that all of them
 *                             walk: the rate at which L2 hits reach the CUs.
 * sink_dev: at least 16 bytes of device memory (never written in practice; keeps the work alive). */
enum { RMLX_FLOOR_EMPTY = 0, RMLX_FLOOR_READ4 = 1, RMLX_FLOOR_READ8 = 2, RMLX_FLOOR_MFMA = 3, RMLX_FLOOR_READ2 = 4,
       RMLX_FLOOR_MFMA_VALU = 5, RMLX_FLOOR_LDS = 6, RMLX_FLOOR_L2_READ = 7 };
int32_t rmlx_hip_measure_floor(int32_t kind, const void* src_dev, size_t bytes, size_t n_src, uint32_t iters,
                               void* sink_dev, size_t count, rmlx_stream stream);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* RMLX_HIP_H */
