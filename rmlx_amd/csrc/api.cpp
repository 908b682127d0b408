// Host side of the C ABI: validation (same rules and messages as the reference's Rust entry
// points), the dispatch ladder, and the composition of the MoE block.  No arithmetic happens
// here and there is no CPU fallback: every path ends in a HIP kernel launch or an error.
#include <cinttypes>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "common.hpp"

// Workspace of the entry point that allocates nothing (rmlx_hip_moe_forward_noalloc): device memory that exists
// from the moment the code object is loaded until the process ends, one copy per GPU.  Host code never uses this
// name as an address: rmlx_hip_init resolves the device address once per device and every use goes through that.
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace rmlx {

namespace {
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};  // device address of `scratch` on every device rmlx_hip_init has seen
}  // namespace

std::string& last_error() {
  thread_local std::string e;
  return e;
}

int32_t fail(int32_t code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  last_error() = buf;
  return code;
}

int32_t checked_u32(size_t v, const char* name, uint32_t* out) {
  if (v > 0xFFFFFFFFull) return fail(RMLX_INVALID_SHAPE, "%s (%zu) exceeds u32::MAX", name, v);
  *out = (uint32_t)v;
  return RMLX_OK;
}

const char* dtype_name(int32_t dt) {
  switch (dt) {
    case RMLX_DTYPE_F32: return "Float32";
    case RMLX_DTYPE_F16: return "Float16";
    case RMLX_DTYPE_BF16: return "Bfloat16";
    case RMLX_DTYPE_U32: return "UInt32";
    case RMLX_DTYPE_U8: return "UInt8";
    default: return "Unknown";
  }
}

DeviceCtx& ctx() {
  static DeviceCtx c;
  return c;
}

int32_t require_init() {
  if (!ctx().ready) return fail(RMLX_RUNTIME_ERROR, "rmlx_hip_init() has not been called (no GPU context)");
  // The current device is a per-thread setting of the runtime: a thread other than the one that called
  // rmlx_hip_init starts on device 0.
  int cur = -1;
  if (hipGetDevice(&cur) == hipSuccess && cur != ctx().device) RMLX_HIP_CHECK(hipSetDevice(ctx().device));
  return RMLX_OK;
}

int32_t finish(hipStream_t stream) {
  if (stream == nullptr) RMLX_HIP_CHECK(hipStreamSynchronize(nullptr));
  return RMLX_OK;
}

// Scratch blocks are pooled per stream and never handed back to the driver while the library is
// loaded: every use is ordered on the owning stream, so a block released by one call can be
// reused by the next call on that stream without synchronisation, and steady-state calls make
// no allocator calls at all.
namespace {
struct Block { void* ptr; size_t bytes; };
std::mutex g_pool_mutex;
std::map<hipStream_t, std::vector<Block>> g_pool;
uint64_t g_pool_allocations = 0;  // hipMalloc calls made for the pool (guarded by g_pool_mutex)
}  // namespace

int32_t Scratch::alloc(size_t bytes, hipStream_t s, Arena* arena) {
  release();
  stream = s;
  if (bytes == 0) bytes = 16;
  if (arena != nullptr) {  // carved from the caller's block, 256-byte aligned, never handed to the pool
    const size_t start = (arena->used + 255) & ~(size_t)255;
    if (start + bytes > arena->capacity)
      return fail(RMLX_INVALID_SHAPE, "the call needs more than the %zu bytes of the static workspace", arena->capacity);
    ptr = arena->base + start;
    size = bytes;
    arena->used = start + bytes;
    pooled = false;
    return RMLX_OK;
  }
  pooled = true;
  {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    std::vector<Block>& free_list = g_pool[s];
    size_t best = free_list.size();
    for (size_t i = 0; i < free_list.size(); ++i)
      if (free_list[i].bytes >= bytes && (best == free_list.size() || free_list[i].bytes < free_list[best].bytes)) best = i;
    if (best != free_list.size()) {
      ptr = free_list[best].ptr;
      size = free_list[best].bytes;
      free_list.erase(free_list.begin() + (long)best);
      return RMLX_OK;
    }
  }
  const size_t rounded = (bytes + 0xFFFFF) & ~(size_t)0xFFFFF;  // 1 MiB granularity
  RMLX_HIP_CHECK(hipMalloc(&ptr, rounded));
  size = rounded;
  {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    ++g_pool_allocations;
  }
  return RMLX_OK;
}

void Scratch::release() {
  if (ptr != nullptr && pooled) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    g_pool[stream].push_back(Block{ptr, size});
  }
  ptr = nullptr;
}

// Frees the idle scratch blocks of a stream (the caller has synchronised it); `forget` also drops its entry.
int32_t trim_pool(hipStream_t s, bool forget) {
  std::vector<Block> blocks;
  {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_pool.find(s);
    if (it == g_pool.end()) return RMLX_OK;
    blocks.swap(it->second);
    if (forget) g_pool.erase(it);
  }
  // every block is handed back; the first failure is what the caller hears about
  hipError_t first = hipSuccess;
  for (const Block& b : blocks) {
    const hipError_t e = hipFree(b.ptr);
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  if (first != hipSuccess) return fail(RMLX_RUNTIME_ERROR, "hipFree of a pooled scratch block failed: %s", hipGetErrorString(first));
  return RMLX_OK;
}

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- the dispatch ladder --------------------------------------------------------------------
// The reference picks by M: QMV for M=1, batched QMV up to a per-chip limit, split-K Steel for
// 32 <= M < 128 and NAX above (crates/rmlx-core/src/ops/quantized.rs:7200-7256).  Here: the
// single-row GEMV for M <= 2 (and up to 16 rows when the group size is not 64), the streaming MFMA
// GEMV (weights read once per chunk of 8 rows; 16 rows for 8-bit weights) for small M, the
// register-weights MFMA GEMM above (the LDS-staged GEMM when K is not a multiple of 512), the
// portable kernel for every shape the fast kernels do not take.
enum { KERNEL_AUTO = 0, KERNEL_QMV = 1, KERNEL_QMM = 2, KERNEL_GENERIC = 3, KERNEL_QMM_BF16 = 4, KERNEL_QMM_LDS = 5,
       KERNEL_QMV_ROWS = 6, KERNEL_QMM_K2 = 7, KERNEL_QMM_RW = 8, KERNEL_QMM_K2_TALL = 9, KERNEL_QMM_K2_FLAT = 10, KERNEL_QMM_K4 = 11 };
constexpr uint32_t kQmvMaxM = 16;
// 4-bit weights at group size 32: weight rows from which the wave-per-tile kernel has the tiles to fill the chip
constexpr uint32_t kWt32MinN = 24576;
// rows of one pass of the single-row kernel
constexpr uint32_t kM1PassRows = 4;
// group size 64: rows taken by the single-row kernel (measured: 3 and 4 rows are faster on the matrix unit)
constexpr uint32_t kM1MaxRows = 2;
constexpr uint32_t kM1MaxRowsOther = 16;  // shapes the multi-row GEMV does not take: the alternative is the portable kernel

// What is fused around a matmul: the store epilogue (kind / ptr / dtype) and the RMSNorm prologue
// (norm_w [K] f16 and inv_rms [M] f32; both null = none).
struct Epilogue {
  int kind = EPI_NONE; const void* ptr = nullptr; int32_t dtype = RMLX_DTYPE_F16;
  const __half* norm_w = nullptr; const float* inv_rms = nullptr;
};

int32_t run_matmul_plain(const rmlx_qweight* qw, const void* x, int32_t x_dtype, uint32_t M, __half* out,
                         int32_t kernel, hipStream_t stream, const Epilogue& epi, bool* epi_done);

// Matmul plus optional store epilogue: fused in the register-weights GEMM and the single-row GEMV, a
// separate elementwise pass after every other kernel.
int32_t run_matmul(const rmlx_qweight* qw, const void* x, int32_t x_dtype, uint32_t M, __half* out,
                   int32_t kernel, hipStream_t stream, const Epilogue& epi = Epilogue()) {
  bool done = false;
  RMLX_TRY(run_matmul_plain(qw, x, x_dtype, M, out, kernel, stream, epi, &done));
  if (epi.kind != EPI_NONE && !done)
    RMLX_TRY(launch_epilogue(out, epi.kind, epi.ptr, epi.dtype, (size_t)M * qw->out_features, stream));
  return RMLX_OK;
}

int32_t run_matmul_plain(const rmlx_qweight* qw, const void* x, int32_t x_dtype, uint32_t M, __half* out,
                         int32_t kernel, hipStream_t stream, const Epilogue& epi, bool* epi_done) {
  uint32_t N, K;
  RMLX_TRY(checked_u32(qw->out_features, "out_features", &N));
  RMLX_TRY(checked_u32(qw->in_features, "in_features", &K));
  if (M == 0) return RMLX_OK;
  const bool ptr_ok = aligned16(qw->w) && aligned16(qw->s) && aligned16(qw->b) && aligned16(x);
  // (the 4-bit multi-row GEMV takes K in whole slabs of 128; the reference's kernel needs K % 512 == 0, quantized.rs:1603-1608)
  const bool can_qmv = ptr_ok && ((qw->bits == 4 && qmv_q4_supported(N, K, qw->group_size)) ||
                                  (qw->bits == 8 && qmv_q8_supported(N, K, qw->group_size)));
  const bool can_qmm_lds = ptr_ok && qmm_supported(N, K, qw->group_size, qw->bits);
  const bool can_qmm_rw = ptr_ok && qmm_rw_supported(N, K, qw->group_size, qw->bits);
  const bool can_qmm = can_qmm_lds || can_qmm_rw;
  // where the multi-row GEMV cannot take the shape (group size, K not a multiple of 512), the single-row
  // kernel also runs small batches, in passes of four rows -- and every batch where no GEMM takes the shape either (K not
  // a multiple of 256 at group sizes 32 and 128, K not a multiple of 64): after the first pass the weights come from
  // L2 / Infinity Cache, about 4 us per four rows at 4096 x 2880 against 40 us on the portable kernel
  const uint32_t m1_rows_other = can_qmm ? kM1MaxRowsOther : 65535u;
  const bool can_m1 = ptr_ok && qmv_m1_supported(N, K, qw->group_size, qw->bits) && M <= (can_qmv ? kM1MaxRows : m1_rows_other);
  // 2-bit weights: the single-row kernel of their own in passes of one row (the alternative is the portable kernel)
  const bool can_q2 = ptr_ok && qw->bits == 2 && M <= 65535u && qmv_q2_supported(N, K, qw->group_size);
  // 4-bit weights at group size 32: the wave-per-tile kernel streams the weights once per 8 rows
  const bool can_wt32 = ptr_ok && qw->bits == 4 && qw->group_size == 32 && qmv_wt_supported(N, K, 32, 8);
  // (its stores and the reads of the fused epilogue operand are 8- / 16-byte vectors)
  const bool can_qmm_k2 = ptr_ok && aligned16(out) && (epi.ptr == nullptr || aligned16(epi.ptr)) &&
                          qmm_k2_supported(N, K, qw->group_size, qw->bits);
  const bool can_qmm_k4 = ptr_ok && aligned16(out) && (epi.ptr == nullptr || aligned16(epi.ptr)) &&
                          qmm_k4_supported(N, K, qw->group_size, qw->bits);
  const bool can_qmm_k2_tall = can_qmm_k2 && qmm_k2_tall_supported(qw->group_size, qw->bits, x_dtype == RMLX_DTYPE_BF16);

  if (kernel == KERNEL_AUTO) {
    // The multi-row GEMV streams the weights once per pass of 8 rows (4-bit; two passes share a workgroup
    // up to 16 rows) or 16 rows (8-bit); the GEMM splits K over several workgroups per tile while its grid
    // is small, which puts its floor near 9 us at 4096 x 4096.  Measured crossovers (W = weight bytes):
    //   4-bit: GEMV up to 8 rows at every shape (N x K = 28672 x 4096: 18 against 22 us, 4096 x 14336: 13 against 18,
    //          2048 x 16384: 10 against 16, 1024 x 28672: 16 against 23); 9 to 16 rows while W <= 12 MiB or N <= 16384
    //          (4096 x 8192: 9 against 12 us, 4096 x 16384: 17 against 19, 8192 x 8192: 18 against 19, 12288 x 4096: 12.7 against
    //          16.2, 16384 x 4096: 15.3 against 16.6, weights cycled through more than 1 GiB; beyond that the GEMM's grid is
    //          large enough to win: 28672 x 4096 22 against 29 us);
    //          17 to 32 rows in passes of 8 while W <= 12 MiB: 4096 x 4096 8.8 / 9.1 / 9.3 us at 17 / 24 / 32 rows against 9.6 /
    //          9.9 / 10.3 on the GEMM; 9216 x 4096 at 32 rows: 20.9 against 17.3, so not beyond; over more than 4096 weight rows
    //          of fewer than 4096 values the GEMM's short k loop wins: 16384 x 1024 at 17 / 32 rows 8.6 / 9.3 against 6.2 us,
    //          8192 x 1536 7.4 / 8.2 against 7.0, 8192 x 2048 at 32 rows 9.2 against 8.3, while 4096 x 3072 keeps the passes, 7.9
    //          against 9.4, as do 4096 x 2048 and 2048 x 2048);
    //   8-bit: GEMV up to 16 rows while W < 48 MiB (4096 x 4096 is 16 MiB; at 12288 x 4096 the GEMM wins, 19 against 23 us).
    const uint64_t wbytes = (uint64_t)N * K * qw->bits / 8;
    // Without the register-weights GEMM (K not a multiple of 512) the alternative is the LDS-staged GEMM with
    // a floor of about 15 us: there the 4-bit GEMV keeps up to passes * W <= 48 MiB.
    const bool small_m = !can_qmm_rw ? M <= kQmvMaxM || (qw->bits == 4 && (uint64_t)((M + 7) / 8) * wbytes <= (48ull << 20))
                         : qw->bits == 4 ? M <= 8 || (M <= kQmvMaxM && (wbytes <= (12ull << 20) || N <= 16384)) ||
                                               (M <= 32 && wbytes <= (12ull << 20) && (N <= 4096 || K >= 4096))
                                         : (M <= kQmvMaxM && wbytes < (48ull << 20));
    // Shapes the K-split GEMV does not take (group size 32) run up to 16 rows on the single-row kernel in passes of four,
    // which streams the weights once per pass: with the register-weights GEMM as the alternative it keeps up to 4 rows
    // (4096 x 4096, 4-bit, group 32: 8.8 against 10.8 us at 4 rows, 11.4 against 11.1 at 8, 17.0 against 11.1 at 16;
    // 8-bit: 7.4 / 11.4, 12.6 / 11.4, 19.8 / 11.7; N = 9216, 8-bit: 14.2 / 20.6, 23.0 / 20.6, 36.8 / 21.2).  Over very
    // wide matrices the wave-per-tile kernel has enough tiles to fill the chip and takes 3 to 8 rows (N = 28672, 4-bit,
    // group 32: 22.8 us against 26.9 on the single-row kernel and 25.1 on the GEMM; N = 16384: 21.4 against 17.6 on the GEMM).
    // With only the LDS-staged GEMM as the alternative (K a multiple of 64 but not of 128) the passes keep up to 8 rows, and
    // up to 16 over matrices below 2 MiB; beyond, the fifth pass costs more than the GEMM (4-bit, 16 rows: 4864 x 896 13.2
    // against 10.6 us, 6912 x 1152 16.9 against 12.3).
    // Short rows make a pass dearer still (a whole-row wave leaves lanes idle below 2048 values): group size 32, 13824 x 1152,
    // 8 / 16 rows 17.5 / 29.9 against 13.0 us, 9728 x 896 at 8 rows 13.7 against 10.8; tiny matrices keep the passes (128 x 896,
    // 16 rows: about 7 against 9.9 us).
    // With its k loop split over more workgroups (launches of few tiles) the GEMM's floor is 11 to 14 us whatever K: from 9
    // rows on it wins over every matrix of 2 MiB or more (16 rows: 4096 x 2880 14.9 against 11.6, 8192 x 2880 25.1 against 14.0,
    // 8-bit 4096 x 2880 15.6 against 11.3; 8 rows: 9.9 against 11.4; but 2048 x 1088, 16 rows: 7.5 against 11.3), and from 5 rows
    // on over 4-bit matrices of 10 MiB or more (8192 x 2880, 6 rows: 15.1 against 13.6).
    const bool passes_lose = !can_qmv && !can_qmm_rw && can_qmm_lds &&
                             ((M > 8 && wbytes >= (2ull << 20)) || (M > 4 && K < 2048 && wbytes >= (3ull << 20)) ||
                              (M > 4 && qw->bits == 4 && wbytes >= (10ull << 20) && N <= 8192));
    const bool m1_first = can_m1 && !passes_lose && (can_qmv || !can_qmm_rw || M <= kM1PassRows);
    // One or two rows over short rows of a tall matrix: a wave of the single-row kernel owns a whole row, and a row of fewer
    // than 2048 values leaves part of its lanes without a load (896: 28 of 64), while the multi-row GEMV splits its tiles
    // over K.  Measured, single-row against multi-row, us: one row, 4-bit: 9728 x 896 5.4 / 4.4, 6912 x 1152 4.6 / 4.2,
    // 13824 x 1152 6.3 / 5.1, 8960 x 1536 5.4 / 5.2, 17920 x 1536 7.1 / 6.5, 16384 x 1024 6.3 / 4.8, 151936 x 896 37.7 / 16.1,
    // 151936 x 1536 39.0 / 25.7 (but 4864 x 896 3.6 / 4.3, 8192 x 1024 4.0 / 4.5, 8192 x 512 4.0 / 4.5, 6144 x 2048 3.9 / 4.7);
    // 65536 x 2048 19.8 / 17.7, 151936 x 2048 42.9 / 37.7 (32768 x 2048 a tie);
    // two rows, where the single-row kernel's second row costs a second set of dot products per weight: 9728 x 896 6.7 / 4.6,
    // 4864 x 896 5.2 / 4.5, 8192 x 512 6.1 / 4.6, 6144 x 2048 5.3 / 4.8, 16384 x 2048 9.6 / 6.8, 151936 x 896 58.3 / 15.8,
    // 8192 x 3072 7.6 / 5.5, 8192 x 4096 7.6 / 6.7, 12288 x 4096 10.2 / 8.7, 28672 x 4096 19.6 / 18.1, 8192 x 8192 12.3 / 11.5,
    // 151936 x 3072 79.1 / 54.2 (but 4096 x 1024 3.9 / 4.5, 4096 x 1536 4.0 / 4.1, 4096 x 8192 6.6 / 8.1, 4096 x 14336 10.7 /
    // 12.9: up to 4096 weight rows the single-row kernel keeps two); 8-bit, two rows: 8192 x 512 5.7 / 3.5,
    // 8192 x 1024 5.8 / 4.3, 16384 x 1024 7.6 / 6.4 (one row: the single-row kernel keeps up).  A fused epilogue or norm
    // stays with the single-row kernel, which applies it in the same launch.
    const bool plain = epi.kind == EPI_NONE && epi.ptr == nullptr && epi.norm_w == nullptr;
    bool short_rows = false;
    if (plain && can_qmv && can_m1 && M <= 2) {
      const uint64_t mib = 1ull << 20;
      if (qw->bits == 4 && M == 1) short_rows = (K < 2048 && wbytes * 2 >= (K % 512 != 0 ? 7 : 13) * mib) || (K == 2048 && wbytes >= 48 * mib);
      else if (qw->bits == 4) short_rows = K <= 8192 && N > 4096 && wbytes >= 2 * mib;
      else if (M == 2) short_rows = K <= 1024 && wbytes >= 4 * mib;
    }
    if (short_rows) kernel = KERNEL_QMV_ROWS;
    else if (can_wt32 && N >= kWt32MinN && M >= 3 && M <= 8) kernel = KERNEL_QMV_ROWS;
    else if ((can_qmv && small_m) || m1_first || can_q2) kernel = KERNEL_QMV;
    else if (can_qmm) kernel = KERNEL_QMM;
    else if (can_qmv) kernel = KERNEL_QMV;
    else kernel = KERNEL_GENERIC;
  } else if ((kernel == KERNEL_QMV && !can_qmv && !can_m1 && !can_q2) || (kernel == KERNEL_QMV_ROWS && !can_qmv && !can_wt32)) {
    return fail(RMLX_INVALID_SHAPE,
                "qmv kernel requires bits in {4,8}, group_size 64 (4-bit: or 128), N %% 16 == 0, K %% 128 == 0 (4-bit) or "
                "K %% 256 == 0 (8-bit) and 16-byte aligned buffers (N=%u K=%u bits=%u group_size=%u)",
                N, K, qw->bits, qw->group_size);
  } else if (kernel == KERNEL_QMM && !can_qmm) {
    return fail(RMLX_INVALID_SHAPE,
                "qmm kernel requires bits in {4,8}, N %% 64 == 0, 16-byte aligned buffers, K %% 64 == 0 and K >= 256 "
                "(N=%u K=%u bits=%u group_size=%u)", N, K, qw->bits, qw->group_size);
  } else if (kernel == KERNEL_QMM_LDS && !can_qmm_lds) {
    return fail(RMLX_INVALID_SHAPE,
                "the LDS-staged qmm kernel requires bits in {4,8}, N %% 64 == 0, K %% 64 == 0, K >= 256 and "
                "16-byte aligned buffers (N=%u K=%u bits=%u group_size=%u)", N, K, qw->bits, qw->group_size);
  } else if (kernel == KERNEL_QMM_BF16 && !(can_qmm_lds && qw->bits == 8 && qw->group_size == 64 && x_dtype == RMLX_DTYPE_BF16)) {
    return fail(RMLX_INVALID_SHAPE, "the bf16 MFMA GEMM takes Bfloat16 activations and 8-bit weights at group size 64 (got %s, bits=%u, "
                "group_size=%u)", dtype_name(x_dtype), qw->bits, qw->group_size);
  } else if (((kernel == KERNEL_QMM_K2 || kernel == KERNEL_QMM_K2_FLAT) && !can_qmm_k2) || (kernel == KERNEL_QMM_RW && !can_qmm_rw)) {
    return fail(RMLX_INVALID_SHAPE,
                "the register-weights qmm kernels require bits in {4,8}, N %% 64 == 0, K %% 512 == 0 (selector 8 at group size 64: "
                "K %% 128 == 0, K >= 512) and 16-byte aligned buffers (N=%u K=%u bits=%u group_size=%u)", N, K, qw->bits, qw->group_size);
  } else if (kernel == KERNEL_QMM_K2_TALL && !can_qmm_k2_tall) {
    return fail(RMLX_INVALID_SHAPE,
                "the 128 x 128 K-split qmm kernel requires bits in {4,8} (8-bit weights at group size 32 / 64: f16 or f32 "
                "activations), N %% 128 == 0, K %% 512 == 0 and 16-byte aligned buffers (N=%u K=%u bits=%u group_size=%u)",
                N, K, qw->bits, qw->group_size);
  } else if (kernel == KERNEL_QMM_K4 && !can_qmm_k4) {
    return fail(RMLX_INVALID_SHAPE,
                "the 32 x 64 K-split qmm kernel requires 4-bit weights at group size 64, N %% 64 == 0, K %% 2048 == 0 and 16-byte "
                "aligned buffers (N=%u K=%u bits=%u group_size=%u)", N, K, qw->bits, qw->group_size);
  } else if (kernel < 0 || kernel > KERNEL_QMM_K4) {
    return fail(RMLX_NOT_FOUND, "unknown kernel selector %d", kernel);
  }
  // The K-split GEMM (32x32x16 MFMAs, K split inside the workgroup).  64 x 128 tiles where that grid is one round over
  // most of the chip: measured 23.8 against 25.4 us at M = 512, 4096 x 4096 and 27.8 against 28.8 us at M = 128,
  // N = 12288 (8-bit).  128 x 128 tiles (every unpacked weight operand feeds four MFMAs) from 0.55 rounds of those on:
  // 29.6 against 35.5 us at M = 640, 37.0 against 41.4 us at M = 1024, 153 against 175 us at M = 4096 (4096 x 4096), 30.9
  // against 37.8 us at M = 192, N = 12288, 31.3 against 36.5 us at M = 256, N = 9216 (144 tiles).  With fewer tiles the
  // smaller tiles of the register-weights GEMM keep more CUs busy.
  uint32_t k2_tile_rows = kernel == KERNEL_QMM_K2_TALL ? 128 : kernel == KERNEL_QMM_K2_FLAT ? 32 : 64;
  // 32 x 64 tiles with K split four ways in the workgroup, where they make between half a round and one round over the chip:
  // with the tile-contiguous copy of the weights (rmlx_hip_qweight_set_gemm_layout) 13.4 against 15.7 us on the
  // register-weights GEMM at M = 128, 4096 x 4096 (14.1 / 17.5 at M = 32, N = 9216; 36.2 / 46.0 at M = 128, K = 14336);
  // without it only over long rows (K = 8192, M = 128: 26.1 / 28.0; K = 14336: 41.3 / 46.0; K = 4096: 15.6 / 15.7).
  if (kernel == KERNEL_QMM && can_qmm_k4 && M > 16) {
    const uint64_t t4 = (uint64_t)((M + 31) / 32) * (N / 64), cus = (uint64_t)ctx().num_cus;
    const bool packed = qw->gemm_packed != nullptr && N % 128 == 0;
    if (t4 <= cus && ((packed && t4 * 2 >= cus) || (K >= 8192 && t4 * 4 >= cus * 3))) kernel = KERNEL_QMM_K4;
  }
  if (kernel == KERNEL_QMM && can_qmm_k2) {
    const uint64_t tiles = (uint64_t)((M + 63) / 64) * (N / 128), tall = (uint64_t)((M + 127) / 128) * (N / 128);
    const uint64_t cus = (uint64_t)ctx().num_cus;
    // (a tile height only while at most a quarter of its rows is padding: 16 rows on 128-row tiles over a very wide
    // matrix measured 150 against 103 us on the register-weights GEMM, N = 151936)
    const bool fits64 = (uint64_t)((M + 63) / 64) * 64 * 3 <= (uint64_t)M * 4, fits128 = (uint64_t)((M + 127) / 128) * 128 * 3 <= (uint64_t)M * 4;
    if (fits64 && tiles * 10 >= cus * 7 && tiles <= cus) kernel = KERNEL_QMM_K2;
    else if (fits128 && can_qmm_k2_tall && tall * 20 >= cus * 11) { kernel = KERNEL_QMM_K2; k2_tile_rows = 128; }
    // 32 x 128 tiles: one round of them takes about 18.5 us at K = 4096 whatever their number (the length of the k loop);
    // the register-weights GEMM is faster while its 32 x 64 tiles fit one round over the chip (15.6 us at M = 128,
    // 4096 x 4096) and slower once it has to take larger tiles (M = 160: 24.4 us, M = 256: 21.1 against 19.3;
    // N = 9216, M = 64: 25.0 against 19.8).  Where the 32-row tiles need more than one round, one round of 64-row tiles
    // still wins (N = 9216, M = 128: 22.2 against 23.7 us).  Measured at K = 4096 only, so longer rows keep the other
    // kernels; so do 8-bit weights over wide matrices (N = 12288, M = 64: 28.6 against 27.7 us).
    else if (K <= 4096 && qmm_rw_tile_work(M, N, K, qw->group_size, qw->bits) >= 16 && !(qw->bits == 8 && N > 8192)) {
      if (M > 32 && (uint64_t)((M + 31) / 32) * (N / 128) <= cus) { kernel = KERNEL_QMM_K2; k2_tile_rows = 32; }
      else if (fits64 && tiles <= cus) kernel = KERNEL_QMM_K2;
    }
  }
  if (kernel == KERNEL_QMM_K2_TALL || kernel == KERNEL_QMM_K2_FLAT) kernel = KERNEL_QMM_K2;
  if (kernel == KERNEL_QMM_RW) kernel = KERNEL_QMM;

  // RMSNorm prologue: fused into the single-row GEMV for one or two rows (while it stages the activations);
  // every other case gets the normalised activations from a pass of its own.
  const __half* norm_w = epi.norm_w;
  const float* inv_rms = epi.inv_rms;
  Scratch normed;
  if (norm_w != nullptr && !(kernel == KERNEL_QMV && can_m1 && qmv_m1_fuses_norm(M, K, qw->bits))) {
    RMLX_TRY(normed.alloc((size_t)M * K * sizeof(__half), stream));
    RMLX_TRY(launch_norm_rows(x, x_dtype, norm_w, inv_rms, M, K, static_cast<__half*>(normed.ptr), stream));
    x = normed.ptr;
    x_dtype = RMLX_DTYPE_F16;
    norm_w = nullptr;
  }

  if (kernel == KERNEL_QMM_K4) {
    Scratch cast;
    const void* xk = x;
    int32_t xk_dtype = x_dtype;
    if (x_dtype == RMLX_DTYPE_F32) {
      xk_dtype = RMLX_DTYPE_F16;
      RMLX_TRY(cast.alloc((size_t)M * K * sizeof(__half), stream));
      RMLX_TRY(launch_cast_to_f16(x, x_dtype, static_cast<__half*>(cast.ptr), (size_t)M * K, stream));
      xk = cast.ptr;
    }
    QmmArgs a{qw->w, qw->s, qw->b, xk, xk_dtype, out, M, N, K, qw->bits, nullptr, 0, epi.kind, epi.ptr, epi.dtype};
    a.w_packed = qw->gemm_packed;
    *epi_done = true;
    return launch_qmm_k4(a, qw->group_size, stream);
  }
  if (kernel == KERNEL_QMM_K2) {
    Scratch cast;
    const void* xk = x;
    int32_t xk_dtype = x_dtype;
    if (x_dtype == RMLX_DTYPE_F32) {
      xk_dtype = RMLX_DTYPE_F16;
      RMLX_TRY(cast.alloc((size_t)M * K * sizeof(__half), stream));
      RMLX_TRY(launch_cast_to_f16(x, x_dtype, static_cast<__half*>(cast.ptr), (size_t)M * K, stream));
      xk = cast.ptr;
    }
    QmmArgs a{qw->w, qw->s, qw->b, xk, xk_dtype, out, M, N, K, qw->bits, nullptr, 0, epi.kind, epi.ptr, epi.dtype};
    a.w_packed = qw->gemm_packed;
    *epi_done = true;
    return launch_qmm_k2(a, qw->group_size, k2_tile_rows, stream);
  }
  // Group size 32 with a K tail (K in whole blocks of 128, not of 512): the register-weights GEMM has two small tile shapes
  // for this group size and pads its last round; from 256 rows on the LDS-staged GEMM with its 128-row tiles is ahead
  // (13824 x 1152: 256 / 512 / 2048 rows 21.6 / 38.9 / 132 against 25.9 / 51.5 / 170 us; 9728 x 896: 17.8 / 26.3 / 77 against
  // 20.0 / 29.9 / 96; 4096 x 11008 at 2048 rows: a tie), below that the register-weights GEMM (32 rows: 8.7 against 12.6 us).
  const bool lds_first = kernel == KERNEL_QMM && can_qmm_lds && qw->group_size == 32 && K % 512 != 0 && M >= 256;
  if (kernel == KERNEL_QMM && can_qmm_rw && !lds_first) {
    // Register-weights GEMM: f16 / bf16 activations straight from the row-major matrix, no workspace
    // (bf16 -> f16 inside the kernel: exact for normal-range values, and f16 weights keep 11
    // significant bits); f32 activations are cast first.
    Scratch cast;
    const void* xk = x;
    int32_t xk_dtype = x_dtype;
    if (x_dtype == RMLX_DTYPE_F32) {
      xk_dtype = RMLX_DTYPE_F16;
      RMLX_TRY(cast.alloc((size_t)M * K * sizeof(__half), stream));
      RMLX_TRY(launch_cast_to_f16(x, x_dtype, static_cast<__half*>(cast.ptr), (size_t)M * K, stream));
      xk = cast.ptr;
    }
    Scratch partial;  // f32 partial sums when the launch is split over K
    const size_t partial_bytes = qmm_rw_workspace_bytes(M, N, K, qw->group_size, qw->bits);
    if (partial_bytes != 0) RMLX_TRY(partial.alloc(partial_bytes, stream));
    QmmArgs a{qw->w, qw->s, qw->b, xk, xk_dtype, out, M, N, K, qw->bits, partial.ptr, 0, epi.kind, epi.ptr, epi.dtype};
    *epi_done = true;
    return launch_qmm_rw(a, qw->group_size, stream);
  }
  if (kernel == KERNEL_QMM || kernel == KERNEL_QMM_BF16 || kernel == KERNEL_QMM_LDS) {
    // The LDS-staged GEMM re-lays the activations out in MFMA operand order first (dtype cast fused in).
    // By default everything is multiplied in f16: bf16 -> f16 is exact for normal-range values and
    // f16 weights keep 11 significant bits.  The bf16 MFMA variant (weights rounded to 8 bits)
    // passes the tolerance with little margin, so it has to be asked for explicitly.
    Scratch ws;
    RMLX_TRY(ws.alloc(qmm_workspace_bytes(M, K, N), stream));
    QmmArgs a{qw->w, qw->s, qw->b, x, x_dtype, out, M, N, K, qw->bits, ws.ptr, kernel == KERNEL_QMM_BF16 ? 1 : 0};
    a.group_size = qw->group_size;
    a.workspace_has_partials = true;
    return launch_qmm(a, stream);
  }

  // Activations of the other kernels: f16 (f32 / bf16 are cast first) -- except that the single-row kernel converts bf16
  // activations itself while it stages them, for one or two rows in one pass: a decoding step of a bf16 model pays no
  // cast launch in front of every matmul (same conversion, same bits).
  const bool m1_bf16 = kernel == KERNEL_QMV && !can_q2 && can_m1 && (x_dtype == RMLX_DTYPE_BF16 || x_dtype == RMLX_DTYPE_F32) &&
                       norm_w == nullptr && qmv_m1_fuses_norm(M, K, qw->bits);  // (f32 rows likewise)
  // (so do the multi-row GEMVs, for every row count they take)
  const bool rows_bf16 = x_dtype == RMLX_DTYPE_BF16 && (qw->bits == 4 || qw->bits == 8) && can_qmv && !can_q2 &&
                         ((kernel == KERNEL_QMV && !can_m1) || (kernel == KERNEL_QMV_ROWS && !can_wt32));
  Scratch cast;
  const void* xk = x;
  if (x_dtype != RMLX_DTYPE_F16 && !m1_bf16 && !rows_bf16) {
    RMLX_TRY(cast.alloc((size_t)M * K * sizeof(__half), stream));
    RMLX_TRY(launch_cast_to_f16(x, x_dtype, static_cast<__half*>(cast.ptr), (size_t)M * K, stream));
    xk = cast.ptr;
  }

  if (kernel == KERNEL_QMV && can_q2)
    return launch_qmv_q2(qw->w, qw->s, qw->b, static_cast<const __half*>(xk), out, M, N, K, qw->group_size, stream);
  if (kernel == KERNEL_QMV && can_m1) {
    *epi_done = true;
    return launch_qmv_m1(qw->w, qw->s, qw->b, static_cast<const __half*>(xk), out, M, N, K, qw->group_size, qw->bits,
                         epi.kind, epi.ptr, epi.dtype, norm_w, norm_w != nullptr ? inv_rms : nullptr, stream,
                         !m1_bf16 ? 0 : (x_dtype == RMLX_DTYPE_BF16 ? 1 : 2));
  }
  if (kernel == KERNEL_QMV_ROWS && can_wt32) {
    QmvArgs a{};
    a.w0 = qw->w; a.s0 = qw->s; a.b0 = qw->b;
    a.N = N; a.K = K;
    a.x = static_cast<const __half*>(xk);
    a.out = out; a.ld_out = N; a.M = M; a.group_size = 32;
    return launch_qmv_wt(a, 8, stream);
  }
  if (kernel == KERNEL_QMV_ROWS) kernel = KERNEL_QMV;
  if (kernel == KERNEL_QMV && qw->bits == 8)
    return launch_qmv_q8(qw->w, qw->s, qw->b, static_cast<const __half*>(xk), out, M, N, K, qw->group_size, stream, rows_bf16 ? 1 : 0);
  if (kernel == KERNEL_QMV) {
    QmvArgs a{};
    a.w0 = qw->w; a.s0 = qw->s; a.b0 = qw->b;
    a.N = N; a.K = K;
    a.x = static_cast<const __half*>(xk);
    a.out = out; a.ld_out = N; a.M = M; a.group_size = qw->group_size;
    a.x_bf16 = rows_bf16 ? 1 : 0;
    return launch_qmv_q4(a, stream);
  }
  GenericArgs g{qw->w, qw->s, qw->b, static_cast<const __half*>(xk), out, nullptr, 0, M, N, K,
                qw->group_size, qw->bits, 1};
  return launch_generic(g, stream);
}

int32_t check_x_dtype(const char* who, int32_t dt) {
  if (dt != RMLX_DTYPE_F32 && dt != RMLX_DTYPE_F16 && dt != RMLX_DTYPE_BF16)
    return fail(RMLX_INVALID_SHAPE, "%s requires Float16 or Float32 input, got %s", who, dtype_name(dt));
  return RMLX_OK;
}

int32_t check_out(const char* who, size_t have, size_t need) {
  if (have < need) return fail(RMLX_INVALID_SHAPE, "%s: output buffer too small: %zu bytes < expected %zu bytes", who, have, need);
  return RMLX_OK;
}

struct ExpertShapes {
  uint32_t E, D, I;
  bool fused;
  bool portable;  // weights the streaming kernels do not take: the portable kernels run the block
  bool gemm;      // the grouped GEMM takes them too (batches with many rows per expert)
  bool gemm_lds;  // the LDS-staged GEMM's grouped form takes them (dimensions in multiples of 64: what is left without `gemm`)
  uint32_t bits;  // of the gate weight
  bool gemm64;    // group size 64 (the 16-row tile is built for it only)
  uint32_t gemm_min_rows;  // of the gate weight's handle (rmlx_hip_qweight_set_expert_gemm_min_rows)
  uint32_t stream_kernel;  // of the gate weight's handle (rmlx_hip_qweight_set_expert_stream_kernel)
  bool wave_tiles;         // the wave-per-tile streaming kernel takes the three projections (4-bit, group size 64)
  bool wave_down;          // ... takes the down projection over chunks of 8 rows
  bool wave_gs32;          // 4-bit weights with group size 32: the wave-per-tile kernel is the only streaming kernel for them
};

// gather_qmm takes raw buffers, so its GEMV / grouped-GEMM crossover is a constant: every entry has exactly
// m_per_batch rows, the streaming GEMV wastes nothing up to a full chunk of 8 rows, and the GEMM wins from 9 rows on.
constexpr uint32_t kGatherGemmMinRows = 9;
// routed block: the form without grouping (every assignment a row of its own) is never taken beyond this many assignments
constexpr uint32_t kDirectMaxAssignments = 128;
// twice the average rows per expert from which the gate / up projection of a decode-sized batch runs in two launches, the
// experts split by their row count (moe_grouped_impl)
// (E = 128, top-8, D = 4096, I = 1536, against K-split gate / up over chunks of 8: 88 tokens 322 / 308 us, 96 tokens 319 / 324,
// 128 tokens 353 / 363, 160 tokens 387 / 402 and 400 on the grouped GEMM, 192 tokens 400 / 397 on the GEMM)
constexpr uint32_t kSplitMinRows2 = 12;
// (experts without a grouped fast path, 2-bit ones among them: streaming an expert per assignment stays far ahead of the
// portable kernels up to this many assignments)
constexpr uint32_t kUngroupedOnlyMaxAssignments = 8192;
// The form without grouping streams an expert once per assignment instead of once per distinct expert of the batch (at
// about 6 against 5 TB/s, and without the grouping launch): worth it while the assignments are at most 1.3 x the distinct
// experts a uniform router picks, E (1 - (1 - K/E)^T).  Measured at E = 128, top-8: 9 tokens 127 against 137 us, 10 tokens
// 141 against 141, 12 tokens 170 against 162; 8-bit experts (three launches): 10 / 11 tokens 267 / 301 against 281 / 309 us, 12
// tokens 321 against 314: 1.37 x.
bool ungrouped_pays(uint32_t T, uint32_t E, uint32_t K, uint32_t bits) {
  if (E == 0 || K > E) return false;
  const double distinct = E * (1.0 - std::pow(1.0 - (double)K / E, (double)T));
  return (uint64_t)T * K <= kDirectMaxAssignments && (double)T * K <= (bits == 8 ? 1.37 : 1.3) * distinct;
}
enum { GATHER_AUTO = 0, GATHER_STREAM = 1, GATHER_GEMM = 2, GATHER_PORTABLE = 3 };

int32_t check_expert_weights(const char* who, const rmlx_qweight* gate, const rmlx_qweight* up,
                             const rmlx_qweight* down, ExpertShapes* sh) {
  if (gate == nullptr || down == nullptr) return fail(RMLX_INVALID_SHAPE, "%s: gate and down weights are required", who);
  const bool fused = up == nullptr;
  size_t E = gate->n_experts, D = gate->in_features, I = fused ? gate->out_features / 2 : gate->out_features;
  if (fused && gate->out_features % 2 != 0) return fail(RMLX_INVALID_SHAPE, "%s: fused gate/up weight needs an even row count", who);
  if (!fused && (up->n_experts != E || up->in_features != D || up->out_features != I))
    return fail(RMLX_INVALID_SHAPE, "%s: up weight shape mismatch", who);
  if (down->n_experts != E || down->in_features != I || down->out_features != D)
    return fail(RMLX_INVALID_SHAPE, "%s: down weight must be [%zu, %zu, %zu], got [%zu, %zu, %zu]", who, E, D, I,
                down->n_experts, down->out_features, down->in_features);
  const rmlx_qweight* all[3] = {gate, up, down};
  bool fast = true, uniform = true;  // uniform: one bit width and one group size, 16-byte aligned buffers
  for (const rmlx_qweight* q : all) {
    if (q == nullptr) continue;
    if (q->bits != 2 && q->bits != 4 && q->bits != 8)
      return fail(RMLX_NOT_FOUND, "%s: no kernel for %u-bit expert weights (2, 4 and 8 are implemented; 3- and 6-bit weights run on the matmul entry points)", who, q->bits);
    // the K-split streaming kernels take 4- and 8-bit weights with group size 64 or 128, the same width for all three
    // projections (gate and up share one launch); 4-bit weights with group size 32 run on the wave-per-tile kernel
    const bool gs_ok = (q->bits == 4 || q->bits == 8) && (q->group_size == 64 || q->group_size == 128);
    if (!gs_ok || q->bits != gate->bits || !aligned16(q->w) || !aligned16(q->s) || !aligned16(q->b)) fast = false;
    if (q->bits != gate->bits || q->group_size != gate->group_size || !aligned16(q->w) || !aligned16(q->s) || !aligned16(q->b))
      uniform = false;
  }
  RMLX_TRY(checked_u32(E, "num_experts", &sh->E));
  RMLX_TRY(checked_u32(D, "hidden_dim", &sh->D));
  RMLX_TRY(checked_u32(I, "intermediate_dim", &sh->I));
  if (gate->bits == 8) {
    if (!qmv_q8_supported(sh->I, sh->D, gate->group_size) || !qmv_q8_supported(sh->D, sh->I, down->group_size)) fast = false;
  } else if (!qmv_q4_supported(sh->I, sh->D, 64) || !qmv_q4_supported(sh->D, sh->I, 64)) {
    fast = false;
  }
  if (up != nullptr && up->group_size != gate->group_size) fast = false;
  sh->fused = fused;
  sh->bits = gate->bits;
  sh->gemm64 = gate->group_size == 64;
  sh->gemm_min_rows = gate->expert_gemm_min_rows;
  sh->stream_kernel = gate->expert_stream_kernel;
  const bool q4_gs64 = fast && gate->bits == 4 && gate->group_size == 64 && down->group_size == 64;
  sh->wave_tiles = q4_gs64 && qmv_wt_supported(sh->I, sh->D, 64, 16) && qmv_wt_supported(sh->D, sh->I, 64, 16);
  sh->wave_down = q4_gs64 && qmv_wt_supported(sh->D, sh->I, 64, 8);
  // 4-bit experts with group size 32: both projections on the wave-per-tile kernel, chunks of 8 rows
  sh->wave_gs32 = uniform && gate->bits == 4 && gate->group_size == 32 && qmv_wt_supported(sh->I, sh->D, 32, 8) &&
                  qmv_wt_supported(sh->D, sh->I, 32, 8);
  if (sh->wave_gs32) fast = true;
  sh->portable = !fast;
  // the grouped GEMM also takes group sizes the streaming kernels do not (32; 128 at 8 bits)
  sh->gemm = uniform && qmm_rw_grouped_supported(sh->I, sh->D, gate->group_size, gate->bits) &&
             qmm_rw_grouped_supported(sh->D, sh->I, gate->group_size, gate->bits);
  sh->gemm_lds = uniform && (gate->bits == 4 || gate->bits == 8) && qmm_supported(sh->I, sh->D, gate->group_size, gate->bits) &&
                 qmm_supported(sh->D, sh->I, gate->group_size, gate->bits);
  return RMLX_OK;
}

// Rows per tile when `rows` positions over at most `groups` experts are multiplied by the grouped GEMM (half
// tiles while an expert has 24 rows or fewer on average: less padding, more workgroups per CU), else 0
uint32_t expert_gemm_tile_rows(const ExpertShapes& sh, uint64_t rows, uint64_t groups) {
  uint32_t min_rows = sh.gemm_min_rows;
  // 8-bit experts cross over at an eighth of the threshold, rounded down (measured: from one row per expert on, against
  // 10 for 4-bit ones: with 16-row tiles the GEMM streams 8-bit weights faster than the 8-bit GEMV does)
  if (sh.bits == 8 && min_rows != 0) min_rows = min_rows >= 16 ? min_rows / 8 : 1;
  // experts that no streaming kernel takes: the alternative streams an expert once per assignment, the GEMM once
  if (sh.portable && min_rows != 0) min_rows = 1;
  if (!sh.gemm || min_rows == 0 || groups == 0 || rows < (uint64_t)min_rows * groups) return 0;
  if (rows <= 7 * groups && sh.gemm64) return 16u;  // (four-wave workgroups, 16 rows: built for group size 64)
  return rows <= 24 * groups ? 32u : kGroupedTileRows;
}

// Which streaming kernel runs the two projections of a decode-sized batch, and over chunks of how many rows.
// gate_up / down: 0 = the K-split kernel (qmv.hip), else the wave-per-tile kernel (qmv_wt.hip) with chunks of that many
// rows (8 or 16).  Selector of the gate handle: 1 = K-split for both, 2 / 3 = wave per tile for both with chunks of 8 / 16
// rows, 0 (the library's choice) and 4 = K-split for gate / up, wave per tile for a down projection whose rows are shorter
// than 4096 (measured at D = 4096, I = 1536: the block takes 254 against 269 us at T = 32 and 348 against 368 us at
// T = 128; over chunks of 8 rows a wave-per-tile gate / up projection is 30 % slower than the K-split one); 5 = as 4, the gate /
// up projection in two launches with the experts split by their row count (moe_grouped_impl; the routed block only).
struct StreamPlan { uint32_t gate_up, down, chunk_rows; };
// rows / groups: the assignments of the call and the experts (or host-side groups) they spread over
StreamPlan expert_stream_plan(const ExpertShapes& sh, size_t rows, size_t groups) {
  StreamPlan pl{0, 0, 8};
  if (sh.wave_gs32) return StreamPlan{8, 8, 8};
  if (sh.stream_kernel == 1) return pl;
  if (sh.stream_kernel == 2 && sh.wave_tiles) pl = StreamPlan{8, 8, 8};
  else if (sh.stream_kernel == 3 && sh.wave_tiles) pl = StreamPlan{16, 16, 16};
  // (Chunks of 16 rows are not picked here: at D = 4096, I = 1536, E = 128 they take 322 us at 8 rows per expert on average
  // against 345 us for K-split gate / up with the wave-per-tile down projection - while no expert has more than 16 rows.
  // One that has adds a seventh round of workgroups to their six: 384 us.  Under uniform random routing that is the case
  // for 11 / 23 / 38 % of the batches at 7 / 7.5 / 8 rows per expert, which makes the expectation a tie.  A caller whose
  // router bounds the rows per expert selects them with selector 3.)
  else if (sh.wave_down && sh.I < 4096) pl.down = 8;
  return pl;
}

// Gate / up projection in two launches over two chunk tables (see launch_moe_sort): tab = first table, cap_small entries, then
// the second, cap_big entries; n[2] = their lengths on the device.
struct SplitTables { const uint32_t* tab; const uint32_t* n; uint32_t cap_small, cap_big; };

// The same block on the portable kernels, for expert weights the streaming GEMV does not take (2-bit,
// group size 32, 8-bit at group size 128, dimensions that are no multiples of 512 (4-bit) or 256 / 16
// (8-bit)) in batches below the grouped GEMM's threshold: every position multiplies with its own expert's rows.  x: f16 [positions, D] (already gathered); expert_of: device u32 [positions]; y: f16 [positions, D].
int32_t run_expert_ffn_portable(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                                const ExpertShapes& sh, const __half* x, const uint32_t* expert_of, uint32_t positions,
                                __half* y, hipStream_t stream) {
  Scratch gu, h;
  const uint32_t gu_cols = 2 * sh.I;
  RMLX_TRY(gu.alloc((size_t)positions * gu_cols * sizeof(__half), stream));
  RMLX_TRY(h.alloc((size_t)positions * sh.I * sizeof(__half), stream));
  __half* g_out = static_cast<__half*>(gu.ptr);
  if (sh.fused) {  // one weight of 2I rows per expert, gate rows first: [positions, 2I]
    GenericArgs a{gate->w, gate->s, gate->b, x, g_out, expert_of, 1, positions, gu_cols, sh.D, gate->group_size, gate->bits, sh.E};
    RMLX_TRY(launch_generic(a, stream));
    RMLX_TRY(launch_silu_gate_strided(g_out, g_out + sh.I, gu_cols, static_cast<__half*>(h.ptr), positions, sh.I, stream));
  } else {         // [positions, I] twice
    __half* u_out = g_out + (size_t)positions * sh.I;
    GenericArgs a{gate->w, gate->s, gate->b, x, g_out, expert_of, 1, positions, sh.I, sh.D, gate->group_size, gate->bits, sh.E};
    GenericArgs b{up->w, up->s, up->b, x, u_out, expert_of, 1, positions, sh.I, sh.D, up->group_size, up->bits, sh.E};
    RMLX_TRY(launch_generic(a, stream));
    RMLX_TRY(launch_generic(b, stream));
    RMLX_TRY(launch_silu_gate(g_out, u_out, static_cast<__half*>(h.ptr), (size_t)positions * sh.I, stream));
  }
  GenericArgs d{down->w, down->s, down->b, static_cast<const __half*>(h.ptr), y, expert_of, 1, positions, sh.D, sh.I,
                down->group_size, down->bits, sh.E};
  return launch_generic(d, stream);
}

// Routing fused in front of the grouping (decode-sized batches): f32 logits [T, E], optional f32 bias [E];
// the picks and their weights are written to idx_out / w_out.
struct FusedRoute { const float* logits; const float* bias; uint32_t* idx_out; float* w_out; };

// The fused gate / up launch of the streaming kernels: both matrices (halves of one stacked buffer, or two), x -> h.
QmvArgs gate_up_args(const rmlx_qweight* gate, const rmlx_qweight* up, const ExpertShapes& sh, const __half* x, __half* h) {
  const uint32_t per = 32 / gate->bits;  // values per u32 word: 8 (4-bit) or 4 (8-bit)
  QmvArgs a{};
  a.w0 = gate->w; a.s0 = gate->s; a.b0 = gate->b;
  if (sh.fused) {
    a.w1 = gate->w + (size_t)sh.I * (sh.D / per);
    a.s1 = gate->s + (size_t)sh.I * (sh.D / gate->group_size);
    a.b1 = gate->b + (size_t)sh.I * (sh.D / gate->group_size);
  } else {
    a.w1 = up->w; a.s1 = up->s; a.b1 = up->b;
  }
  const size_t rows_per_expert = sh.fused ? 2 * (size_t)sh.I : sh.I;
  a.N = sh.I; a.K = sh.D;
  a.expert_stride_w = rows_per_expert * (sh.D / per);
  a.expert_stride_s = rows_per_expert * (sh.D / gate->group_size);
  a.group_size = gate->group_size;
  a.x = x;
  a.out = h; a.ld_out = sh.I; a.out_f32 = 0; a.dual = 1;
  return a;
}

// Both projections of these experts run on the single-row kernels (one row per expert): 4- or 8-bit, one format for the
// three matrices, any group size, the shapes of the single-row GEMV, aligned buffers.
bool single_row_experts(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down, const ExpertShapes& sh) {
  if ((gate->bits != 4 && gate->bits != 8) || down->bits != gate->bits) return false;
  if (up != nullptr && (up->bits != gate->bits || up->group_size != gate->group_size)) return false;
  for (const rmlx_qweight* q : {gate, up, down})
    if (q != nullptr && (!aligned16(q->w) || !aligned16(q->s) || !aligned16(q->b))) return false;
  return qmv_m1_gate_up_supported(sh.I, sh.D, gate->group_size, gate->bits) && qmv_m1_supported(sh.D, sh.I, down->group_size, down->bits);
}

// gate/up + SwiGLU then down, over a device chunk table.  h: f16 [positions, I] scratch.
// The expert FFN over row tiles of 64 rows of one expert each on the grouped form of the LDS-staged GEMM (expert dimensions in
// multiples of 64 that the register-weights grouped GEMM does not take): gate / up (one stacked matrix, or two launches), SwiGLU
// as a pass of its own, down.  x: f16 rows reached through row_map (nullable); y16: f16 [positions, D] in the table's row order.
int32_t run_expert_ffn_lds(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down, const ExpertShapes& sh,
                           const __half* x, const uint32_t* row_map, const uint32_t* tile_tab, const uint32_t* n_tiles,
                           uint32_t max_tiles, uint32_t positions, __half* y16, hipStream_t s, Arena* arena, uint32_t tile_rows = 64) {
  const uint32_t per = 32 / gate->bits, gs = gate->group_size;
  Scratch ws, gu, h;
  const uint32_t kmax = sh.D > sh.I ? sh.D : sh.I;
  RMLX_TRY(ws.alloc(qmm_grouped_workspace_bytes(max_tiles, kmax, tile_rows), s, arena));
  RMLX_TRY(gu.alloc((size_t)positions * 2 * sh.I * 2, s, arena));
  RMLX_TRY(h.alloc((size_t)positions * sh.I * 2, s, arena));
  GroupedQmmArgs a{};
  a.w = gate->w; a.s = gate->s; a.b = gate->b;
  a.K = sh.D; a.bits = gate->bits; a.group_size = gs;
  a.x = x; a.row_map = row_map; a.out_f32 = 0;
  a.tile_tab = tile_tab; a.n_tiles_dev = n_tiles; a.max_tiles = max_tiles; a.tile_rows = tile_rows;
  __half* g_out = static_cast<__half*>(gu.ptr);
  if (sh.fused) {  // one stacked matrix per expert: [positions, 2I] = (gate | up)
    a.N = 2 * sh.I;
    a.expert_stride_w = (uint64_t)2 * sh.I * (sh.D / per); a.expert_stride_s = (uint64_t)2 * sh.I * (sh.D / gs);
    a.out = g_out;
    RMLX_TRY(launch_qmm_grouped(a, ws.ptr, s));
    RMLX_TRY(launch_silu_gate_strided(g_out, g_out + sh.I, 2 * sh.I, static_cast<__half*>(h.ptr), positions, sh.I, s));
  } else {
    a.N = sh.I;
    a.expert_stride_w = (uint64_t)sh.I * (sh.D / per); a.expert_stride_s = (uint64_t)sh.I * (sh.D / gs);
    a.out = g_out;
    RMLX_TRY(launch_qmm_grouped(a, ws.ptr, s));
    a.w = up->w; a.s = up->s; a.b = up->b; a.out = g_out + (size_t)positions * sh.I;
    RMLX_TRY(launch_qmm_grouped(a, ws.ptr, s));
    RMLX_TRY(launch_silu_gate(g_out, g_out + (size_t)positions * sh.I, static_cast<__half*>(h.ptr), (size_t)positions * sh.I, s));
  }
  GroupedQmmArgs d{};
  d.w = down->w; d.s = down->s; d.b = down->b;
  d.N = sh.D; d.K = sh.I; d.bits = down->bits; d.group_size = gs;
  d.expert_stride_w = (uint64_t)sh.D * (sh.I / per); d.expert_stride_s = (uint64_t)sh.D * (sh.I / gs);
  d.x = static_cast<const __half*>(h.ptr); d.row_map = nullptr; d.out = y16; d.out_f32 = 0;
  d.tile_tab = tile_tab; d.n_tiles_dev = n_tiles; d.max_tiles = max_tiles; d.tile_rows = tile_rows;
  return launch_qmm_grouped(d, ws.ptr, s);
}

int32_t run_expert_ffn(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                       const ExpertShapes& sh, const __half* x, const uint32_t* row_map,
                       const uint32_t* chunk_tab, const uint32_t* n_chunks, uint32_t max_chunks, __half* h,
                       void* y, int y_f32, uint32_t gemm_tile_rows, const StreamPlan& plan, hipStream_t stream,
                       const SplitTables* split = nullptr) {
  const uint32_t per = 32 / gate->bits;  // values per u32 word: 8 (4-bit) or 4 (8-bit)
  if (gemm_tile_rows != 0) {  // the table holds row tiles of that many rows and n_chunks its length
    const uint32_t gs = gate->group_size;  // one group size for the three projections (ExpertShapes::gemm)
    GroupedQmmArgs a{};
    a.w = gate->w; a.s = gate->s; a.b = gate->b;
    if (sh.fused) {
      a.w1 = gate->w + (size_t)sh.I * (sh.D / per);
      a.s1 = gate->s + (size_t)sh.I * (sh.D / gs);
      a.b1 = gate->b + (size_t)sh.I * (sh.D / gs);
    } else {
      a.w1 = up->w; a.s1 = up->s; a.b1 = up->b;
    }
    const size_t rows = sh.fused ? 2 * (size_t)sh.I : sh.I;
    a.N = sh.I; a.K = sh.D; a.bits = gate->bits; a.group_size = gs;
    a.expert_stride_w = rows * (sh.D / per);
    a.expert_stride_s = rows * (sh.D / gs);
    a.x = x; a.row_map = row_map; a.out = h; a.out_f32 = 0;
    a.tile_tab = chunk_tab; a.n_tiles_dev = n_chunks; a.max_tiles = max_chunks; a.tile_rows = gemm_tile_rows;
    RMLX_TRY(launch_qmm_rw_grouped(a, stream));
    GroupedQmmArgs d{};
    d.w = down->w; d.s = down->s; d.b = down->b;
    d.N = sh.D; d.K = sh.I; d.bits = down->bits; d.group_size = gs;
    d.expert_stride_w = (size_t)sh.D * (sh.I / per);
    d.expert_stride_s = (size_t)sh.D * (sh.I / gs);
    d.x = h; d.row_map = nullptr; d.out = y; d.out_f32 = y_f32;
    d.tile_tab = chunk_tab; d.n_tiles_dev = n_chunks; d.max_tiles = max_chunks; d.tile_rows = gemm_tile_rows;
    return launch_qmm_rw_grouped(d, stream);
  }
  QmvArgs a = gate_up_args(gate, up, sh, x, h);
  a.row_map = row_map;
  a.chunk_tab = chunk_tab; a.n_chunks_dev = n_chunks; a.max_chunks = max_chunks; a.mr = 8;
  // (the table holds chunks of at most plan.chunk_rows rows)
  if (split != nullptr) {
    // experts with up to 8 rows: one chunk each on the K-split kernel; the others in chunks of up to 16 rows on the
    // wave-per-tile kernel with two activation images, which streams their weights once
    a.chunk_tab = split->tab; a.n_chunks_dev = split->n; a.max_chunks = split->cap_small;
    RMLX_TRY(launch_qmv_q4(a, stream));
    a.chunk_tab = split->tab + 3 * (size_t)split->cap_small; a.n_chunks_dev = split->n + 1; a.max_chunks = split->cap_big;
    RMLX_TRY(launch_qmv_wt(a, 16, stream));
  } else if (plan.gate_up != 0) RMLX_TRY(launch_qmv_wt(a, plan.gate_up, stream));
  else RMLX_TRY(gate->bits == 8 ? launch_qmv_q8_tab(a, stream) : launch_qmv_q4(a, stream));

  if (y == nullptr) return RMLX_OK;  // (the caller runs the down projection itself)
  QmvArgs d{};
  d.w0 = down->w; d.s0 = down->s; d.b0 = down->b;
  d.N = sh.D; d.K = sh.I;
  d.expert_stride_w = (size_t)sh.D * (sh.I / per);
  d.expert_stride_s = (size_t)sh.D * (sh.I / down->group_size);
  d.group_size = down->group_size;
  d.x = h; d.row_map = nullptr;
  d.out = y; d.ld_out = sh.D; d.out_f32 = y_f32; d.dual = 0;
  d.chunk_tab = chunk_tab; d.n_chunks_dev = n_chunks; d.max_chunks = max_chunks; d.mr = 8;
  if (plan.down != 0) return launch_qmv_wt(d, plan.down, stream);
  return gate->bits == 8 ? launch_qmv_q8_tab(d, stream) : launch_qmv_q4(d, stream);
}

}  // namespace
}  // namespace rmlx

using namespace rmlx;

extern "C" {

const char* rmlx_hip_last_error(void) { return last_error().c_str(); }

// ---- runtime shim ---------------------------------------------------------------------------

int32_t rmlx_hip_init(int32_t device) {
  int count = 0;
  RMLX_HIP_CHECK(hipGetDeviceCount(&count));
  if (device < 0 || device >= count)
    return fail(RMLX_RUNTIME_ERROR, "device %d not available (%d HIP devices visible)", device, count);
  RMLX_HIP_CHECK(hipSetDevice(device));
  hipDeviceProp_t prop;
  RMLX_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(RMLX_RUNTIME_ERROR, "device %d is %s; this library only contains gfx950 code", device, prop.gcnArchName);
  if (device < kMaxDevices && g_static_scratch[device] == nullptr) {
    void* p = nullptr;
    RMLX_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_static_scratch[device] = p;
  }
  ctx().device = device;
  ctx().num_cus = prop.multiProcessorCount;
  ctx().ready = true;
  return RMLX_OK;
}

int32_t rmlx_hip_device_info(int64_t out[8]) {
  RMLX_TRY(require_init());
  hipDeviceProp_t prop;
  RMLX_HIP_CHECK(hipGetDeviceProperties(&prop, ctx().device));
  out[0] = prop.multiProcessorCount;
  out[1] = prop.warpSize;
  out[2] = (int64_t)prop.sharedMemPerBlock;
  out[3] = (int64_t)(prop.totalGlobalMem >> 20);
  out[4] = prop.clockRate;
  out[5] = prop.memoryClockRate;
  out[6] = prop.memoryBusWidth;
  out[7] = prop.l2CacheSize;
  return RMLX_OK;
}

int32_t rmlx_hip_malloc(void** dev_ptr, size_t bytes) {
  RMLX_TRY(require_init());
  RMLX_HIP_CHECK(hipMalloc(dev_ptr, bytes == 0 ? 16 : bytes));
  return RMLX_OK;
}
int32_t rmlx_hip_free(void* dev_ptr) {
  RMLX_HIP_CHECK(hipFree(dev_ptr));
  return RMLX_OK;
}
int32_t rmlx_hip_memset(void* dev_ptr, int32_t value, size_t bytes, rmlx_stream stream) {
  RMLX_HIP_CHECK(hipMemsetAsync(dev_ptr, value, bytes, (hipStream_t)stream));
  return finish((hipStream_t)stream);
}
int32_t rmlx_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, rmlx_stream stream) {
  if (bytes == 0) return RMLX_OK;
  if (stream == nullptr) RMLX_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  else RMLX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  return RMLX_OK;
}
int32_t rmlx_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, rmlx_stream stream) {
  if (bytes == 0) return RMLX_OK;
  if (stream == nullptr) RMLX_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  else RMLX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
  return RMLX_OK;
}
int32_t rmlx_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, rmlx_stream stream) {
  if (bytes == 0) return RMLX_OK;
  RMLX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return finish((hipStream_t)stream);
}
int32_t rmlx_hip_stream_create(rmlx_stream* out) {
  RMLX_TRY(require_init());
  hipStream_t s;
  RMLX_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *out = s;
  return RMLX_OK;
}
int32_t rmlx_hip_stream_sync(rmlx_stream stream) {
  RMLX_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  return RMLX_OK;
}
int32_t rmlx_hip_stream_destroy(rmlx_stream stream) {
  // The stream's scratch blocks go back to the driver first: a later stream may get the same handle value and
  // must not inherit blocks whose last kernels were ordered on this one.
  // Every step runs whatever the one before it returned (nothing may leak); the first error is reported.
  const hipError_t sync_err = hipStreamSynchronize((hipStream_t)stream);
  const int32_t trim_status = trim_pool((hipStream_t)stream, true);
  const std::string trim_msg = last_error();
  const hipError_t destroy_err = hipStreamDestroy((hipStream_t)stream);
  if (sync_err != hipSuccess) return fail(RMLX_RUNTIME_ERROR, "hipStreamSynchronize failed: %s", hipGetErrorString(sync_err));
  if (trim_status != RMLX_OK) { last_error() = trim_msg; return trim_status; }
  if (destroy_err != hipSuccess) return fail(RMLX_RUNTIME_ERROR, "hipStreamDestroy failed: %s", hipGetErrorString(destroy_err));
  return RMLX_OK;
}
int32_t rmlx_hip_trim_pool(rmlx_stream stream) {
  RMLX_TRY(require_init());
  RMLX_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  return trim_pool((hipStream_t)stream, false);
}
int32_t rmlx_hip_graph_begin(rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (stream == nullptr) return fail(RMLX_INVALID_SHAPE, "graph_begin: recording needs a stream (the null stream is synchronous)");
  RMLX_HIP_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return RMLX_OK;
}
int32_t rmlx_hip_graph_end(rmlx_stream stream, rmlx_graph* out) {
  if (out == nullptr) return fail(RMLX_INVALID_SHAPE, "graph_end: out handle pointer is null");
  *out = nullptr;
  hipGraph_t g = nullptr;
  RMLX_HIP_CHECK(hipStreamEndCapture((hipStream_t)stream, &g));
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) return fail(RMLX_RUNTIME_ERROR, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  *out = exec;
  return RMLX_OK;
}
int32_t rmlx_hip_graph_launch(rmlx_graph graph, rmlx_stream stream) {
  if (graph == nullptr) return fail(RMLX_INVALID_SHAPE, "graph_launch: null graph");
  RMLX_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)stream));
  return RMLX_OK;
}
int32_t rmlx_hip_graph_destroy(rmlx_graph graph) {
  if (graph != nullptr) RMLX_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph));
  return RMLX_OK;
}
uint64_t rmlx_hip_scratch_allocations(void) {
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  return g_pool_allocations;
}
int32_t rmlx_hip_event_create(rmlx_event* out) {
  RMLX_TRY(require_init());
  hipEvent_t e;
  RMLX_HIP_CHECK(hipEventCreate(&e));
  *out = e;
  return RMLX_OK;
}
int32_t rmlx_hip_event_record(rmlx_event ev, rmlx_stream stream) {
  RMLX_HIP_CHECK(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
  return RMLX_OK;
}
int32_t rmlx_hip_event_sync(rmlx_event ev) {
  RMLX_HIP_CHECK(hipEventSynchronize((hipEvent_t)ev));
  return RMLX_OK;
}
int32_t rmlx_hip_event_elapsed_ms(rmlx_event start, rmlx_event stop, float* ms) {
  RMLX_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return RMLX_OK;
}
int32_t rmlx_hip_event_destroy(rmlx_event ev) {
  RMLX_HIP_CHECK(hipEventDestroy((hipEvent_t)ev));
  return RMLX_OK;
}

// ---- QuantizedWeight --------------------------------------------------------------------------

int32_t rmlx_hip_qweight_create(const void* weights_dev, size_t weights_bytes, const void* scales_dev,
                                size_t scales_bytes, const void* biases_dev, size_t biases_bytes,
                                uint32_t group_size, uint32_t bits, size_t out_features, size_t in_features,
                                size_t n_experts, rmlx_qweight** out) {
  if (out == nullptr) return fail(RMLX_INVALID_SHAPE, "qweight_create: out handle pointer is null");
  *out = nullptr;
  if (bits != 2 && bits != 3 && bits != 4 && bits != 6 && bits != 8)
    return fail(RMLX_INVALID_SHAPE, "unsupported bit width %u; must be one of [2, 3, 4, 6, 8]", bits);
  if (group_size != 32 && group_size != 64 && group_size != 128)
    return fail(RMLX_INVALID_SHAPE, "unsupported group_size %u; must be one of [32, 64, 128]", group_size);
  if (in_features % group_size != 0)
    return fail(RMLX_INVALID_SHAPE, "in_features (%zu) must be a multiple of group_size (%u)", in_features, group_size);
  if (n_experts == 0) return fail(RMLX_INVALID_SHAPE, "n_experts must be non-zero");
  const size_t total = n_experts * out_features * in_features;
  const size_t per = 32 / bits;
  const size_t expected_w = ((total + per - 1) / per) * 4;
  if (weights_bytes < expected_w)
    return fail(RMLX_INVALID_SHAPE, "weights_buf too small: %zu bytes < expected %zu bytes for [%zu, %zu] at %u bits",
                weights_bytes, expected_w, out_features, in_features, bits);
  const size_t groups = total / group_size;
  const size_t expected_s = groups * 2;
  if (scales_bytes < expected_s)
    return fail(RMLX_INVALID_SHAPE, "scales_buf too small: %zu bytes < expected %zu bytes (%zu groups)", scales_bytes,
                expected_s, groups);
  if (biases_bytes < expected_s)
    return fail(RMLX_INVALID_SHAPE, "biases_buf too small: %zu bytes < expected %zu bytes (%zu groups)", biases_bytes,
                expected_s, groups);
  if (total != 0 && (weights_dev == nullptr || scales_dev == nullptr || biases_dev == nullptr))
    return fail(RMLX_INVALID_SHAPE, "qweight_create: null device buffer");
  rmlx_qweight* q = new rmlx_qweight;
  q->w = static_cast<const uint32_t*>(weights_dev);
  q->s = static_cast<const __half*>(scales_dev);
  q->b = static_cast<const __half*>(biases_dev);
  q->group_size = group_size;
  q->bits = bits;
  q->out_features = out_features;
  q->in_features = in_features;
  q->n_experts = n_experts;
  *out = q;
  return RMLX_OK;
}

int32_t rmlx_hip_qweight_destroy(rmlx_qweight* qw) {
  delete qw;
  return RMLX_OK;
}

// ---- qmv / qmm ------------------------------------------------------------------------------------

int32_t rmlx_hip_affine_quantized_matmul(const rmlx_qweight* qw, const rmlx_array* vec, void* out_f16_dev,
                                         size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr || vec == nullptr) return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul: null argument");
  if (vec->dtype != RMLX_DTYPE_F32 && vec->dtype != RMLX_DTYPE_F16 && vec->dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul requires Float16 or Float32 input vec, got %s",
                dtype_name(vec->dtype));
  if (numel(vec) != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "vec.numel() (%zu) != in_features (%zu)", numel(vec), qw->in_features);
  if (qw->n_experts != 1) return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul: weight is a stacked expert weight");
  RMLX_TRY(check_out("affine_quantized_matmul", out_bytes, qw->out_features * 2));
  RMLX_TRY(run_matmul(qw, vec->data, vec->dtype, 1, static_cast<__half*>(out_f16_dev), KERNEL_AUTO, (hipStream_t)stream));
  return finish((hipStream_t)stream);
}

int32_t rmlx_hip_qmm_select(const rmlx_qweight* qw, const rmlx_array* x, int32_t kernel, void* out_f16_dev,
                            size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr || x == nullptr) return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched: null argument");
  RMLX_TRY(check_x_dtype("affine_quantized_matmul_batched", x->dtype));
  if (x->ndim != 2)
    return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched requires 2D input x, got %dD", x->ndim);
  if (x->shape[1] != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "x.shape[1] (%zu) != in_features (%zu)", x->shape[1], qw->in_features);
  if (qw->bits != 4 && qw->bits != 8 && kernel != KERNEL_GENERIC)
    return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched requires bits==4 or bits==8, got %u", qw->bits);
  if (qw->n_experts != 1) return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched: weight is a stacked expert weight");
  uint32_t M;
  RMLX_TRY(checked_u32(x->shape[0], "M", &M));
  RMLX_TRY(check_out("affine_quantized_matmul_batched", out_bytes, (size_t)M * qw->out_features * 2));
  RMLX_TRY(run_matmul(qw, x->data, x->dtype, M, static_cast<__half*>(out_f16_dev), kernel, (hipStream_t)stream));
  return finish((hipStream_t)stream);
}

int32_t rmlx_hip_affine_quantized_matmul_batched(const rmlx_qweight* qw, const rmlx_array* x, void* out_f16_dev,
                                                 size_t out_bytes, rmlx_stream stream) {
  return rmlx_hip_qmm_select(qw, x, KERNEL_AUTO, out_f16_dev, out_bytes, stream);
}

namespace {
int32_t qmm_with_epilogue(const char* what, const char* operand, int kind, const rmlx_qweight* qw, const rmlx_array* x,
                          const rmlx_array* e, void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr || x == nullptr || e == nullptr) return fail(RMLX_INVALID_SHAPE, "%s: null argument", what);
  RMLX_TRY(check_x_dtype(what, x->dtype));
  if (x->ndim != 2) return fail(RMLX_INVALID_SHAPE, "%s requires 2D input x, got %dD", what, x->ndim);
  if (x->shape[1] != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "x.shape[1] (%zu) != in_features (%zu)", x->shape[1], qw->in_features);
  if (qw->bits != 4 && qw->bits != 8) return fail(RMLX_INVALID_SHAPE, "%s requires bits==4 or bits==8, got %u", what, qw->bits);
  if (qw->n_experts != 1) return fail(RMLX_INVALID_SHAPE, "%s: weight is a stacked expert weight", what);
  if (e->ndim != 2 || e->shape[0] != x->shape[0] || e->shape[1] != qw->out_features)
    return fail(RMLX_INVALID_SHAPE, "%s: %s shape must be [%zu, %zu]", what, operand, x->shape[0], qw->out_features);
  if (e->dtype != RMLX_DTYPE_F16 && e->dtype != RMLX_DTYPE_F32)
    return fail(RMLX_INVALID_SHAPE, "%s: %s must be Float16 or Float32, got %s", what, operand, dtype_name(e->dtype));
  uint32_t M;
  RMLX_TRY(checked_u32(x->shape[0], "M", &M));
  RMLX_TRY(check_out(what, out_bytes, (size_t)M * qw->out_features * 2));
  Epilogue epi;
  epi.kind = kind; epi.ptr = e->data; epi.dtype = e->dtype;
  RMLX_TRY(run_matmul(qw, x->data, x->dtype, M, static_cast<__half*>(out_f16_dev), KERNEL_AUTO, (hipStream_t)stream, epi));
  return finish((hipStream_t)stream);
}
}  // namespace

int32_t rmlx_hip_qmm_norm(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* norm_weight,
                          const rmlx_array* inv_rms, void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr || x == nullptr || norm_weight == nullptr || inv_rms == nullptr)
    return fail(RMLX_INVALID_SHAPE, "qmm_norm: null argument");
  RMLX_TRY(check_x_dtype("qmm_norm", x->dtype));
  if (x->ndim != 2) return fail(RMLX_INVALID_SHAPE, "qmm_norm requires 2D input x, got %dD", x->ndim);
  if (x->shape[1] != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "x.shape[1] (%zu) != in_features (%zu)", x->shape[1], qw->in_features);
  if (qw->bits != 4 && qw->bits != 8) return fail(RMLX_INVALID_SHAPE, "qmm_norm requires bits==4 or bits==8, got %u", qw->bits);
  if (qw->n_experts != 1) return fail(RMLX_INVALID_SHAPE, "qmm_norm: weight is a stacked expert weight");
  if (norm_weight->dtype != RMLX_DTYPE_F16 || numel(norm_weight) != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "qmm_norm: norm_weight must be Float16 [%zu], got %s with %zu elements", qw->in_features,
                dtype_name(norm_weight->dtype), numel(norm_weight));
  if (inv_rms->dtype != RMLX_DTYPE_F32 || numel(inv_rms) != x->shape[0])
    return fail(RMLX_INVALID_SHAPE, "qmm_norm: inv_rms must be Float32 [%zu], got %s with %zu elements", x->shape[0],
                dtype_name(inv_rms->dtype), numel(inv_rms));
  if (!aligned16(norm_weight->data)) return fail(RMLX_INVALID_SHAPE, "qmm_norm: norm_weight must be 16-byte aligned");
  uint32_t M;
  RMLX_TRY(checked_u32(x->shape[0], "M", &M));
  RMLX_TRY(check_out("qmm_norm", out_bytes, (size_t)M * qw->out_features * 2));
  Epilogue fuse;
  fuse.norm_w = static_cast<const __half*>(norm_weight->data);
  fuse.inv_rms = static_cast<const float*>(inv_rms->data);
  RMLX_TRY(run_matmul(qw, x->data, x->dtype, M, static_cast<__half*>(out_f16_dev), KERNEL_AUTO, (hipStream_t)stream, fuse));
  return finish((hipStream_t)stream);
}

int32_t rmlx_hip_qmm_add_residual(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* residual,
                                  void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  return qmm_with_epilogue("qmm_add_residual_into_cb", "residual", EPI_RESIDUAL, qw, x, residual, out_f16_dev, out_bytes, stream);
}

int32_t rmlx_hip_qmm_swiglu(const rmlx_qweight* qw, const rmlx_array* x, const rmlx_array* gate_result,
                            void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  return qmm_with_epilogue("qmm_swiglu_into_cb", "gate_result", EPI_SWIGLU, qw, x, gate_result, out_f16_dev, out_bytes, stream);
}

int32_t rmlx_hip_qmm_encode_many(const rmlx_qweight* const* qws, size_t n_qw, const rmlx_array* x,
                                 void* const* outs_f16_dev, size_t n_out, size_t out_bytes, size_t count,
                                 int32_t kernel, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qws == nullptr || outs_f16_dev == nullptr || x == nullptr || n_qw == 0 || n_out == 0)
    return fail(RMLX_INVALID_SHAPE, "qmm_encode_many: null or empty argument");
  RMLX_TRY(check_x_dtype("affine_quantized_matmul_batched", x->dtype));
  if (x->ndim != 2) return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched requires 2D input x, got %dD", x->ndim);
  for (size_t i = 0; i < n_qw; ++i) {
    if (qws[i] == nullptr || qws[i]->n_experts != 1 || qws[i]->in_features != qws[0]->in_features ||
        qws[i]->out_features != qws[0]->out_features)
      return fail(RMLX_INVALID_SHAPE, "qmm_encode_many: weight %zu does not match weight 0", i);
    // (a single row is the qmv entry point, which takes every bit width: quantized.rs:1309-1411)
    if (qws[i]->bits != 4 && qws[i]->bits != 8 && !(x->shape[0] == 1))
      return fail(RMLX_INVALID_SHAPE, "affine_quantized_matmul_batched requires bits==4 or bits==8, got %u", qws[i]->bits);
  }
  if (x->shape[1] != qws[0]->in_features)
    return fail(RMLX_INVALID_SHAPE, "x.shape[1] (%zu) != in_features (%zu)", x->shape[1], qws[0]->in_features);
  uint32_t M;
  RMLX_TRY(checked_u32(x->shape[0], "M", &M));
  RMLX_TRY(check_out("qmm_encode_many", out_bytes, (size_t)M * qws[0]->out_features * 2));
  hipStream_t s = (hipStream_t)stream;
  for (size_t i = 0; i < count; ++i)
    RMLX_TRY(run_matmul(qws[i % n_qw], x->data, x->dtype, M, static_cast<__half*>(outs_f16_dev[i % n_out]), kernel, s));
  return finish(s);
}

int32_t rmlx_hip_quantized_linear_forward(const rmlx_qweight* qw, const rmlx_array* x, const void* bias_f16_dev,
                                          void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr || x == nullptr) return fail(RMLX_INVALID_SHAPE, "QuantizedLinear: null argument");
  size_t batch, feat;
  if (x->ndim == 1) { batch = 1; feat = x->shape[0]; }
  else if (x->ndim == 2) { batch = x->shape[0]; feat = x->shape[1]; }
  else return fail(RMLX_INVALID_SHAPE, "QuantizedLinear: input must be 1D or 2D, got %dD", x->ndim);
  if (dtype_size(x->dtype) == 0 || x->dtype == RMLX_DTYPE_U32 || x->dtype == RMLX_DTYPE_U8)
    return fail(RMLX_INVALID_SHAPE, "QuantizedLinear: unsupported input dtype %s", dtype_name(x->dtype));
  if (feat != qw->in_features)
    return fail(RMLX_INVALID_SHAPE, "QuantizedLinear: input features mismatch: %zu vs %zu", feat, qw->in_features);
  if (qw->bits != 4 && qw->bits != 8)
    return fail(RMLX_INVALID_SHAPE, "QuantizedLinear: bits must be 4 or 8, got %u", qw->bits);
  uint32_t M, N;
  RMLX_TRY(checked_u32(batch, "batch", &M));
  RMLX_TRY(checked_u32(qw->out_features, "out_features", &N));
  RMLX_TRY(check_out("QuantizedLinear", out_bytes, (size_t)M * N * 2));
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(run_matmul(qw, x->data, x->dtype, M, static_cast<__half*>(out_f16_dev), KERNEL_AUTO, s));
  if (bias_f16_dev != nullptr)
    RMLX_TRY(launch_add_bias_rows(static_cast<__half*>(out_f16_dev), static_cast<const __half*>(bias_f16_dev), M, N, s));
  return finish(s);
}

// ---- gather_qmm -----------------------------------------------------------------------------------

int32_t rmlx_hip_gather_qmm_select(const rmlx_array* x, const void* w_packed_dev, size_t w_bytes, const void* scales_dev,
                                   size_t scales_bytes, const void* biases_dev, size_t biases_bytes,
                                   const rmlx_array* indices, size_t batch, size_t m_per_batch, size_t n, size_t k,
                                   size_t n_experts, uint32_t group_size, int32_t kernel, void* out_f16_dev,
                                   size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (kernel < GATHER_AUTO || kernel > GATHER_PORTABLE) return fail(RMLX_NOT_FOUND, "gather_qmm: unknown kernel selector %d", kernel);
  if (x == nullptr || indices == nullptr) return fail(RMLX_INVALID_SHAPE, "gather_qmm: null argument");
  if (x->dtype != RMLX_DTYPE_F32 && x->dtype != RMLX_DTYPE_F16)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm requires Float32 or Float16 input x, got %s", dtype_name(x->dtype));
  if (indices->dtype != RMLX_DTYPE_U32)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: indices must be UInt32, got %s", dtype_name(indices->dtype));
  if (k == 0 || n == 0 || m_per_batch == 0)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: dimensions must be non-zero (k=%zu, n=%zu, m_per_batch=%zu)", k, n, m_per_batch);
  if (n_experts == 0) return fail(RMLX_INVALID_SHAPE, "gather_qmm: n_experts must be non-zero");
  const size_t expected_x = batch * m_per_batch * k;
  if (numel(x) != expected_x)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: x has %zu elements but expected batch(%zu) * m_per_batch(%zu) * k(%zu) = %zu",
                numel(x), batch, m_per_batch, k, expected_x);
  if (numel(indices) != batch)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: indices length %zu != batch %zu", numel(indices), batch);
  if (group_size == 0) return fail(RMLX_INVALID_SHAPE, "gather_qmm: group_size must be non-zero");
  if (k % 2 != 0) return fail(RMLX_INVALID_SHAPE, "gather_qmm: K (%zu) must be even for Q4 packing", k);
  if (k % group_size != 0)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: K (%zu) must be a multiple of group_size (%u)", k, group_size);
  if (k % 8 != 0) return fail(RMLX_INVALID_SHAPE, "gather_qmm: K (%zu) must be a multiple of pack_factor (8)", k);
  const size_t half_k = k / 2, gpr = k / group_size;
  const size_t expected_w = n_experts * n * half_k;
  if (w_bytes < expected_w)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: w_packed_buf too small: %zu bytes < expected %zu bytes (n_experts=%zu, N=%zu, K/2=%zu)",
                w_bytes, expected_w, n_experts, n, half_k);
  const size_t expected_s = n_experts * n * gpr * 2;
  if (scales_bytes < expected_s)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: scales_buf too small: %zu bytes < expected %zu bytes (n_experts=%zu, N=%zu, groups_per_row=%zu)",
                scales_bytes, expected_s, n_experts, n, gpr);
  if (biases_bytes < expected_s)
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: biases_buf too small: %zu bytes < expected %zu bytes (n_experts=%zu, N=%zu, groups_per_row=%zu)",
                biases_bytes, expected_s, n_experts, n, gpr);
  uint32_t B32, M32, N32, K32, E32;
  RMLX_TRY(checked_u32(batch, "batch", &B32));
  RMLX_TRY(checked_u32(m_per_batch, "M_per_batch", &M32));
  RMLX_TRY(checked_u32(n, "N", &N32));
  RMLX_TRY(checked_u32(k, "K", &K32));
  RMLX_TRY(checked_u32(n_experts, "n_experts", &E32));
  RMLX_TRY(checked_u32(batch * m_per_batch, "batch * M_per_batch", &M32));
  RMLX_TRY(check_out("gather_qmm", out_bytes, batch * m_per_batch * n * 2));
  if (batch == 0) return RMLX_OK;  // empty result

  hipStream_t s = (hipStream_t)stream;
  const uint32_t* idx = static_cast<const uint32_t*>(indices->data);
  if (stream == nullptr) {  // the reference validates every index on the host (quantized.rs:9514-9524)
    std::vector<uint32_t> host(batch);
    RMLX_HIP_CHECK(hipMemcpy(host.data(), idx, batch * 4, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < batch; ++i)
      if (host[i] >= n_experts)
        return fail(RMLX_INVALID_SHAPE, "gather_qmm: index[%zu]=%u out of range [0, %zu)", i, host[i], n_experts);
  }

  const uint32_t rows = B32 * (uint32_t)m_per_batch;
  Scratch cast;
  const __half* xk = static_cast<const __half*>(x->data);
  if (x->dtype != RMLX_DTYPE_F16) {
    RMLX_TRY(cast.alloc((size_t)rows * k * 2, s));
    RMLX_TRY(launch_cast_to_f16(x->data, x->dtype, static_cast<__half*>(cast.ptr), (size_t)rows * k, s));
    xk = static_cast<const __half*>(cast.ptr);
  }
  const uint32_t* w = static_cast<const uint32_t*>(w_packed_dev);
  const __half* sc = static_cast<const __half*>(scales_dev);
  const __half* bi = static_cast<const __half*>(biases_dev);
  // group size 32 streams on the wave-per-tile kernel (chunks of 8 rows as well)
  const bool wt32 = group_size == 32 && qmv_wt_supported(N32, K32, 32, 8);
  const bool fast = (qmv_q4_supported(N32, K32, group_size) || wt32) && aligned16(w) && aligned16(sc) &&
                    aligned16(bi) && aligned16(xk);
  // (measured, 32 entries over 3072 x 4096 weights: 8 rows 50 us streamed; 12 / 16 / 32 rows 61 / 64 / 76 us on the GEMM
  // with 16- / 32-row tiles against 95 / 99 / 172 us streamed)
  const bool can_gemm = aligned16(w) && aligned16(sc) && aligned16(bi) && aligned16(xk) &&
                        qmm_rw_grouped_supported(N32, K32, group_size, 4);
  if ((kernel == GATHER_GEMM && !can_gemm) || (kernel == GATHER_STREAM && !fast))
    return fail(RMLX_INVALID_SHAPE, "gather_qmm: the selected kernel does not take N=%u K=%u group_size=%u (or a buffer is not 16-byte aligned)",
                N32, K32, group_size);
  if (kernel == GATHER_GEMM || (kernel == GATHER_AUTO && can_gemm && m_per_batch >= kGatherGemmMinRows)) {
    // many rows per entry: row tiles of one expert each on the grouped MFMA GEMM
    const uint32_t tile_rows = m_per_batch <= 16 && group_size == 64 ? 16u : (m_per_batch <= 32 ? 32u : kGroupedTileRows);
    const uint32_t per = ((uint32_t)m_per_batch + tile_rows - 1) / tile_rows;
    const uint64_t n_tiles = (uint64_t)B32 * per;
    if (n_tiles > 0x7FFFFFu) return fail(RMLX_INVALID_SHAPE, "gather_qmm: too many row tiles (%" PRIu64 ")", n_tiles);
    Scratch tab;
    RMLX_TRY(tab.alloc((size_t)n_tiles * 12 + 4, s));
    uint32_t* t = static_cast<uint32_t*>(tab.ptr);
    RMLX_TRY(launch_build_gather_chunks(idx, B32, (uint32_t)m_per_batch, E32, tile_rows, t, t + 3 * n_tiles, s));
    GroupedQmmArgs a{};
    a.w = w; a.s = sc; a.b = bi;
    a.N = N32; a.K = K32; a.bits = 4; a.group_size = group_size;
    a.expert_stride_w = (uint64_t)n * (k / 8);
    a.expert_stride_s = (uint64_t)n * gpr;
    a.x = xk; a.out = out_f16_dev;
    a.tile_tab = t; a.n_tiles_dev = t + 3 * n_tiles; a.max_tiles = (uint32_t)n_tiles; a.tile_rows = tile_rows;
    RMLX_TRY(launch_qmm_rw_grouped(a, s));
  } else if (kernel == GATHER_AUTO && !can_gemm && !fast && m_per_batch >= kGatherGemmMinRows && (uint64_t)rows >= 96 &&
             qmm_supported(N32, K32, group_size, 4) && aligned16(w) && aligned16(sc) && aligned16(bi) && aligned16(xk) &&
             (uint64_t)B32 * (((uint32_t)m_per_batch + 63) / 64) <= 65535) {
    // many rows per entry over dimensions in multiples of 64 that the register-weights grouped GEMM does not take: row tiles
    // of 64 rows of one entry (128 from 65 rows per entry on) on the grouped form of the LDS-staged GEMM
    const uint32_t lds_rows = m_per_batch > 64 ? 128u : 64u;
    const uint32_t per = ((uint32_t)m_per_batch + lds_rows - 1) / lds_rows, n_tiles = B32 * per;
    Scratch tab, ws;
    RMLX_TRY(tab.alloc((size_t)n_tiles * 12 + 4, s));
    uint32_t* t = static_cast<uint32_t*>(tab.ptr);
    RMLX_TRY(launch_build_gather_chunks(idx, B32, (uint32_t)m_per_batch, E32, lds_rows, t, t + 3 * (size_t)n_tiles, s));
    RMLX_TRY(ws.alloc(qmm_grouped_workspace_bytes(n_tiles, K32, lds_rows), s));
    GroupedQmmArgs a{};
    a.w = w; a.s = sc; a.b = bi;
    a.N = N32; a.K = K32; a.bits = 4; a.group_size = group_size;
    a.expert_stride_w = (uint64_t)n * (k / 8);
    a.expert_stride_s = (uint64_t)n * gpr;
    a.x = xk; a.out = out_f16_dev;
    a.tile_tab = t; a.n_tiles_dev = t + 3 * (size_t)n_tiles; a.max_tiles = n_tiles; a.tile_rows = lds_rows;
    RMLX_TRY(launch_qmm_grouped(a, ws.ptr, s));
  } else if (m_per_batch == 1 && kernel == GATHER_AUTO && qmv_m1_supported(N32, K32, group_size, 4) && aligned16(w) &&
             aligned16(sc) && aligned16(bi) && aligned16(xk)) {
    // one row per index: the single-row kernel with a weight matrix per activation row -- one launch, no chunk table
    RMLX_TRY(launch_qmv_m1_gather(w, sc, bi, (uint64_t)n * (k / 8), (uint64_t)n * gpr, E32, xk, idx, B32,
                                  static_cast<__half*>(out_f16_dev), N32, K32, group_size, 4, s));
  } else if (!fast && kernel == GATHER_AUTO && rows <= kUngroupedOnlyMaxAssignments && qmv_m1_supported(N32, K32, group_size, 4) &&
             aligned16(w) && aligned16(sc) && aligned16(bi) && aligned16(xk)) {
    // several rows per index over a shape no streaming or grouped kernel takes (rows off the multiples of 128): every row on
    // the single-row kernel with its entry's weight matrix, instead of the portable kernel
    RMLX_TRY(launch_qmv_m1_gather(w, sc, bi, (uint64_t)n * (k / 8), (uint64_t)n * gpr, E32, xk, idx, rows,
                                  static_cast<__half*>(out_f16_dev), N32, K32, group_size, 4, s, (uint32_t)m_per_batch));
  } else if (fast && kernel != GATHER_PORTABLE) {
    const uint64_t per = ((uint64_t)m_per_batch + 7) / 8, n_chunks = (uint64_t)B32 * per;
    if (n_chunks > 0x7FFFFFFFull) return fail(RMLX_INVALID_SHAPE, "gather_qmm: too many row chunks (%" PRIu64 ")", n_chunks);
    Scratch tab;
    RMLX_TRY(tab.alloc((size_t)n_chunks * 12, s));
    RMLX_TRY(launch_build_gather_chunks(idx, B32, (uint32_t)m_per_batch, E32, 8, static_cast<uint32_t*>(tab.ptr), nullptr, s));
    QmvArgs a{};
    a.w0 = w; a.s0 = sc; a.b0 = bi;
    a.N = N32; a.K = K32;
    a.expert_stride_w = (uint64_t)n * (k / 8);
    a.expert_stride_s = (uint64_t)n * gpr;
    a.x = xk; a.out = out_f16_dev; a.ld_out = N32;
    a.mr = m_per_batch >= 5 ? 8 : (m_per_batch >= 3 ? 4 : (m_per_batch == 2 ? 2 : 1));
    a.group_size = group_size;
    // a launch takes at most 65535 chunks (the chunk index is the second grid dimension); the table's entries
    // name absolute rows, so a longer table is simply walked in pieces
    for (uint64_t first = 0; first < n_chunks; first += 65535) {
      a.chunk_tab = static_cast<const uint32_t*>(tab.ptr) + 3 * first;
      a.max_chunks = (uint32_t)(n_chunks - first < 65535 ? n_chunks - first : 65535);
      RMLX_TRY(wt32 ? launch_qmv_wt(a, 8, s) : launch_qmv_q4(a, s));
    }
  } else {
    GenericArgs g{w, sc, bi, xk, static_cast<__half*>(out_f16_dev), idx, (uint32_t)m_per_batch, rows, N32, K32,
                  group_size, 4, E32};
    RMLX_TRY(launch_generic(g, s));
  }
  return finish(s);
}

int32_t rmlx_hip_gather_qmm(const rmlx_array* x, const void* w_packed_dev, size_t w_bytes, const void* scales_dev,
                            size_t scales_bytes, const void* biases_dev, size_t biases_bytes,
                            const rmlx_array* indices, size_t batch, size_t m_per_batch, size_t n, size_t k,
                            size_t n_experts, uint32_t group_size, void* out_f16_dev, size_t out_bytes,
                            rmlx_stream stream) {
  return rmlx_hip_gather_qmm_select(x, w_packed_dev, w_bytes, scales_dev, scales_bytes, biases_dev, biases_bytes, indices,
                                    batch, m_per_batch, n, k, n_experts, group_size, GATHER_AUTO, out_f16_dev, out_bytes, stream);
}

// ---- routing / grouping / data movement ----------------------------------------------------------------

}  // extern "C"

namespace {
int32_t topk_route_impl(const rmlx_array* gate_logits, size_t top_k, const rmlx_array* expert_bias,
                        int32_t renormalize, uint32_t* expert_indices_dev, float* expert_weights_dev,
                        uint32_t* expert_counts_dev, uint32_t* dispatch_offsets_dev, rmlx_stream stream, Arena* arena) {
  RMLX_TRY(require_init());
  if (gate_logits == nullptr) return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: null gate_logits");
  if (gate_logits->ndim != 2)
    return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: gate_logits must be 2D [N, E], got %dD", gate_logits->ndim);
  if (gate_logits->dtype != RMLX_DTYPE_F32 && gate_logits->dtype != RMLX_DTYPE_F16)
    return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: gate_logits must be Float16 or Float32, got %s",
                dtype_name(gate_logits->dtype));
  if (top_k == 0 || top_k > 8) return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: top_k must be in [1, 8], got %zu", top_k);
  const size_t T = gate_logits->shape[0], E = gate_logits->shape[1];
  if (top_k > E) return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: top_k (%zu) > num_experts (%zu)", top_k, E);
  if (E > 256) return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: num_experts (%zu) exceeds maximum 256", E);
  if (expert_bias != nullptr) {
    if (expert_bias->ndim != 1)
      return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: expert_bias must be 1D [E], got %dD", expert_bias->ndim);
    if (expert_bias->shape[0] != E)
      return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: expert_bias length %zu != num_experts %zu", expert_bias->shape[0], E);
    if (expert_bias->dtype != RMLX_DTYPE_F32 && expert_bias->dtype != RMLX_DTYPE_F16)
      return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: expert_bias must be Float16 or Float32, got %s",
                  dtype_name(expert_bias->dtype));
  }
  uint32_t T32, A32;
  RMLX_TRY(checked_u32(T, "seq_len", &T32));
  RMLX_TRY(checked_u32(T * top_k, "seq_len * top_k", &A32));
  hipStream_t s = (hipStream_t)stream;
  // f16 inputs are widened to f32 first, as the reference does (topk_route.rs:474-483).
  Scratch lg32, bias32;
  const float* lg = static_cast<const float*>(gate_logits->data);
  if (gate_logits->dtype == RMLX_DTYPE_F16) {
    RMLX_TRY(lg32.alloc(T * E * 4, s, arena));
    RMLX_TRY(launch_cast_f16_to_f32(static_cast<const __half*>(gate_logits->data), static_cast<float*>(lg32.ptr), T * E, s));
    lg = static_cast<const float*>(lg32.ptr);
  }
  const float* bias = nullptr;
  if (expert_bias != nullptr) {
    bias = static_cast<const float*>(expert_bias->data);
    if (expert_bias->dtype == RMLX_DTYPE_F16) {
      RMLX_TRY(bias32.alloc(E * 4, s, arena));
      RMLX_TRY(launch_cast_f16_to_f32(static_cast<const __half*>(expert_bias->data), static_cast<float*>(bias32.ptr), E, s));
      bias = static_cast<const float*>(bias32.ptr);
    }
  }
  RMLX_TRY(launch_topk_route(lg, bias, T32, (uint32_t)E, (uint32_t)top_k, renormalize, expert_indices_dev,
                             expert_weights_dev, expert_counts_dev, dispatch_offsets_dev, s));
  return finish(s);
}
}  // namespace

extern "C" {

int32_t rmlx_hip_topk_route(const rmlx_array* gate_logits, size_t top_k, const rmlx_array* expert_bias,
                            int32_t renormalize, uint32_t* expert_indices_dev, float* expert_weights_dev,
                            uint32_t* expert_counts_dev, uint32_t* dispatch_offsets_dev, rmlx_stream stream) {
  return topk_route_impl(gate_logits, top_k, expert_bias, renormalize, expert_indices_dev, expert_weights_dev,
                         expert_counts_dev, dispatch_offsets_dev, stream, nullptr);
}

int32_t rmlx_hip_moe_sort(const uint32_t* expert_indices_dev, size_t n_assign, size_t n_experts,
                          uint32_t* sorted_assign_dev, uint32_t* offsets_dev, rmlx_stream stream) {
  RMLX_TRY(require_init());
  uint32_t A, E;
  RMLX_TRY(checked_u32(n_assign, "n_assign", &A));
  RMLX_TRY(checked_u32(n_experts, "n_experts", &E));
  if (E == 0) return fail(RMLX_INVALID_SHAPE, "moe_sort: n_experts must be non-zero");
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_moe_sort(expert_indices_dev, A, E, 1, sorted_assign_dev, nullptr, nullptr, nullptr, offsets_dev, nullptr, nullptr, 8, s));
  return finish(s);
}

int32_t rmlx_hip_index_gather(const void* src_f16_dev, size_t src_rows, size_t d, const uint32_t* idx_dev, size_t n,
                              void* dst_f16_dev, rmlx_stream stream) {
  RMLX_TRY(require_init());
  uint32_t R, D, N;
  RMLX_TRY(checked_u32(src_rows, "src_rows", &R));
  RMLX_TRY(checked_u32(d, "d", &D));
  RMLX_TRY(checked_u32(n, "n", &N));
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_index_gather(static_cast<const __half*>(src_f16_dev), D, idx_dev, N, R, static_cast<__half*>(dst_f16_dev), s));
  return finish(s);
}

int32_t rmlx_hip_scatter_weighted_add(const void* src_f16_dev, size_t n, size_t d, const uint32_t* tok_dev,
                                      const float* w_dev, void* dst_f16_dev, size_t dst_rows, rmlx_stream stream) {
  RMLX_TRY(require_init());
  uint32_t N, D, R;
  RMLX_TRY(checked_u32(n, "n", &N));
  RMLX_TRY(checked_u32(d, "d", &D));
  RMLX_TRY(checked_u32(dst_rows, "dst_rows", &R));
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_scatter_weighted_add(static_cast<const __half*>(src_f16_dev), N, D, tok_dev, w_dev,
                                       static_cast<__half*>(dst_f16_dev), R, s));
  return finish(s);
}

int32_t rmlx_hip_silu_gate(const void* gate_in_f16_dev, const void* up_in_f16_dev, void* out_f16_dev, size_t numel_,
                           rmlx_stream stream) {
  RMLX_TRY(require_init());
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_silu_gate(static_cast<const __half*>(gate_in_f16_dev), static_cast<const __half*>(up_in_f16_dev),
                            static_cast<__half*>(out_f16_dev), numel_, s));
  return finish(s);
}

// ---- expert FFN -------------------------------------------------------------------------------------

int32_t rmlx_hip_expert_group_grouped_forward(const rmlx_qweight* gate, const rmlx_qweight* up,
                                              const rmlx_qweight* down, size_t n_items,
                                              const uint32_t* expert_idx_host, const uint32_t* batch_sizes_host,
                                              const rmlx_array* x, void* out_f16_dev, size_t out_bytes,
                                              rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (n_items == 0) return RMLX_OK;  // empty in -> empty out (expert_group.rs:314-316)
  ExpertShapes sh;
  RMLX_TRY(check_expert_weights("ExpertGroup", gate, up, down, &sh));
  if (x == nullptr || expert_idx_host == nullptr || batch_sizes_host == nullptr)
    return fail(RMLX_INVALID_SHAPE, "ExpertGroup: null argument");
  size_t total = 0;
  for (size_t i = 0; i < n_items; ++i) total += batch_sizes_host[i];
  // row chunks of one expert each: 8 rows for the streaming GEMV, whole row tiles for the grouped GEMM
  const uint32_t gemm = expert_gemm_tile_rows(sh, total, n_items);
  const StreamPlan plan = expert_stream_plan(sh, total, n_items);
  const uint32_t chunk_rows = gemm ? gemm : plan.chunk_rows;
  std::vector<uint32_t> tab;
  total = 0;
  for (size_t i = 0; i < n_items; ++i) {
    if (expert_idx_host[i] >= sh.E)
      return fail(RMLX_INVALID_SHAPE, "ExpertGroup: expert_idx %u >= num_experts %u", expert_idx_host[i], sh.E);
    for (uint32_t r = 0; r < batch_sizes_host[i]; r += chunk_rows) {
      tab.push_back(expert_idx_host[i]);
      tab.push_back((uint32_t)(total + r));
      tab.push_back(batch_sizes_host[i] - r < chunk_rows ? batch_sizes_host[i] - r : chunk_rows);
    }
    total += batch_sizes_host[i];
  }
  if (x->ndim != 2) return fail(RMLX_INVALID_SHAPE, "ExpertGroup: input must be 2D [batch, D], got %dD", x->ndim);
  if (x->shape[1] != sh.D) return fail(RMLX_INVALID_SHAPE, "ExpertGroup: input dim %zu != hidden_dim %u", x->shape[1], sh.D);
  if (x->shape[0] != total)
    return fail(RMLX_INVALID_SHAPE, "ExpertGroup: packed input has %zu rows but the batch sizes sum to %zu", x->shape[0], total);
  if (x->dtype != RMLX_DTYPE_F16 && x->dtype != RMLX_DTYPE_F32 && x->dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_INVALID_SHAPE, "ExpertGroup: unsupported dtype %s for SiLU", dtype_name(x->dtype));
  uint32_t rows;
  RMLX_TRY(checked_u32(total, "total_tokens", &rows));
  RMLX_TRY(check_out("ExpertGroup", out_bytes, total * sh.D * 2));
  if (total == 0) return RMLX_OK;
  const uint32_t n_chunks = (uint32_t)(tab.size() / 3);
  if (n_chunks > 65535) return fail(RMLX_INVALID_SHAPE, "ExpertGroup: too many row chunks (%u)", n_chunks);
  tab.push_back(n_chunks);  // the table's length travels behind it

  hipStream_t s = (hipStream_t)stream;
  Scratch cast, dtab, h;
  const __half* xk = static_cast<const __half*>(x->data);
  if (x->dtype != RMLX_DTYPE_F16) {
    RMLX_TRY(cast.alloc(total * sh.D * 2, s));
    RMLX_TRY(launch_cast_to_f16(x->data, x->dtype, static_cast<__half*>(cast.ptr), total * sh.D, s));
    xk = static_cast<const __half*>(cast.ptr);
  }
  if (sh.portable && !gemm) {  // expert of every packed row, then the portable kernels
    std::vector<uint32_t> expert_of;
    expert_of.reserve(total);
    for (size_t i = 0; i < n_items; ++i) expert_of.insert(expert_of.end(), batch_sizes_host[i], expert_idx_host[i]);
    RMLX_TRY(dtab.alloc(total * 4, s));
    RMLX_HIP_CHECK(hipMemcpyAsync(dtab.ptr, expert_of.data(), total * 4, hipMemcpyHostToDevice, s));
    RMLX_HIP_CHECK(hipStreamSynchronize(s));  // `expert_of` is pageable host memory owned by this call
    const uint32_t* experts = static_cast<const uint32_t*>(dtab.ptr);
    // dimensions in multiples of 64: row tiles of 64 (or 128) rows of one item on the grouped form of the LDS-staged GEMM, from
    // three rows per item on (see moe_grouped_impl)
    if (sh.gemm_lds && sh.gemm_min_rows != 0 && total >= 3 * n_items && aligned16(xk)) {
      std::vector<uint32_t> tiles;
      size_t first = 0;
      const uint32_t tile_rows = total >= 64 * n_items ? 128u : 64u;  // (as in moe_grouped_impl)
      for (size_t i = 0; i < n_items; ++i) {
        for (uint32_t r = 0; r < batch_sizes_host[i]; r += tile_rows) {
          tiles.push_back(expert_idx_host[i]);
          tiles.push_back((uint32_t)(first + r));
          tiles.push_back(batch_sizes_host[i] - r < tile_rows ? batch_sizes_host[i] - r : tile_rows);
        }
        first += batch_sizes_host[i];
      }
      const uint32_t n_t = (uint32_t)(tiles.size() / 3);
      if (n_t <= 65535) {
        tiles.push_back(n_t);
        Scratch ttab;
        RMLX_TRY(ttab.alloc(tiles.size() * 4, s));
        RMLX_HIP_CHECK(hipMemcpyAsync(ttab.ptr, tiles.data(), tiles.size() * 4, hipMemcpyHostToDevice, s));
        RMLX_HIP_CHECK(hipStreamSynchronize(s));  // `tiles` is pageable host memory owned by this call
        const uint32_t* tt = static_cast<const uint32_t*>(ttab.ptr);
        RMLX_TRY(run_expert_ffn_lds(gate, up, down, sh, xk, nullptr, tt, tt + 3 * (size_t)n_t, n_t, rows,
                                    static_cast<__half*>(out_f16_dev), s, nullptr, tile_rows));
        return finish(s);
      }
    }
    // where the single-row kernels take the weights (4- / 8-bit, rows in whole 16-byte pieces: a hidden size of 2880), every
    // row multiplies with its own expert on them -- an expert streamed once per row, far ahead of the portable kernels
    if (rows <= kUngroupedOnlyMaxAssignments && sh.stream_kernel != 1 && aligned16(xk) && single_row_experts(gate, up, down, sh)) {
      RMLX_TRY(h.alloc(total * sh.I * 2, s));
      RMLX_TRY(launch_qmv_m1_gate_up(gate_up_args(gate, up, sh, xk, static_cast<__half*>(h.ptr)), gate->bits, experts, rows, 1, sh.E, s));
      RMLX_TRY(launch_qmv_m1_gather(down->w, down->s, down->b, (uint64_t)sh.D * (sh.I * down->bits / 32),
                                    (uint64_t)sh.D * (sh.I / down->group_size), sh.E, static_cast<const __half*>(h.ptr), experts, rows,
                                    static_cast<__half*>(out_f16_dev), sh.D, sh.I, down->group_size, down->bits, s));
      return finish(s);
    }
    RMLX_TRY(run_expert_ffn_portable(gate, up, down, sh, xk, experts, rows, static_cast<__half*>(out_f16_dev), s));
    return finish(s);
  }
  if (!aligned16(xk)) return fail(RMLX_INVALID_SHAPE, "ExpertGroup: input must be 16-byte aligned");
  // One row per expert (a decoding token's experts): both projections on the single-row kernel's layout -- a wave per
  // pair of gate and up rows, then a wave per down row, each expert streamed once with whole-row contiguous loads.
  bool single_rows = !gemm && sh.stream_kernel != 1 && single_row_experts(gate, up, down, sh);
  for (size_t i = 0; i < n_items && single_rows; ++i) single_rows = batch_sizes_host[i] == 1;
  if (single_rows) {
    RMLX_TRY(dtab.alloc(n_items * 4, s));
    RMLX_HIP_CHECK(hipMemcpyAsync(dtab.ptr, expert_idx_host, n_items * 4, hipMemcpyHostToDevice, s));
    RMLX_HIP_CHECK(hipStreamSynchronize(s));  // the caller's host array need not outlive the call
    RMLX_TRY(h.alloc(total * sh.I * 2, s));
    const uint32_t* experts = static_cast<const uint32_t*>(dtab.ptr);
    RMLX_TRY(launch_qmv_m1_gate_up(gate_up_args(gate, up, sh, xk, static_cast<__half*>(h.ptr)), gate->bits, experts, rows, 1, sh.E, s));
    RMLX_TRY(launch_qmv_m1_gather(down->w, down->s, down->b, (uint64_t)sh.D * (sh.I * down->bits / 32),
                                  (uint64_t)sh.D * (sh.I / down->group_size), sh.E, static_cast<const __half*>(h.ptr), experts, rows,
                                  static_cast<__half*>(out_f16_dev), sh.D, sh.I, down->group_size, down->bits, s));
    return finish(s);
  }
  RMLX_TRY(dtab.alloc(tab.size() * 4, s));
  RMLX_HIP_CHECK(hipMemcpyAsync(dtab.ptr, tab.data(), tab.size() * 4, hipMemcpyHostToDevice, s));
  RMLX_HIP_CHECK(hipStreamSynchronize(s));  // `tab` is pageable host memory owned by this call
  RMLX_TRY(h.alloc(total * sh.I * 2, s));
  const uint32_t* dev_tab = static_cast<const uint32_t*>(dtab.ptr);
  RMLX_TRY(run_expert_ffn(gate, up, down, sh, xk, nullptr, dev_tab, dev_tab + 3 * (size_t)n_chunks, n_chunks,
                          static_cast<__half*>(h.ptr), out_f16_dev, 0, gemm, plan, s));
  return finish(s);
}

}  // extern "C"

namespace {
int32_t moe_grouped_impl(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                         const rmlx_array* x, const uint32_t* expert_indices_dev, const float* expert_weights_dev,
                         size_t top_k, void* out_f16_dev, size_t out_bytes, rmlx_stream stream, const FusedRoute* route,
                         Arena* arena) {
  RMLX_TRY(require_init());
  ExpertShapes sh;
  RMLX_TRY(check_expert_weights("MoeLayer", gate, up, down, &sh));
  if (x == nullptr) return fail(RMLX_INVALID_SHAPE, "MoeLayer: null input");
  if (x->ndim != 2) return fail(RMLX_INVALID_SHAPE, "MoeLayer: input must be 2D [seq_len, hidden_dim], got %dD", x->ndim);
  if (x->shape[1] != sh.D) return fail(RMLX_INVALID_SHAPE, "MoeLayer: input dim %zu != hidden_dim %u", x->shape[1], sh.D);
  if (x->dtype != RMLX_DTYPE_F16 && x->dtype != RMLX_DTYPE_F32 && x->dtype != RMLX_DTYPE_BF16)
    return fail(RMLX_INVALID_SHAPE, "MoeLayer: unsupported input dtype %s", dtype_name(x->dtype));
  if (top_k == 0 || top_k > 8) return fail(RMLX_INVALID_SHAPE, "MoeLayer: top_k must be in [1, 8], got %zu", top_k);
  const size_t T = x->shape[0];
  uint32_t T32, A;
  RMLX_TRY(checked_u32(T, "seq_len", &T32));
  RMLX_TRY(checked_u32(T * top_k, "seq_len * top_k", &A));
  RMLX_TRY(check_out("MoeLayer", out_bytes, T * sh.D * 2));
  if (T == 0) return RMLX_OK;
  hipStream_t s = (hipStream_t)stream;
  // `direct`: a few tokens, no grouping at all (below).  A call that brings logits instead of picks: the gate / up
  // workgroups of the direct form rank their token's experts themselves, so any number of tokens; `small`: at most 8
  // tokens, which the one-workgroup routing + grouping launch takes; everything else routes with the routing kernel and
  // goes on as if the caller had brought the picks.
  // (weights that no streaming kernel takes -- dimensions off the multiples of 128, group size 32 with long or odd rows --
  // stay on it until the grouped GEMM takes the batch, at every batch size where that does not take the shape either: an
  // expert per assignment on the single-row kernels is far ahead of the portable kernels)
  const uint32_t gemm_rows = expert_gemm_tile_rows(sh, A, sh.E);  // (0: the batch is below the grouped GEMM's threshold)
  // (experts in multiples of 64 that the register-weights grouped GEMM does not take -- a hidden size of 2880: the grouped form
  // of the LDS-staged GEMM from one row per expert on, where the form without grouping would stream an expert per assignment)
  // (E = 32, top-4, D = I = 2880: 16 tokens 196 us without grouping against about 300 us, 32 tokens 393 against 307 us: from three
  // rows per expert on)
  const bool lds_gemm = sh.portable && !sh.gemm && sh.gemm_lds && sh.gemm_min_rows != 0 && A >= 3 * sh.E &&
                        !ungrouped_pays(T32, sh.E, (uint32_t)top_k, gate->bits) && A / 64 + sh.E <= 65535;
  const bool only_single_row = sh.portable && gemm_rows == 0 && !lds_gemm && A <= kUngroupedOnlyMaxAssignments;
  const bool direct = (ungrouped_pays(T32, sh.E, (uint32_t)top_k, gate->bits) || only_single_row) && sh.stream_kernel != 1 &&
                      single_row_experts(gate, up, down, sh) && (route == nullptr || sh.E <= 256);
  // (its down projection adds the weighted expert outputs itself where the wave-per-tile kernel takes the weights)
  const bool fused_down = sh.wave_down && qmv_wt_combine_supported(sh.D, sh.I, down->group_size, (uint32_t)top_k);
  const bool small = route != nullptr && !sh.portable && T32 <= 8 && route_sort_fusable(T32, sh.E, (uint32_t)top_k);
  if (route != nullptr && !direct && !small) {
    RMLX_TRY(launch_topk_route(route->logits, route->bias, T32, sh.E, (uint32_t)top_k, 1, route->idx_out, route->w_out, nullptr,
                               nullptr, s));
    route = nullptr;
  }
  // many rows per expert: the grouped GEMM over row tiles instead of the streaming GEMV over chunks of 8 rows
  const uint32_t gemm = route == nullptr ? gemm_rows : 0u;
  StreamPlan plan = expert_stream_plan(sh, A, sh.E);
  if (route != nullptr && plan.chunk_rows != 8) {  // (the fused routing + grouping launch writes chunks of 8 rows)
    plan.chunk_rows = 8;
    if (plan.gate_up) plan.gate_up = 8;
    if (plan.down) plan.down = 8;
  }
  const uint32_t chunk_rows = gemm ? gemm : plan.chunk_rows;
  const uint32_t max_chunks = A / chunk_rows + (A < sh.E ? A : sh.E);
  if (max_chunks > 65535) return fail(RMLX_INVALID_SHAPE, "MoeLayer: too many row chunks (%u); split the batch", max_chunks);

  Scratch cast, meta, h, y;
  const __half* xk = static_cast<const __half*>(x->data);
  // (the form without grouping converts bf16 activations itself while it stages them: no cast launch in a decoding step)
  const bool direct_bf16 = direct && x->dtype == RMLX_DTYPE_BF16;
  if (x->dtype != RMLX_DTYPE_F16 && !direct_bf16) {
    RMLX_TRY(cast.alloc(T * sh.D * 2, s, arena));
    RMLX_TRY(launch_cast_to_f16(x->data, x->dtype, static_cast<__half*>(cast.ptr), T * sh.D, s));
    xk = static_cast<const __half*>(cast.ptr);
  }
  // A few tokens: no grouping at all.  Every assignment is one row in assignment order, and the down
  // projection adds the token's weighted expert outputs itself - two launches (gate / up that routes, down + combine)
  // instead of four, no [assignments, D] intermediate.  An expert picked by two tokens is streamed once per
  // token (at 4 tokens of 8 picks over 128 experts: 32 rows for 31 experts; see ungrouped_pays).
  if (direct) {
    if (!aligned16(xk)) return fail(RMLX_INVALID_SHAPE, "MoeLayer: input must be 16-byte aligned");
    RMLX_TRY(h.alloc((size_t)A * sh.I * 2, s, arena));
    // One row per expert: the gate / up projection on the single-row GEMV's layout (a wave per pair of gate and up rows,
    // dot products instead of a matrix unit that would multiply 15 empty rows), and no routing launch: every workgroup
    // ranks its token's experts itself, one wave, while the activations arrive (1 / 2 / 4 tokens of 8 picks: 23.4 / 37.0 /
    // 59.5 us against 24.4 / 37.8 / 61.0 us with a routing launch in front).
    QmvArgs a = gate_up_args(gate, up, sh, xk, static_cast<__half*>(h.ptr));
    a.x_bf16 = direct_bf16 ? 1 : 0;
    if (route != nullptr) {
      a.route_logits = route->logits; a.route_bias = route->bias; a.route_idx_out = route->idx_out; a.route_w_out = route->w_out;
      a.route_renorm = 1;
    }
    const uint32_t* picks = route != nullptr ? route->idx_out : expert_indices_dev;
    const float* pick_weights = route != nullptr ? route->w_out : expert_weights_dev;
    RMLX_TRY(launch_qmv_m1_gate_up(a, gate->bits, route != nullptr ? nullptr : picks, A, (uint32_t)top_k, sh.E, s));
    const uint64_t down_stride_w = (uint64_t)sh.D * (sh.I * down->bits / 32), down_stride_s = (uint64_t)sh.D * (sh.I / down->group_size);
    // (4-bit: where the wave-per-tile kernel takes the weights its down + combine is ahead, 59.7 against 64.7 us at 4 tokens)
    if (qmv_m1_down_combine_supported(sh.D, sh.I, down->group_size, down->bits, (uint32_t)top_k) && (down->bits == 8 || !fused_down)) {
      RMLX_TRY(launch_qmv_m1_down_combine(down->w, down->s, down->b, down_stride_w, down_stride_s, sh.E, static_cast<const __half*>(h.ptr),
                                          picks, pick_weights, T32, (uint32_t)top_k, sh.D, sh.I, down->group_size, down->bits,
                                          static_cast<__half*>(out_f16_dev), s));
    } else if (fused_down) {
      RMLX_TRY(launch_qmv_wt_combine(down->w, down->s, down->b, down_stride_w, down_stride_s, sh.E, static_cast<const __half*>(h.ptr),
                                     picks, pick_weights, T32, (uint32_t)top_k, sh.D, sh.I, static_cast<__half*>(out_f16_dev), s));
    } else {
      // a long intermediate dimension (beyond 4096 at 4 bits, 2048 at 8): the down projection as a single-row gather, then
      // the weighted sum of a token's rows -- three launches
      RMLX_TRY(y.alloc((size_t)A * sh.D * 2, s, arena));
      RMLX_TRY(launch_qmv_m1_gather(down->w, down->s, down->b, down_stride_w, down_stride_s, sh.E, static_cast<const __half*>(h.ptr),
                                    picks, A, static_cast<__half*>(y.ptr), sh.D, sh.I, down->group_size, down->bits, s));
      RMLX_TRY(launch_moe_combine_rows_f16(static_cast<const __half*>(y.ptr), picks, pick_weights, T32, (uint32_t)top_k, sh.D, sh.E,
                                           static_cast<__half*>(out_f16_dev), s));
    }
    return finish(s);
  }
  if (lds_gemm) {
    // grouping into row tiles of 64 (or 128) rows of one expert, then per projection: activations to the GEMM's fragment layout (through
    // the token map for the first), the grouped LDS-staged GEMM, SwiGLU as a pass of its own, and the weighted combine
    if (!aligned16(xk)) return fail(RMLX_INVALID_SHAPE, "MoeLayer: input must be 16-byte aligned");
    // (tiles of 128 rows from 64 rows per expert on: E = 32, top-4, D = I = 2880, 512 / 768 / 2048 tokens 483 / 618 / 1231 -> 470 / 491 /
    // 1023 us; at 32 rows per expert 422 against 350 us)
    const uint32_t tile_rows = A >= (uint64_t)64 * sh.E ? 128u : 64u;
    const uint32_t max_tiles = A / tile_rows + (A < sh.E ? A : sh.E);
    RMLX_TRY(meta.alloc(((size_t)3 * A + 3 * (size_t)max_tiles + 4) * 4, s, arena));
    uint32_t* sorted = static_cast<uint32_t*>(meta.ptr);
    uint32_t* sorted_tok = sorted + A;
    uint32_t* inv = sorted_tok + A;
    uint32_t* tile_tab = inv + A;
    uint32_t* n_tiles = tile_tab + 3 * (size_t)max_tiles;
    RMLX_TRY(launch_moe_sort(expert_indices_dev, A, sh.E, (uint32_t)top_k, sorted, sorted_tok, inv, nullptr, nullptr, tile_tab, n_tiles, tile_rows, s));
    Scratch y16;
    RMLX_TRY(y16.alloc((size_t)A * sh.D * 2, s, arena));
    RMLX_TRY(run_expert_ffn_lds(gate, up, down, sh, xk, sorted_tok, tile_tab, n_tiles, max_tiles, A, static_cast<__half*>(y16.ptr), s, arena, tile_rows));
    RMLX_TRY(launch_moe_combine_f16(static_cast<const __half*>(y16.ptr), inv, expert_weights_dev, T32, (uint32_t)top_k, sh.D,
                                    static_cast<__half*>(out_f16_dev), s));
    return finish(s);
  }
  // 2-bit experts: the form without grouping on the 2-bit single-row kernel with a weight matrix per row -- routing,
  // gate / up, SwiGLU, down, weighted sum, every expert streamed once per assignment in whole rows (the portable kernels
  // below are the alternative).
  if (sh.portable && !gemm && gate->bits == 2 && down->bits == 2 && (up == nullptr || (up->bits == 2 && up->group_size == gate->group_size)) &&
      A <= kUngroupedOnlyMaxAssignments && qmv_q2_supported(sh.I, sh.D, gate->group_size) &&
      qmv_q2_supported(sh.D, sh.I, down->group_size) && aligned16(xk) && aligned16(gate->w) && aligned16(down->w) &&
      (up == nullptr || aligned16(up->w)) && (!sh.fused || ((size_t)sh.I * (sh.D / 16) * 4) % 16 == 0)) {
    if (route != nullptr)
      RMLX_TRY(launch_topk_route(route->logits, route->bias, T32, sh.E, (uint32_t)top_k, 1, route->idx_out, route->w_out,
                                 nullptr, nullptr, s));
    Scratch gu, y16;
    const uint32_t gs = gate->group_size;
    const size_t rows_per_expert = sh.fused ? 2 * (size_t)sh.I : sh.I;
    const uint64_t gw = rows_per_expert * (sh.D / 16), gsb = rows_per_expert * (sh.D / gs);
    RMLX_TRY(gu.alloc((size_t)A * 2 * sh.I * 2, s, arena));
    RMLX_TRY(h.alloc((size_t)A * sh.I * 2, s, arena));
    __half* g_out = static_cast<__half*>(gu.ptr);
    if (sh.fused) {  // one stacked matrix: [A, 2I] = (gate | up)
      RMLX_TRY(launch_qmv_q2_gather(gate->w, gate->s, gate->b, gw, gsb, sh.E, xk, (uint32_t)top_k, expert_indices_dev, A, g_out,
                                    2 * sh.I, sh.D, gs, s));
      RMLX_TRY(launch_silu_gate_strided(g_out, g_out + sh.I, 2 * sh.I, static_cast<__half*>(h.ptr), A, sh.I, s));
    } else {
      __half* u_out = g_out + (size_t)A * sh.I;
      RMLX_TRY(launch_qmv_q2_gather(gate->w, gate->s, gate->b, gw, gsb, sh.E, xk, (uint32_t)top_k, expert_indices_dev, A, g_out, sh.I,
                                    sh.D, gs, s));
      RMLX_TRY(launch_qmv_q2_gather(up->w, up->s, up->b, gw, gsb, sh.E, xk, (uint32_t)top_k, expert_indices_dev, A, u_out, sh.I, sh.D,
                                    gs, s));
      RMLX_TRY(launch_silu_gate(g_out, u_out, static_cast<__half*>(h.ptr), (size_t)A * sh.I, s));
    }
    RMLX_TRY(y16.alloc((size_t)A * sh.D * 2, s, arena));
    RMLX_TRY(launch_qmv_q2_gather(down->w, down->s, down->b, (uint64_t)sh.D * (sh.I / 16), (uint64_t)sh.D * (sh.I / down->group_size),
                                  sh.E, static_cast<const __half*>(h.ptr), 1, expert_indices_dev, A, static_cast<__half*>(y16.ptr), sh.D,
                                  sh.I, down->group_size, s));
    RMLX_TRY(launch_moe_combine_rows_f16(static_cast<const __half*>(y16.ptr), expert_indices_dev, expert_weights_dev, T32,
                                         (uint32_t)top_k, sh.D, sh.E, static_cast<__half*>(out_f16_dev), s));
    return finish(s);
  }
  if (sh.portable && !gemm && arena != nullptr)
    return fail(RMLX_NOT_FOUND, "MoeLayer: these expert weights run on the portable kernels, which the entry point "
                                "without allocations does not cover (2-, 4- or 8-bit weights, group size 32, 64 or 128, "
                                "16-byte aligned buffers, whole 16-byte pieces of a row per lane)");
  if (sh.portable && !gemm) {
    // Assignments stay in their own order: position a holds token a / top_k and expert idx[a].
    if (route != nullptr)
      RMLX_TRY(launch_topk_route(route->logits, route->bias, T32, sh.E, (uint32_t)top_k, 1, route->idx_out, route->w_out,
                                 nullptr, nullptr, s));
    Scratch xr, y16;
    RMLX_TRY(meta.alloc((size_t)2 * A * 4, s));
    uint32_t* tok = static_cast<uint32_t*>(meta.ptr);
    uint32_t* ident = tok + A;
    RMLX_TRY(launch_identity_positions(tok, ident, A, (uint32_t)top_k, s));
    RMLX_TRY(xr.alloc((size_t)A * sh.D * 2, s));
    RMLX_TRY(launch_index_gather(xk, sh.D, tok, A, T32, static_cast<__half*>(xr.ptr), s));
    RMLX_TRY(y16.alloc((size_t)A * sh.D * 2, s));
    RMLX_TRY(run_expert_ffn_portable(gate, up, down, sh, static_cast<const __half*>(xr.ptr), expert_indices_dev, A,
                                     static_cast<__half*>(y16.ptr), s));
    RMLX_TRY(y.alloc((size_t)A * sh.D * 4, s));
    RMLX_TRY(launch_cast_f16_to_f32(static_cast<const __half*>(y16.ptr), static_cast<float*>(y.ptr), (size_t)A * sh.D, s));
    RMLX_TRY(launch_moe_combine(static_cast<const float*>(y.ptr), ident, expert_weights_dev, T32, (uint32_t)top_k, sh.D,
                                static_cast<__half*>(out_f16_dev), s));
    return finish(s);
  }
  if (!aligned16(xk)) return fail(RMLX_INVALID_SHAPE, "MoeLayer: input must be 16-byte aligned");
  // Gate / up in two launches, the experts split by their row count (see run_expert_ffn): between the batch sizes where
  // nearly every expert is one chunk of 8 rows and the grouped GEMM's threshold, chunks of 8 stream an expert with 9 to 16
  // rows twice and chunks of 16 on the wave-per-tile kernel are slower for the others.
  const bool split = route == nullptr && gemm == 0 && sh.bits == 4 && sh.wave_tiles && plan.gate_up == 0 && plan.chunk_rows == 8 &&
                     (sh.stream_kernel == 5 || (sh.stream_kernel == 0 && (uint64_t)A * 2 >= (uint64_t)kSplitMinRows2 * sh.E &&
                                                (uint64_t)sh.I * sh.D >= (4ull << 20)));  // (small experts: the second launch costs
                                                                                          // more than it saves, E = 40, D = 1536,
                                                                                          // I = 512 at 32 tokens: 48 against 35 us)
  const uint32_t cap_small = A < sh.E ? A : sh.E, cap_big = A / 8 + 1;
  const size_t split_words = split ? 3 * ((size_t)cap_small + cap_big) + 4 : 0;
  // meta: sorted[A] | sorted_tok[A] | inv[A] | chunk_tab[3*max_chunks] | n_chunks[1] (| split tables | their lengths[2])
  RMLX_TRY(meta.alloc(((size_t)3 * A + 3 * (size_t)max_chunks + 4 + split_words) * 4, s, arena));
  uint32_t* sorted = static_cast<uint32_t*>(meta.ptr);
  uint32_t* sorted_tok = sorted + A;
  uint32_t* inv = sorted_tok + A;
  uint32_t* chunk_tab = inv + A;
  uint32_t* n_chunks = chunk_tab + 3 * (size_t)max_chunks;
  uint32_t* split_tab = split ? n_chunks + 4 : nullptr;
  uint32_t* split_n = split ? split_tab + 3 * ((size_t)cap_small + cap_big) : nullptr;
  const SplitTables split_tabs{split_tab, split_n, cap_small, cap_big};
  if (route != nullptr)
    RMLX_TRY(launch_route_sort_small(route->logits, route->bias, T32, sh.E, (uint32_t)top_k, 1, route->idx_out, route->w_out,
                                     sorted, sorted_tok, inv, chunk_tab, n_chunks, s));
  else
    RMLX_TRY(launch_moe_sort(expert_indices_dev, A, sh.E, (uint32_t)top_k, sorted, sorted_tok, inv, nullptr, nullptr, chunk_tab, n_chunks,
                             chunk_rows, s, split_tab, split_n, cap_small));
  RMLX_TRY(h.alloc((size_t)A * sh.I * 2, s, arena));
  RMLX_TRY(y.alloc((size_t)A * sh.D * 4, s, arena));
  RMLX_TRY(run_expert_ffn(gate, up, down, sh, xk, sorted_tok, chunk_tab, n_chunks, max_chunks,
                          static_cast<__half*>(h.ptr), y.ptr, 1, gemm, plan, s, split ? &split_tabs : nullptr));
  RMLX_TRY(launch_moe_combine(static_cast<const float*>(y.ptr), inv, expert_weights_dev, T32, (uint32_t)top_k, sh.D,
                              static_cast<__half*>(out_f16_dev), s));
  return finish(s);
}
}  // namespace

extern "C" {

size_t rmlx_hip_qweight_gemm_layout_bytes(const rmlx_qweight* qw) {
  if (qw == nullptr || qw->n_experts != 1) return 0;
  return gemm_layout_bytes(qw->out_features, qw->in_features, qw->bits);
}

int32_t rmlx_hip_qweight_set_gemm_layout(rmlx_qweight* qw, void* dst_dev, size_t dst_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (qw == nullptr) return fail(RMLX_INVALID_SHAPE, "QuantizedWeight: null handle");
  if (dst_dev == nullptr) {  // back to the one layout
    qw->gemm_packed = nullptr;
    return RMLX_OK;
  }
  const size_t need = rmlx_hip_qweight_gemm_layout_bytes(qw);
  if (need == 0)
    return fail(RMLX_INVALID_SHAPE, "QuantizedWeight: no GEMM layout for this weight (4- or 8-bit, out_features %% 128 == 0, in_features %% 512 == 0, "
                                    "one expert; got bits=%u out_features=%zu in_features=%zu n_experts=%zu)", qw->bits, qw->out_features,
                qw->in_features, qw->n_experts);
  if (dst_bytes < need) return fail(RMLX_INVALID_SHAPE, "QuantizedWeight: GEMM layout buffer too small: %zu bytes < expected %zu bytes", dst_bytes, need);
  if (!aligned16(dst_dev) || !aligned16(qw->w)) return fail(RMLX_INVALID_SHAPE, "QuantizedWeight: GEMM layout buffers must be 16-byte aligned");
  uint32_t N, K;
  RMLX_TRY(checked_u32(qw->out_features, "out_features", &N));
  RMLX_TRY(checked_u32(qw->in_features, "in_features", &K));
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_gemm_repack(qw->w, N, K, qw->bits, dst_dev, s));
  RMLX_TRY(finish(s));
  qw->gemm_packed = dst_dev;
  return RMLX_OK;
}

uint32_t rmlx_hip_qweight_set_expert_gemm_min_rows(rmlx_qweight* qw, uint32_t min_rows) {
  if (qw == nullptr) return 0;
  const uint32_t prev = qw->expert_gemm_min_rows;
  qw->expert_gemm_min_rows = min_rows;
  return prev;
}

uint32_t rmlx_hip_qweight_set_expert_stream_kernel(rmlx_qweight* qw, uint32_t kind) {
  if (qw == nullptr) return 0;
  const uint32_t prev = qw->expert_stream_kernel;
  if (kind <= 5) qw->expert_stream_kernel = kind;
  return prev;
}

int32_t rmlx_hip_moe_forward_grouped(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                                     const rmlx_array* x, const uint32_t* expert_indices_dev,
                                     const float* expert_weights_dev, size_t top_k, void* out_f16_dev, size_t out_bytes,
                                     rmlx_stream stream) {
  return moe_grouped_impl(gate, up, down, x, expert_indices_dev, expert_weights_dev, top_k, out_f16_dev, out_bytes, stream,
                          nullptr, nullptr);
}

}  // extern "C"

namespace {
int32_t moe_forward_impl(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                         const rmlx_array* x, const rmlx_array* gate_logits, size_t top_k,
                         const rmlx_array* expert_bias, void* out_f16_dev, size_t out_bytes, rmlx_stream stream,
                         Arena* arena) {
  RMLX_TRY(require_init());
  if (x == nullptr || gate_logits == nullptr) return fail(RMLX_INVALID_SHAPE, "MoeLayer: null argument");
  if (gate_logits->ndim != 2 || x->ndim != 2 || gate_logits->shape[0] != x->shape[0])
    return fail(RMLX_INVALID_SHAPE, "MoeLayer: gate_logits must be [seq_len, num_experts] matching x");
  if (gate != nullptr && gate_logits->shape[1] != gate->n_experts)
    return fail(RMLX_INVALID_SHAPE, "MoeLayer: gate_logits has %zu experts but the weights hold %zu",
                gate_logits->shape[1], gate->n_experts);
  const size_t T = x->shape[0];
  if (top_k == 0 || top_k > 8) return fail(RMLX_INVALID_SHAPE, "gpu_topk_route: top_k must be in [1, 8], got %zu", top_k);
  hipStream_t s = (hipStream_t)stream;
  Scratch route;
  RMLX_TRY(route.alloc(T * top_k * 8 + 16, s, arena));
  uint32_t* idx = static_cast<uint32_t*>(route.ptr);
  float* wts = reinterpret_cast<float*>(idx + T * top_k);
  // f32 logits (and bias): the block picks its routed form itself (moe_grouped_impl)
  if (gate != nullptr && gate_logits->dtype == RMLX_DTYPE_F32 && gate_logits->data != nullptr && top_k <= gate->n_experts &&
      (expert_bias == nullptr || (expert_bias->dtype == RMLX_DTYPE_F32 && expert_bias->ndim == 1 &&
                                  expert_bias->shape[0] == gate->n_experts && expert_bias->data != nullptr)) &&
      gate->n_experts <= 256) {
    const FusedRoute fr{static_cast<const float*>(gate_logits->data),
                        expert_bias != nullptr ? static_cast<const float*>(expert_bias->data) : nullptr, idx, wts};
    return moe_grouped_impl(gate, up, down, x, idx, wts, top_k, out_f16_dev, out_bytes, stream, &fr, arena);
  }
  // Asynchronous inner calls need a real stream handle: the null stream means "synchronous".
  RMLX_TRY(topk_route_impl(gate_logits, top_k, expert_bias, 1, idx, wts, nullptr, nullptr, stream, arena));
  RMLX_TRY(moe_grouped_impl(gate, up, down, x, idx, wts, top_k, out_f16_dev, out_bytes, stream, nullptr, arena));
  return finish(s);
}
}  // namespace

extern "C" {

int32_t rmlx_hip_moe_forward(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                             const rmlx_array* x, const rmlx_array* gate_logits, size_t top_k,
                             const rmlx_array* expert_bias, void* out_f16_dev, size_t out_bytes, rmlx_stream stream) {
  return moe_forward_impl(gate, up, down, x, gate_logits, top_k, expert_bias, out_f16_dev, out_bytes, stream, nullptr);
}

// The routed block for callers that cannot allocate (HIP graph capture, serving loops that forbid it): every
// intermediate is carved from the static workspace, so the call makes no hipMalloc / hipFree.  Calls on one GPU
// share that workspace: two of them in flight at the same time race.
int32_t rmlx_hip_moe_forward_noalloc(const rmlx_qweight* gate, const rmlx_qweight* up, const rmlx_qweight* down,
                                     const rmlx_array* x, const rmlx_array* gate_logits, size_t top_k,
                                     const rmlx_array* expert_bias, void* out_f16_dev, size_t out_bytes,
                                     rmlx_stream stream) {
  RMLX_TRY(require_init());
  void* base = ctx().device < kMaxDevices ? g_static_scratch[ctx().device] : nullptr;
  if (base == nullptr) return fail(RMLX_RUNTIME_ERROR, "the static workspace was not resolved on device %d", ctx().device);
  if (gate == nullptr || down == nullptr || x == nullptr || gate_logits == nullptr)
    return fail(RMLX_INVALID_SHAPE, "MoeLayer: null argument");
  if (x->ndim == 2 && top_k >= 1 && top_k <= 8) {
    // upper bound of what the block carves, every piece rounded up to 256 bytes
    const size_t T = x->shape[0], A = T * top_k, E = gate->n_experts, D = gate->in_features;
    const size_t I = up == nullptr ? gate->out_features / 2 : gate->out_features;
    auto r256 = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t max_chunks = A / 8 + (A < E ? A : E);
    const size_t split_words = 3 * ((A < E ? A : E) + A / 8 + 1) + 4;  // (the two tables of the split gate / up launch)
    size_t need = r256(A * 8 + 16) + r256((3 * A + 3 * max_chunks + 4 + split_words) * 4) + r256(A * I * 2) + r256(A * D * 4);
    if (x->dtype != RMLX_DTYPE_F16) need += r256(T * D * 2);
    if (gate_logits->dtype == RMLX_DTYPE_F16) need += r256(T * E * 4);
    if (expert_bias != nullptr && expert_bias->dtype == RMLX_DTYPE_F16) need += r256(E * 4);
    if (need > kStaticScratchBytes)
      return fail(RMLX_INVALID_SHAPE,
                  "MoeLayer (entry point without allocations): %zu tokens x top-%zu at hidden %zu / intermediate %zu need "
                  "%zu bytes of workspace, the static workspace holds %zu; split the batch or call rmlx_hip_moe_forward",
                  T, top_k, D, I, need, kStaticScratchBytes);
  }
  Arena arena;
  arena.base = static_cast<char*>(base);
  arena.capacity = kStaticScratchBytes;
  return moe_forward_impl(gate, up, down, x, gate_logits, top_k, expert_bias, out_f16_dev, out_bytes, stream, &arena);
}

// ---- AWQ / GPTQ dequantisation ---------------------------------------------------------------------

int32_t rmlx_hip_awq_dequant(const void* qweight_dev, size_t qweight_bytes, const void* qzeros_dev,
                             size_t qzeros_bytes, const void* scales_f32_dev, size_t scales_bytes, size_t rows,
                             size_t cols, size_t group_size, void* out_f32_dev, size_t out_bytes,
                             rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (cols % 8 != 0) return fail(RMLX_INVALID_SHAPE, "awq_dequant: cols (%zu) must be a multiple of 8 (pack factor)", cols);
  if (group_size == 0) return fail(RMLX_INVALID_SHAPE, "awq_dequant: group_size must be > 0");
  if (rows % group_size != 0)
    return fail(RMLX_INVALID_SHAPE, "awq_dequant: rows (%zu) must be a multiple of group_size (%zu)", rows, group_size);
  const size_t num_groups = rows / group_size, cols_packed = cols / 8;
  if (qweight_bytes < rows * cols_packed * 4)
    return fail(RMLX_INVALID_SHAPE, "awq_dequant: qweight buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                qweight_bytes, rows * cols_packed * 4, rows, cols_packed);
  if (qzeros_bytes < num_groups * cols_packed * 4)
    return fail(RMLX_INVALID_SHAPE, "awq_dequant: qzeros buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                qzeros_bytes, num_groups * cols_packed * 4, num_groups, cols_packed);
  if (scales_bytes < num_groups * cols * 4)
    return fail(RMLX_INVALID_SHAPE, "awq_dequant: scales buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                scales_bytes, num_groups * cols * 4, num_groups, cols);
  RMLX_TRY(check_out("awq_dequant", out_bytes, rows * cols * 4));
  uint32_t r32, c32, g32;
  RMLX_TRY(checked_u32(rows, "rows", &r32));
  RMLX_TRY(checked_u32(cols, "cols", &c32));
  RMLX_TRY(checked_u32(group_size, "group_size", &g32));
  if (rows * cols != 0 && (qweight_dev == nullptr || qzeros_dev == nullptr || scales_f32_dev == nullptr || out_f32_dev == nullptr))
    return fail(RMLX_INVALID_SHAPE, "awq_dequant: null device buffer");
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_awq_dequant(static_cast<const uint32_t*>(qweight_dev), static_cast<const uint32_t*>(qzeros_dev),
                              static_cast<const float*>(scales_f32_dev), static_cast<float*>(out_f32_dev), r32, c32,
                              g32, s));
  return finish(s);
}

int32_t rmlx_hip_gptq_dequant(const void* qweight_dev, size_t qweight_bytes, const void* qzeros_dev,
                              size_t qzeros_bytes, const void* scales_f32_dev, size_t scales_bytes,
                              const int32_t* g_idx_dev, size_t g_idx_bytes, size_t in_features, size_t out_features,
                              size_t group_size, void* out_f32_dev, size_t out_bytes, rmlx_stream stream) {
  RMLX_TRY(require_init());
  if (in_features % 8 != 0)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: in_features (%zu) must be a multiple of 8 (pack factor)", in_features);
  if (out_features % 8 != 0)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: out_features (%zu) must be a multiple of 8 (pack factor for qzeros)",
                out_features);
  if (group_size == 0) return fail(RMLX_INVALID_SHAPE, "gptq_dequant: group_size must be > 0");
  const bool has_g_idx = g_idx_dev != nullptr;
  if (!has_g_idx && in_features % group_size != 0)
    return fail(RMLX_INVALID_SHAPE,
                "gptq_dequant: in_features (%zu) must be a multiple of group_size (%zu) when g_idx is not provided",
                in_features, group_size);
  const size_t rows_packed = in_features / 8, cols_packed = out_features / 8;
  // with g_idx the group count is whatever the scales buffer holds (quantized.rs:2443-2450)
  const size_t num_groups = has_g_idx ? (out_features == 0 ? 0 : scales_bytes / 4 / out_features) : in_features / group_size;
  if (qweight_bytes < rows_packed * out_features * 4)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: qweight buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                qweight_bytes, rows_packed * out_features * 4, rows_packed, out_features);
  if (qzeros_bytes < num_groups * cols_packed * 4)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: qzeros buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                qzeros_bytes, num_groups * cols_packed * 4, num_groups, cols_packed);
  if (scales_bytes < num_groups * out_features * 4)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: scales buffer too small: %zu bytes < expected %zu bytes for [%zu, %zu]",
                scales_bytes, num_groups * out_features * 4, num_groups, out_features);
  if (has_g_idx && g_idx_bytes < in_features * 4)
    return fail(RMLX_INVALID_SHAPE, "gptq_dequant: g_idx buffer too small: %zu bytes < expected %zu bytes for [%zu]",
                g_idx_bytes, in_features * 4, in_features);
  RMLX_TRY(check_out("gptq_dequant", out_bytes, in_features * out_features * 4));
  uint32_t k32, n32, g32, ng32;
  RMLX_TRY(checked_u32(in_features, "in_features", &k32));
  RMLX_TRY(checked_u32(out_features, "out_features", &n32));
  RMLX_TRY(checked_u32(group_size, "group_size", &g32));
  RMLX_TRY(checked_u32(num_groups, "num_groups", &ng32));
  if (in_features * out_features != 0) {
    if (qweight_dev == nullptr || qzeros_dev == nullptr || scales_f32_dev == nullptr || out_f32_dev == nullptr)
      return fail(RMLX_INVALID_SHAPE, "gptq_dequant: null device buffer");
    if (num_groups == 0) return fail(RMLX_INVALID_SHAPE, "gptq_dequant: the scales buffer holds no complete group");
  }
  hipStream_t s = (hipStream_t)stream;
  RMLX_TRY(launch_gptq_dequant(static_cast<const uint32_t*>(qweight_dev), static_cast<const uint32_t*>(qzeros_dev),
                               static_cast<const float*>(scales_f32_dev), g_idx_dev, static_cast<float*>(out_f32_dev),
                               k32, n32, g32, ng32, s));
  return finish(s);
}

}  // extern "C"
