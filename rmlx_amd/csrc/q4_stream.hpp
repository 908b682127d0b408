// Device helpers shared by the 4-bit streaming GEMV kernels (qmv.hip, qmv_wt.hip): nibble -> f16 unpacking with
// mask-or only, the matching activation permutation, lane exchanges, and a barrier that leaves global loads in flight.
#pragma once
#include "common.hpp"

namespace rmlx {
namespace q4 {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));


// The masks and offsets arrive in registers (Q4Consts): with one of each pair in a scalar and one in a vector
// register, and + or is a single instruction.
struct Q4Consts { uint32_t m0, m1, k0, k1; };
__device__ __forceinline__ h8 unpack_q4_word(uint32_t w, const Q4Consts& q) {
  uint32_t t = w >> 8;
  u4 p;
  p.x = (w & q.m0) | q.k0;  // k+0, k+4   (+1024)
  p.y = (w & q.m1) | q.k1;  // k+1, k+5   (+64)
  p.z = (t & q.m0) | q.k0;  // k+2, k+6   (+1024)
  p.w = (t & q.m1) | q.k1;  // k+3, k+7   (+64)
  return __builtin_bit_cast(h8, p);
}

// v + (value of lane ^ 32): v_permlane32_swap exchanges the upper half of its first operand with the lower half
// of its second, so both registers end up holding one half of v in all lanes.  (Written as assembly: through the
// builtin this compiler reads the first result twice.  The wait states cover a vector write just before.)
__device__ __forceinline__ float add_other_half(float v) {
  uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1" : "+v"(a), "+v"(b));
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}

// x halves (k0..k7) -> slot order (0,4,1,5,2,6,3,7), matching unpack_q4_word.
__device__ __forceinline__ u4 permute_x8(u4 d) {
  u4 o;
  o.x = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);
  return o;
}

// 8 bf16 values -> 8 f16 values through f32, rounded to nearest even (what the cast kernel does)
__device__ __forceinline__ u4 bf16x8_to_f16(u4 v) {
  typedef _Float16 h2c __attribute__((ext_vector_type(2)));
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
    const h2c pair = {(_Float16)lo, (_Float16)hi};
    w[e] = __builtin_bit_cast(uint32_t, pair);
  }
  return (u4){w[0], w[1], w[2], w[3]};
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + __expf(-v)); }

__device__ __forceinline__ uint32_t swap16(uint32_t v) {  // value of lane ^ 16
  return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F);
}

__device__ __forceinline__ float swap8(float v) {  // value of lane ^ 8
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x201F));
}

struct __attribute__((packed, aligned(4))) U4Unaligned { uint32_t v[4]; };

// Workgroup barrier for data exchanged through LDS: waits for this wave's LDS traffic only.  (__syncthreads() also
// waits for every global load in flight, i.e. for the next tile's weights that were requested on purpose.)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

}  // namespace q4
}  // namespace rmlx
