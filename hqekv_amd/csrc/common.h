// Shared device/host helpers for libhqekv (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hqekv.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

#define HQ_WAVE 64

namespace hq {

// host side: record an error string (thread local) and return the code
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

__device__ __forceinline__ float h2f(half_t h) { return (float)h; }
__device__ __forceinline__ half_t f2h(float f) { return (half_t)f; }

// bit-field extract of a `bits`-wide code at position i of a packed word
template <int BITS>
__device__ __forceinline__ uint32_t code_at(uint32_t w, int i) {
  return __builtin_amdgcn_ubfe(w, (uint32_t)(i * BITS), (uint32_t)BITS);
}

// exchange with the lane 1 or 2 apart inside a quad: one DPP move, no trip through the LDS crossbar
template <int M>
__device__ __forceinline__ uint32_t quad_xor_u(uint32_t v) {
  static_assert(M == 1 || M == 2, "quad permutes reach the lanes 1 and 2 apart");
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, M == 1 ? 0xB1 : 0x4E, 0xf, 0xf, true);
}
template <int M>
__device__ __forceinline__ float quad_xor_f(float v) {
  return __builtin_bit_cast(float, quad_xor_u<M>(__builtin_bit_cast(uint32_t, v)));
}

// butterfly exchange across the 64-lane wavefront (through the LDS crossbar: keep it off hot paths)
__device__ __forceinline__ float xor_f(float v, int m) { return __shfl_xor(v, m, HQ_WAVE); }
__device__ __forceinline__ uint32_t xor_u(uint32_t v, int m) {
  return (uint32_t)__shfl_xor((int)v, m, HQ_WAVE);
}

// Wave-wide reductions without the LDS crossbar: four DPP steps reduce each row of 16 lanes in place
// (quad permutes for lanes 1 and 2 apart, then the two mirrors), two lane-row swaps bring the four row
// results into row 0, and lane 0 is broadcast.  The swaps need idle issue slots before and after them
// that the compiler does not insert around inline asm.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ void row_swap16(float &a, float &b) {
  asm volatile("s_nop 7\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 7" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void row_swap32(float &a, float &b) {
  asm volatile("s_nop 7\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 7" : "+v"(a), "+v"(b));
}
#define HQ_WAVE_REDUCE(OP_)                                              \
  v = OP_(v, dpp_f<0xB1>(v));  /* quad_perm [1,0,3,2] */                \
  v = OP_(v, dpp_f<0x4E>(v));  /* quad_perm [2,3,0,1] */                \
  v = OP_(v, dpp_f<0x141>(v)); /* row_half_mirror     */                \
  v = OP_(v, dpp_f<0x140>(v)); /* row_mirror          */                \
  float o = v;                                                           \
  row_swap16(v, o); /* rows 0 and 2: o = rows 1 and 3 */                 \
  v = OP_(v, o);                                                         \
  o = v;                                                                 \
  row_swap32(v, o); /* row 0: o = row 2 */                               \
  v = OP_(v, o);                                                         \
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
__device__ __forceinline__ float hq_add(float a, float b) { return a + b; }
__device__ __forceinline__ float wave_sum(float v) { HQ_WAVE_REDUCE(hq_add) }
__device__ __forceinline__ float wave_max(float v) { HQ_WAVE_REDUCE(fmaxf) }
#undef HQ_WAVE_REDUCE

// Buffer addressing: a 128-bit descriptor per (b, head) slab in scalar registers, a per-lane byte offset
// that never changes, and the row offset in a scalar register -- no vector ALU work per load, and reads
// past the end of the slab return zero instead of faulting.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t buf_u32(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, (int)row_off, 0);
}
// a 16-bit element, zero-extended into a 32-bit register
__device__ __forceinline__ uint32_t buf_u16(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  return (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, (int)row_off, 0);
}
__device__ __forceinline__ half_t buf_f16(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  const unsigned short u = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, (int)row_off, 0);
  half_t h;
  __builtin_memcpy(&h, &u, 2);
  return h;
}

}  // namespace hq
