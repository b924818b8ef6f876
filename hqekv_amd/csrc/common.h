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

// butterfly exchange across the 64-lane wavefront
__device__ __forceinline__ float xor_f(float v, int m) { return __shfl_xor(v, m, HQ_WAVE); }
__device__ __forceinline__ uint32_t xor_u(uint32_t v, int m) {
  return (uint32_t)__shfl_xor((int)v, m, HQ_WAVE);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += xor_f(v, m);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, xor_f(v, m));
  return v;
}

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
