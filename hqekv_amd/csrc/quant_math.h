// Arithmetic shared by the quantise / dequantise kernels and the cache-migration kernel (gfx950): every routine
// here evaluates one step of the reference's fp16 chains with its roundings made explicit, so that any kernel
// built from them produces the same bits.  Include after "common.h", with fp contraction off.
#pragma once

#include "common.h"

#pragma clang fp contract(off)

namespace hq {

typedef float float2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t h2_bits(half2_t h) {
  uint32_t u;
  __builtin_memcpy(&u, &h, 4);
  return u;
}
__device__ __forceinline__ half2_t bits_h2(uint32_t u) {
  half2_t h;
  __builtin_memcpy(&h, &u, 4);
  return h;
}

// How the element-wise part of the chain is evaluated (results are those of the chain above, bit for bit):
//  * u = rnd16(x - mn) is one packed fp16 subtraction.  Rounding an fp16 sum first to fp32 (24-bit
//    significand >= 2*11+2) and then to fp16 gives the directly rounded fp16 sum, so there is nothing
//    to gain from the detour through fp32 that the op-by-op evaluation takes.
//  * v = rnd16(f32(u) / f32(scale)) is rnd16(f32(u) * r) with r the fp32 reciprocal of the group's
//    scale after one Newton step.  A quotient of two 11-bit significands is never closer than
//    1/(2047*4095) (relative) to a midpoint of the fp16 grid, which is more than the error of the
//    rounded product; hqekv_selftest_quant_division compares the two over all 2^32 operand pairs.
//    scale == 0 (constant group, or a range that underflows) and a non-finite scale keep the hardware
//    reciprocal (inf / 0 / NaN), which reproduces x/0 = inf, 0/0 = NaN and x/inf = 0.
//  * rne(clamp(v, 0, qmax)) is read from the significand of rnd16(clamp(v) + 1024): the fp16 grid has
//    spacing 1 on [1024, 2048) and 1024 is even, so the sum is 1024 + rne(v) exactly.  max() drops a
//    NaN operand, which turns the 0/0 of a constant group into code 0.
__device__ __forceinline__ float group_recip(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  const float e = __builtin_fmaf(-s, r0, 1.0f);
  const float r = __builtin_fmaf(e, r0, r0);
  // +-normal or +-denormal: classes 3, 4, 7, 8
  return __builtin_amdgcn_classf(s, 0x198) ? r : r0;
}

// fp16 bit patterns of 1024 + code for the pair (a, b) of already centred (x - mn) fp32 values
template <int BITS>
__device__ __forceinline__ uint32_t code_pair_biased(float ua, float ra, float ub, float rb) {
  constexpr _Float16 QMAX = (_Float16)((1 << BITS) - 1);
  const float2_t q = {ua * ra, ub * rb};
  half2_t v = __builtin_convertvector(q, half2_t);
  v = __builtin_elementwise_max(v, (half2_t){(_Float16)0, (_Float16)0});
  v = __builtin_elementwise_min(v, (half2_t){QMAX, QMAX});
  v = v + (half2_t){(_Float16)1024, (_Float16)1024};
  return h2_bits(v);
}

// z[i] holds (1024 + code[i], 1024 + code[i + N]) for i < N, N * BITS <= 16:
// returns code[i] at bit i*BITS and code[i + N] at bit 16 + i*BITS.
template <int BITS, int N>
__device__ __forceinline__ uint32_t horner_pack(const uint32_t *z) {
  constexpr uint32_t MASK = ((1u << BITS) - 1u) * 0x00010001u;
  uint32_t w = z[N - 1] & MASK;
#pragma unroll
  for (int i = N - 2; i >= 0; --i) w = (z[i] & MASK) | (w << BITS);
  return w;
}

// torch.min / torch.max over a group return the element with the LOWEST INDEX among equal ones (ATen's
// MinOps / MaxOps break ties by index), which decides the sign of a minimum or maximum that is zero when the group
// holds both +0 and -0.  The hardware minimum prefers -0 and the maximum +0, so groups whose minimum or maximum is
// a zero look the sign up: the bit pattern of the first zero among N values in index order, or 1 if there is none.
template <int N>
__device__ __forceinline__ uint32_t first_zero_bits(const half_t (&x)[N]) {
  uint32_t r = 1u;
#pragma unroll
  for (int i = N - 1; i >= 0; --i) {
    const uint32_t b = (uint32_t)__builtin_bit_cast(unsigned short, x[i]);
    if ((b & 0x7fffu) == 0u) r = b;
  }
  return r;
}

struct Normal1Stats {
  half_t mean_h, std_h;
  float thr;  // std * 2^-25
};
struct Welford {
  float mean, m2;
};
// merge of two adjacent halves of n_half elements each (n_half a power of two, so every factor is exact)
__device__ __forceinline__ Welford welford_merge(Welford a, Welford b, float n_half) {
  const float delta = b.mean - a.mean;
  Welford r;
  r.mean = a.mean + delta * 0.5f;
  r.m2 = (a.m2 + b.m2) + ((delta * delta) * n_half) * 0.5f;
  return r;
}
// the tree over N = 2^k adjacent values held by one lane
template <int N>
__device__ __forceinline__ Welford welford_tree(const float (&x)[N]) {
  Welford w[N];
#pragma unroll
  for (int i = 0; i < N; ++i) w[i] = Welford{x[i], 0.f};
#pragma unroll
  for (int span = 1; span < N; span *= 2)
#pragma unroll
    for (int i = 0; i < N; i += 2 * span) w[i] = welford_merge(w[i], w[i + span], (float)span);
  return w[0];
}
__device__ __forceinline__ Normal1Stats normal1_finish(Welford w) {
  Normal1Stats st;
  st.mean_h = (half_t)w.mean;
  st.std_h = (half_t)__builtin_sqrtf(w.m2 / 31.0f);
  st.thr = (float)st.std_h * 0x1p-25f;
  return st;
}
__device__ __forceinline__ uint32_t normal1_code(half_t u, float thr) {
  const float uf = (float)u;
  return (uf > 0.0f && uf > thr) ? 1u : 0u;
}

}  // namespace hq
