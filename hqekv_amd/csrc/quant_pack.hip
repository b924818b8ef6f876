// Quantise-and-pack / unpack-and-dequantise kernels (gfx950).
//
// The arithmetic follows, operation for operation, the fp16 chain of the reference quantiser
// (quant/pack_unpack.py:166-175) as PyTorch evaluates it on a GPU:
//   mn, mx            group min / max
//   d     = rnd16(mx - mn)
//   scale = rnd16(f32(d) * (1.0f / qmax))        tensor / python-int = multiply by fp32 reciprocal
//   u     = rnd16(x - mn)
//   v     = rnd16(f32(u) / f32(scale))           correctly rounded fp32 divide
//   code  = int(rne(clamp(v, 0, qmax)))          NaN (0/0 of a constant group) -> 0
// and the pack of quant/pack_unpack.py:40-51: word_j = OR_i code[j*pf+i] << (i*bits).
// Every fp16 rounding above is made explicit through a conversion so the compiler cannot
// contract or reassociate across it.
#include "common.h"
#include "quant_math.h"

#pragma clang fp contract(off)

namespace hq {

// ---------------------------------------------------------------- rows: groups along a contiguous axis
// 4 lanes per 32-element group, 8 contiguous fp16 (one 128-bit load) per lane.  grid.x enumerates
// (outer slab, block of 64 groups); a slab's groups are numbered row-major over (row, group in row).
template <int BITS>
__global__ __launch_bounds__(256) void quant_rows_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xr, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ scale, half_t *__restrict__ zero, int64_t so, int64_t sr,
    uint32_t groups_per_row, int gpr_shift, uint32_t groups_per_slab, uint32_t blocks_per_slab) {
  constexpr int PF = 32 / BITS;
  constexpr float INV_QMAX = 1.0f / (float)((1 << BITS) - 1);
  const uint32_t o = blockIdx.x / blocks_per_slab;
  const uint32_t blk = blockIdx.x - o * blocks_per_slab;
  const uint32_t gin = blk * 64u + (threadIdx.x >> 2);
  const uint32_t sub = threadIdx.x & 3;
  if (gin >= groups_per_slab) return;  // the four lanes of a group leave together
  uint32_t r, g;
  if (gpr_shift >= 0) {
    r = gin >> gpr_shift;
    g = gin & (groups_per_row - 1u);
  } else {
    r = gin / groups_per_row;
    g = gin - r * groups_per_row;
  }

  const uint4 raw = *reinterpret_cast<const uint4 *>(x + (int64_t)o * xo + (int64_t)r * xr + g * 32u + sub * 8u);
  const half2_t p[4] = {bits_h2(raw.x), bits_h2(raw.y), bits_h2(raw.z), bits_h2(raw.w)};

  half2_t lo2 = __builtin_elementwise_min(__builtin_elementwise_min(p[0], p[1]), __builtin_elementwise_min(p[2], p[3]));
  half2_t hi2 = __builtin_elementwise_max(__builtin_elementwise_max(p[0], p[1]), __builtin_elementwise_max(p[2], p[3]));
  // (min, -max) in one register: one packed min per butterfly step serves both
  half2_t mm = {(half_t)__builtin_fminf((float)lo2[0], (float)lo2[1]), (half_t)(-__builtin_fmaxf((float)hi2[0], (float)hi2[1]))};
  mm = __builtin_elementwise_min(mm, bits_h2(quad_xor_u<1>(h2_bits(mm))));
  mm = __builtin_elementwise_min(mm, bits_h2(quad_xor_u<2>(h2_bits(mm))));
  half_t mn_h = mm[0];
  float mn = (float)mn_h, mx = -(float)mm[1];
  // A zero extreme takes the sign of the group's first zero (torch's tie rule, see first_zero_bits).  The wave
  // branches around this as a whole (a scalar branch on the ballot): groups with a zero extreme are rare, and a
  // predicated copy of the block in every lane's path cost the kernel 5-10 %.
  const bool zero_extreme = __builtin_fminf(__builtin_fabsf(mn), __builtin_fabsf(mx)) == 0.0f;   // mn == 0 or mx == 0
  if (__builtin_amdgcn_ballot_w64(zero_extreme) != 0 && zero_extreme) {
    // (the condition is the same for the four lanes of a group: they hold its minimum and maximum)
    const half_t mine[8] = {p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
    const uint32_t own = first_zero_bits(mine);
    const uint32_t x1 = quad_xor_u<1>(own), x2 = quad_xor_u<2>(own), x3 = quad_xor_u<1>(x2);  // lanes sub^1, sub^2, sub^3
    uint32_t by_lane[4];
#pragma unroll
    for (int l = 0; l < 4; ++l) by_lane[l] = (sub == (uint32_t)l) ? own : (sub == (uint32_t)(l ^ 1)) ? x1 : (sub == (uint32_t)(l ^ 2)) ? x2 : x3;
    uint32_t first = 1u;
#pragma unroll
    for (int l = 3; l >= 0; --l)
      if (by_lane[l] != 1u) first = by_lane[l];
    const half_t z = __builtin_bit_cast(half_t, (unsigned short)first);   // (a zero extreme implies a zero element)
    if (mn == 0.0f) {
      mn_h = z;
      mn = (float)z;
    }
    if (mx == 0.0f) mx = (float)z;
  }

  const half_t d = (half_t)(mx - mn);
  const half_t sc = (half_t)((float)d * INV_QMAX);
  const float rcp = group_recip((float)sc);

  const half2_t mn2 = {mn_h, mn_h};
  float u[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t c = p[i] - mn2;
    u[2 * i] = (float)c[0];
    u[2 * i + 1] = (float)c[1];
  }

  uint32_t *crow = code + (int64_t)o * co + (int64_t)r * cr + g * (32 / PF);
  if (BITS == 8) {
    uint32_t z[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      z[0] = code_pair_biased<8>(u[4 * h + 0], rcp, u[4 * h + 2], rcp);
      z[1] = code_pair_biased<8>(u[4 * h + 1], rcp, u[4 * h + 3], rcp);
      crow[sub * 2 + h] = horner_pack<8, 2>(z);
    }
  } else {
    uint32_t z[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) z[i] = code_pair_biased<BITS>(u[i], rcp, u[i + 4], rcp);
    if (BITS == 4) {
      crow[sub] = horner_pack<4, 4>(z);
    } else if (BITS == 1) {
      const uint32_t w = horner_pack<1, 4>(z);             // codes 0-3 in bits 0-3, codes 4-7 in bits 16-19
      const uint32_t b8 = (w & 0xfu) | ((w >> 12) & 0xf0u);  // this lane's 8 codes
      const uint32_t b16 = b8 | (quad_xor_u<1>(b8) << 8);        // even lanes: two lanes' codes in order
      const uint32_t other = quad_xor_u<2>(b16);
      if (sub == 0) crow[0] = b16 | (other << 16);
    } else {
      const uint32_t w = horner_pack<2, 4>(z);             // codes 0-3 in byte 0, codes 4-7 in byte 2
      const uint32_t h = __builtin_amdgcn_perm(0u, w, 0x0c0c0200u);   // 16 bits: this lane's 8 codes
      const uint32_t other = quad_xor_u<1>(h);
      if ((sub & 1) == 0) crow[sub >> 1] = h | (other << 16);
    }
  }
  if (sub == 0) {
    scale[(int64_t)o * so + (int64_t)r * sr + g] = sc;
    zero[(int64_t)o * so + (int64_t)r * sr + g] = mn_h;
  }
}

// ---------------------------------------------------------------- K handed over token-major
// A workgroup of 8 wavefronts takes 256 tokens (8 groups of 32) of one slab.  Within a wavefront a lane
// owns two adjacent channels (lane & 7) of one token group (lane >> 3) and keeps that 32 x 2 fp16 tile in
// registers; the 8 wavefronts cover 128 channels per pass.  The eight lanes that share a channel pair hold
// eight consecutive token groups, so each channel row of the code / scale / zero planes is written in runs
// of 8 groups (64 to 256 bytes of codes) instead of one group at a time.
constexpr int QK_GROUPS_PER_BLOCK = 8;

template <int BITS>
__global__ __launch_bounds__(512) void quant_k_tokenmajor_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xt, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ scale, half_t *__restrict__ zero, int64_t so, int64_t sr,
    uint32_t D, uint32_t n_groups) {
  constexpr int PF = 32 / BITS;
  constexpr int WPG = 32 / PF;  // words per group
  constexpr int HALF = PF / 2;
  constexpr float INV_QMAX = 1.0f / (float)((1 << BITS) - 1);
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t cp = lane & 7u, tg = lane >> 3;
  const uint32_t G0 = blockIdx.x * QK_GROUPS_PER_BLOCK;
  const uint32_t G = G0 + tg;
  const int64_t o = blockIdx.y;
  const uint32_t row_b = (uint32_t)xt * 2u;  // bytes between token rows
  const uint32_t groups_here = min((uint32_t)QK_GROUPS_PER_BLOCK, n_groups - G0);
  const rsrc_t rx = make_rsrc(x + o * xo + (int64_t)G0 * 32 * xt, (groups_here * 32u - 1u) * row_b + D * 2u);

  for (uint32_t c0 = wv * 16u; c0 < D; c0 += 128u) {
    const uint32_t c = c0 + cp * 2u;
    const bool live = (G < n_groups) && (c < D);
    const uint32_t voff = live ? tg * 32u * row_b + c * 2u : 0u;  // idle lanes re-read the first element
    half2_t t[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) t[k] = bits_h2(buf_u32(rx, voff, (uint32_t)k * row_b));

    half2_t lo2 = t[0], hi2 = t[0];
#pragma unroll
    for (int k = 1; k < 32; ++k) {
      lo2 = __builtin_elementwise_min(lo2, t[k]);
      hi2 = __builtin_elementwise_max(hi2, t[k]);
    }
    const bool zero_extreme = (float)lo2[0] == 0.0f || (float)hi2[0] == 0.0f || (float)lo2[1] == 0.0f || (float)hi2[1] == 0.0f;
    if (__builtin_amdgcn_ballot_w64(zero_extreme) != 0)   // rare: the wave branches around it as a whole
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      if ((float)lo2[ch] == 0.0f || (float)hi2[ch] == 0.0f) {  // a zero extreme takes the sign of the group's first zero
        half_t col[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) col[k] = t[k][ch];
        const half_t z = __builtin_bit_cast(half_t, (unsigned short)first_zero_bits(col));
        if ((float)lo2[ch] == 0.0f) lo2[ch] = z;
        if ((float)hi2[ch] == 0.0f) hi2[ch] = z;
      }
    }
    half_t sc[2];
    float rcp[2];
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      const half_t d = (half_t)((float)hi2[ch] - (float)lo2[ch]);
      sc[ch] = (half_t)((float)d * INV_QMAX);
      rcp[ch] = group_recip((float)sc[ch]);
    }
    float u[2][32];
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      const half2_t cpair = t[k] - lo2;
      u[0][k] = (float)cpair[0];
      u[1][k] = (float)cpair[1];
    }
    if (live) {
#pragma unroll
      for (int ch = 0; ch < 2; ++ch) {
        uint32_t *crow = code + o * co + (int64_t)(c + ch) * cr + (int64_t)G * WPG;
#pragma unroll
        for (int wj = 0; wj < WPG; ++wj) {
          uint32_t z[HALF];
#pragma unroll
          for (int i = 0; i < HALF; ++i)
            z[i] = code_pair_biased<BITS>(u[ch][wj * PF + i], rcp[ch], u[ch][wj * PF + i + HALF], rcp[ch]);
          crow[wj] = horner_pack<BITS, HALF>(z);
        }
        scale[o * so + (int64_t)(c + ch) * sr + G] = sc[ch];
        zero[o * so + (int64_t)(c + ch) * sr + G] = lo2[ch];
      }
    }
  }
}

// ---------------------------------------------------------------- 1-bit normal-quantile quantiser
// quant/pack_unpack.py:218-253 with bit == 1: std, mean = torch.std_mean(group) (unbiased; fp32
// accumulation, results rounded to fp16), v = rnd16(rnd16(x - mean) / std), code = searchsorted([0, inf], v)
// = [v > 0].  Only the sign of v and whether it underflows to zero matter:
//   code = (u > 0) and (u > std * 2^-25),  u = rnd16(x - mean)
// (u / std rounds to a positive fp16 exactly when it exceeds half the smallest denormal; std == 0 gives
// +inf -> 1, std == inf gives 0).  A NaN -- 0/0 of a constant group -- becomes code 0.
// The statistics follow torch's GPU reduction of a 32-element row operation for operation (ATen's WelfordOps,
// native/SharedReduceOps.h, driven by native/cuda/Reduce.cuh: one element per thread, then a tree over ADJACENT
// partners -- shuffle distances 1, 2, 4, 8, 16 -- each step merging two equal halves in fp32):
//   delta = mean_b - mean_a;  mean = mean_a + delta * 0.5;  M2 = (M2_a + M2_b) + ((delta * delta) * n_half) * 0.5
// with a the lower-indexed half; then std = sqrt(M2 / 31), both results rounded to fp16.  Compared bit for bit
// with torch.std_mean executed on the device by the GPU tests.
// rows: 4 lanes per 32-element group, 8 contiguous fp16 per lane (same decomposition as quant_rows_kernel)
__global__ __launch_bounds__(256) void normal1_rows_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xr, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ stdv, half_t *__restrict__ meanv, int64_t so, int64_t sr,
    uint32_t groups_per_row, int gpr_shift, uint32_t groups_per_slab, uint32_t blocks_per_slab) {
  const uint32_t o = blockIdx.x / blocks_per_slab;
  const uint32_t blk = blockIdx.x - o * blocks_per_slab;
  const uint32_t gin = blk * 64u + (threadIdx.x >> 2);
  const uint32_t sub = threadIdx.x & 3;
  if (gin >= groups_per_slab) return;  // the four lanes of a group leave together
  uint32_t r, g;
  if (gpr_shift >= 0) {
    r = gin >> gpr_shift;
    g = gin & (groups_per_row - 1u);
  } else {
    r = gin / groups_per_row;
    g = gin - r * groups_per_row;
  }
  const uint4 raw = *reinterpret_cast<const uint4 *>(x + (int64_t)o * xo + (int64_t)r * xr + g * 32u + sub * 8u);
  half_t v[8];
  __builtin_memcpy(v, &raw, 16);
  float xf[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) xf[i] = (float)v[i];
  Welford w = welford_tree<8>(xf);
  // the group's four lanes: the lane with the lower elements is the left partner of each merge
  {
    const Welford o = Welford{quad_xor_f<1>(w.mean), quad_xor_f<1>(w.m2)};
    w = (sub & 1) ? welford_merge(o, w, 8.f) : welford_merge(w, o, 8.f);
  }
  {
    const Welford o = Welford{quad_xor_f<2>(w.mean), quad_xor_f<2>(w.m2)};
    w = (sub & 2) ? welford_merge(o, w, 16.f) : welford_merge(w, o, 16.f);
  }
  const Normal1Stats st = normal1_finish(w);
  uint32_t b8 = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) b8 |= normal1_code((half_t)((float)v[i] - (float)st.mean_h), st.thr) << i;
  const uint32_t b16 = b8 | (quad_xor_u<1>(b8) << 8);
  const uint32_t other = quad_xor_u<2>(b16);
  if (sub == 0) {
    code[(int64_t)o * co + (int64_t)r * cr + g] = b16 | (other << 16);
    stdv[(int64_t)o * so + (int64_t)r * sr + g] = st.std_h;
    meanv[(int64_t)o * so + (int64_t)r * sr + g] = st.mean_h;
  }
}

// K handed over token-major: same decomposition as quant_k_tokenmajor_kernel (a lane owns two channels of
// one 32-token group)
__global__ __launch_bounds__(512) void normal1_k_tokenmajor_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xt, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ stdv, half_t *__restrict__ meanv, int64_t so, int64_t sr,
    uint32_t D, uint32_t n_groups) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t cp = lane & 7u, tg = lane >> 3;
  const uint32_t G0 = blockIdx.x * QK_GROUPS_PER_BLOCK;
  const uint32_t G = G0 + tg;
  const int64_t o = blockIdx.y;
  const uint32_t row_b = (uint32_t)xt * 2u;
  const uint32_t groups_here = min((uint32_t)QK_GROUPS_PER_BLOCK, n_groups - G0);
  const rsrc_t rx = make_rsrc(x + o * xo + (int64_t)G0 * 32 * xt, (groups_here * 32u - 1u) * row_b + D * 2u);
  for (uint32_t c0 = wv * 16u; c0 < D; c0 += 128u) {
    const uint32_t c = c0 + cp * 2u;
    const bool live = (G < n_groups) && (c < D);
    const uint32_t voff = live ? tg * 32u * row_b + c * 2u : 0u;
    half2_t t[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) t[k] = bits_h2(buf_u32(rx, voff, (uint32_t)k * row_b));
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      float xf[32];
#pragma unroll
      for (int k = 0; k < 32; ++k) xf[k] = (float)t[k][ch];
      const Normal1Stats st = normal1_finish(welford_tree<32>(xf));
      uint32_t w = 0;
#pragma unroll
      for (int k = 0; k < 32; ++k) w |= normal1_code((half_t)((float)t[k][ch] - (float)st.mean_h), st.thr) << k;
      if (live) {
        code[o * co + (int64_t)(c + ch) * cr + G] = w;
        stdv[o * so + (int64_t)(c + ch) * sr + G] = st.std_h;
        meanv[o * so + (int64_t)(c + ch) * sr + G] = st.mean_h;
      }
    }
  }
}

// ---------------------------------------------------------------- exhaustive check of the division
// Every pair of fp16 bit patterns (u, s): v' = rnd16(f32(u) * group_recip(f32(s))) against the correctly
// rounded v = rnd16(f32(u) / f32(s)), and the 8-bit codes rne(clamp(., 0, 255)) of both (the 4- and 2-bit
// codes are min(code8, qmax)).  The two quotients can differ only where v is an fp16 denormal: there the
// fp16 grid is coarse enough for u/s to fall exactly on a midpoint, and the product's last-place error
// decides the tie -- some 30000 times below the 0.5 at which a code changes.
// counts[0]: code mismatches over all 2^32 pairs; counts[1]: code mismatches with both sign bits clear
// (the quantiser's domain: u = x - min >= 0, s = range / qmax >= 0, or NaN); counts[2]: pairs with
// v' != v (two NaNs count as equal); counts[3]: the largest |v| (as fp16 bits) among those.
__device__ __forceinline__ int code8_of(half_t v) {
  const float c = __builtin_fminf(__builtin_fmaxf((float)v, 0.0f), 255.0f);
  return (int)__builtin_rintf(c);
}

__global__ __launch_bounds__(256) void selftest_division_kernel(unsigned long long *counts) {
  const uint32_t sbits = blockIdx.x;  // 65536 blocks: one scale pattern each
  half_t s;
  {
    const unsigned short b = (unsigned short)sbits;
    __builtin_memcpy(&s, &b, 2);
  }
  const float sf = (float)s;
  const float rcp = group_recip(sf);
  unsigned long long bad_all = 0, bad_dom = 0, bad_v = 0, max_v = 0;
  for (uint32_t ub = threadIdx.x; ub < 65536u; ub += 256u) {
    half_t u;
    const unsigned short b = (unsigned short)ub;
    __builtin_memcpy(&u, &b, 2);
    const float uf = (float)u;
    const half_t fast = (half_t)(uf * rcp);
    const half_t ref = (half_t)(uf / sf);
    unsigned short fb, rb;
    __builtin_memcpy(&fb, &fast, 2);
    __builtin_memcpy(&rb, &ref, 2);
    const bool both_nan = (fast != fast) && (ref != ref);
    if (fb != rb && !both_nan) {
      ++bad_v;
      const unsigned long long mag = rb & 0x7fffu;
      max_v = mag > max_v ? mag : max_v;
    }
    if (code8_of(fast) != code8_of(ref)) {
      ++bad_all;
      if (((ub | sbits) & 0x8000u) == 0) ++bad_dom;
    }
  }
  if (bad_all) atomicAdd(&counts[0], bad_all);
  if (bad_dom) atomicAdd(&counts[1], bad_dom);
  if (bad_v) {
    atomicAdd(&counts[2], bad_v);
    atomicMax(&counts[3], max_v);
  }
}

// ---------------------------------------------------------------- unpack (+ dequantise)
// One packed word per thread.  out = rnd16(rnd16(c * scale) + zero) (quant/pack_unpack.py:331-332).
// NORMAL (1 bit): out = rnd16(rnd16(+-k * std) + mean), k = fp16(0.6745) (quant/pack_unpack.py:371-375).
template <int BITS, bool DEQUANT, bool NORMAL = false>
__global__ __launch_bounds__(256) void dequant_rows_kernel(
    const uint32_t *__restrict__ code, int64_t co, int64_t cr, const half_t *__restrict__ scale,
    const half_t *__restrict__ zero, int64_t so, int64_t sr, half_t *__restrict__ out, int64_t oo,
    int64_t orow, int64_t n_rows, int64_t words_per_row, int64_t n_words) {
  constexpr int PF = 32 / BITS;
  const int64_t wid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (wid >= n_words) return;
  const int64_t j = wid % words_per_row;
  const int64_t rr = wid / words_per_row;
  const int64_t r = rr % n_rows;
  const int64_t o = rr / n_rows;
  const uint32_t w = code[o * co + r * cr + j];
  half_t s = (half_t)1.0f, z = (half_t)0.0f;
  if (DEQUANT) {
    const int64_t g = (j * PF) / 32;
    s = scale[o * so + r * sr + g];
    z = zero[o * so + r * sr + g];
  }
  // Both steps as fp16 operations (each a single rounding of the exact result).  Written through fp32 the
  // compiler turns the product into a mixed-precision fma with a +0 addend, which loses the sign of a -0
  // product (code 0 times a negative or -0 scale; the -0.6745 centre times a std of +0).
  half_t vals[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const uint32_t ci = code_at<BITS>(w, i);
    if (NORMAL) {
      const half_t m = (ci != 0u ? (half_t)0.67431640625f : (half_t)-0.67431640625f) * s;
      vals[i] = m + z;
    } else if (DEQUANT) {
      const half_t m = (half_t)(float)ci * s;  // first rounding (the code itself is exact in fp16)
      vals[i] = m + z;                         // second rounding
    } else {
      vals[i] = (half_t)(float)ci;
    }
  }
  half_t *po = out + o * oo + r * orow + j * PF;
  constexpr int NV = PF * 2 / 8;  // 8-byte stores
  uint2 tmp[NV];
  __builtin_memcpy(tmp, vals, PF * 2);
#pragma unroll
  for (int k = 0; k < NV; ++k) reinterpret_cast<uint2 *>(po)[k] = tmp[k];
}

// ---------------------------------------------------------------- plain pack of int32 codes
template <int BITS>
__global__ __launch_bounds__(256) void pack_i32_kernel(const int32_t *__restrict__ q,
                                                       uint32_t *__restrict__ code, int64_t n_words) {
  constexpr int PF = 32 / BITS;
  const int64_t wid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (wid >= n_words) return;
  const int32_t *src = q + wid * PF;
  uint32_t w = 0;
#pragma unroll
  for (int i = 0; i < PF; ++i) w |= (uint32_t)src[i] << (i * BITS);  // no masking, like the reference
  code[wid] = w;
}

static inline bool bits_ok(int bits) { return bits == 1 || bits == 2 || bits == 4 || bits == 8; }

}  // namespace hq

using namespace hq;

extern "C" int hqekv_quant_pack_rows(const void *x, int64_t xo, int64_t xr, void *code, int64_t co,
                                     int64_t cr, void *scale, void *zero, int64_t so, int64_t sr,
                                     int64_t n_outer, int64_t n_rows, int64_t L, int bits,
                                     void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "quant_pack_rows: bits must be 1, 2, 4 or 8 (got %d)", bits);
  if (n_outer < 0 || n_rows < 0 || L < 0 || L % 32 != 0)
    return fail(HQEKV_E_ARG, "quant_pack_rows: L=%lld must be a non-negative multiple of 32", (long long)L);
  const int64_t n_groups = n_outer * n_rows * (L / 32);
  if (n_groups == 0) return HQEKV_OK;
  if (!x || !code || !scale || !zero) return fail(HQEKV_E_ARG, "quant_pack_rows: null pointer");
  if (((uintptr_t)x & 15) || (xo % 8) || (xr % 8))
    return fail(HQEKV_E_ALIGN, "quant_pack_rows: x rows must be 16-byte aligned");
  const int64_t gpr = L / 32, gps = n_rows * gpr;
  const int64_t bps = (gps + 63) / 64;
  if (gps > 0x7fffffffLL || bps * n_outer > 0x7fffffffLL)
    return fail(HQEKV_E_ARG, "quant_pack_rows: too many groups");
  int shift = -1;
  if ((gpr & (gpr - 1)) == 0) for (shift = 0; (1LL << shift) < gpr; ++shift) {}
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)(bps * n_outer)), block(256);
#define LAUNCH(B_)                                                                              \
  hipLaunchKernelGGL(quant_rows_kernel<B_>, grid, block, 0, st, (const half_t *)x, xo, xr,     \
                     (uint32_t *)code, co, cr, (half_t *)scale, (half_t *)zero, so, sr,         \
                     (uint32_t)gpr, shift, (uint32_t)gps, (uint32_t)bps)
  if (bits == 1) LAUNCH(1); else if (bits == 2) LAUNCH(2); else if (bits == 4) LAUNCH(4); else LAUNCH(8);
#undef LAUNCH
  return check_launch("quant_rows_kernel");
}

extern "C" int hqekv_quant_pack_k_tokenmajor(const void *x, int64_t xo, int64_t xt, void *code,
                                             int64_t co, int64_t cr, void *scale, void *zero,
                                             int64_t so, int64_t sr, int64_t n_outer, int64_t T,
                                             int64_t D, int bits, void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: bits must be 1, 2, 4 or 8 (got %d)", bits);
  if (n_outer < 0 || T < 0 || T % 32 != 0 || D <= 0 || D % 2 != 0)
    return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: need T %% 32 == 0 and even D (T=%lld D=%lld)",
                (long long)T, (long long)D);
  if (n_outer == 0 || T == 0) return HQEKV_OK;
  if (!x || !code || !scale || !zero) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: null pointer");
  if (((uintptr_t)x & 3) || (xo % 2) || (xt % 2))
    return fail(HQEKV_E_ALIGN, "quant_pack_k_tokenmajor: x rows must be 4-byte aligned");
  if (n_outer > 65535) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: n_outer > 65535");
  // 32-bit byte offsets inside one block of 256 token rows
  if (xt < D || xt > (1LL << 22) || D > (1LL << 22) || T / 32 > 0x7fffffffLL)
    return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: need D <= xt <= 2^22 (xt=%lld D=%lld)", (long long)xt, (long long)D);
  const int64_t n_groups = T / 32;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((n_groups + QK_GROUPS_PER_BLOCK - 1) / QK_GROUPS_PER_BLOCK), (unsigned)n_outer), block(512);
#define LAUNCH(B_)                                                                                  \
  hipLaunchKernelGGL(quant_k_tokenmajor_kernel<B_>, grid, block, 0, st, (const half_t *)x, xo, xt, \
                     (uint32_t *)code, co, cr, (half_t *)scale, (half_t *)zero, so, sr,             \
                     (uint32_t)D, (uint32_t)n_groups)
  if (bits == 1) LAUNCH(1); else if (bits == 2) LAUNCH(2); else if (bits == 4) LAUNCH(4); else LAUNCH(8);
#undef LAUNCH
  return check_launch("quant_k_tokenmajor_kernel");
}

extern "C" int hqekv_normal1_quant_pack_rows(const void *x, int64_t xo, int64_t xr, void *code, int64_t co,
                                             int64_t cr, void *stdv, void *meanv, int64_t so, int64_t sr,
                                             int64_t n_outer, int64_t n_rows, int64_t L, void *stream) {
  if (n_outer < 0 || n_rows < 0 || L < 0 || L % 32 != 0)
    return fail(HQEKV_E_ARG, "normal1_quant_pack_rows: L=%lld must be a non-negative multiple of 32", (long long)L);
  const int64_t n_groups = n_outer * n_rows * (L / 32);
  if (n_groups == 0) return HQEKV_OK;
  if (!x || !code || !stdv || !meanv) return fail(HQEKV_E_ARG, "normal1_quant_pack_rows: null pointer");
  if (((uintptr_t)x & 15) || (xo % 8) || (xr % 8))
    return fail(HQEKV_E_ALIGN, "normal1_quant_pack_rows: x rows must be 16-byte aligned");
  const int64_t gpr = L / 32, gps = n_rows * gpr;
  const int64_t bps = (gps + 63) / 64;
  if (gps > 0x7fffffffLL || bps * n_outer > 0x7fffffffLL)
    return fail(HQEKV_E_ARG, "normal1_quant_pack_rows: too many groups");
  int shift = -1;
  if ((gpr & (gpr - 1)) == 0) for (shift = 0; (1LL << shift) < gpr; ++shift) {}
  hipLaunchKernelGGL(normal1_rows_kernel, dim3((unsigned)(bps * n_outer)), dim3(256), 0, (hipStream_t)stream,
                     (const half_t *)x, xo, xr, (uint32_t *)code, co, cr, (half_t *)stdv, (half_t *)meanv, so, sr,
                     (uint32_t)gpr, shift, (uint32_t)gps, (uint32_t)bps);
  return check_launch("normal1_rows_kernel");
}

extern "C" int hqekv_normal1_quant_pack_k_tokenmajor(const void *x, int64_t xo, int64_t xt, void *code,
                                                     int64_t co, int64_t cr, void *stdv, void *meanv,
                                                     int64_t so, int64_t sr, int64_t n_outer, int64_t T,
                                                     int64_t D, void *stream) {
  if (n_outer < 0 || T < 0 || T % 32 != 0 || D <= 0 || D % 2 != 0)
    return fail(HQEKV_E_ARG, "normal1_quant_pack_k_tokenmajor: need T %% 32 == 0 and even D (T=%lld D=%lld)",
                (long long)T, (long long)D);
  if (n_outer == 0 || T == 0) return HQEKV_OK;
  if (!x || !code || !stdv || !meanv) return fail(HQEKV_E_ARG, "normal1_quant_pack_k_tokenmajor: null pointer");
  if (((uintptr_t)x & 3) || (xo % 2) || (xt % 2))
    return fail(HQEKV_E_ALIGN, "normal1_quant_pack_k_tokenmajor: x rows must be 4-byte aligned");
  if (n_outer > 65535) return fail(HQEKV_E_ARG, "normal1_quant_pack_k_tokenmajor: n_outer > 65535");
  if (xt < D || xt > (1LL << 22) || D > (1LL << 22) || T / 32 > 0x7fffffffLL)
    return fail(HQEKV_E_ARG, "normal1_quant_pack_k_tokenmajor: need D <= xt <= 2^22 (xt=%lld D=%lld)", (long long)xt, (long long)D);
  const int64_t n_groups = T / 32;
  dim3 grid((unsigned)((n_groups + QK_GROUPS_PER_BLOCK - 1) / QK_GROUPS_PER_BLOCK), (unsigned)n_outer);
  hipLaunchKernelGGL(normal1_k_tokenmajor_kernel, grid, dim3(512), 0, (hipStream_t)stream, (const half_t *)x, xo, xt,
                     (uint32_t *)code, co, cr, (half_t *)stdv, (half_t *)meanv, so, sr, (uint32_t)D, (uint32_t)n_groups);
  return check_launch("normal1_k_tokenmajor_kernel");
}

extern "C" int hqekv_normal1_dequant_unpack_rows(const void *code, int64_t co, int64_t cr, const void *stdv,
                                                 const void *meanv, int64_t so, int64_t sr, void *out,
                                                 int64_t oo, int64_t orow, int64_t n_outer, int64_t n_rows,
                                                 int64_t L, void *stream) {
  if (n_outer < 0 || n_rows < 0 || L < 0 || L % 32 != 0)
    return fail(HQEKV_E_ARG, "normal1_dequant_unpack_rows: bad L=%lld", (long long)L);
  const int64_t n_words = n_outer * n_rows * (L / 32);
  if (n_words == 0) return HQEKV_OK;
  if (!code || !out || !stdv || !meanv) return fail(HQEKV_E_ARG, "normal1_dequant_unpack_rows: null pointer");
  if (((uintptr_t)out & 7) || (oo % 4) || (orow % 4))
    return fail(HQEKV_E_ALIGN, "normal1_dequant_unpack_rows: out rows must be 8-byte aligned");
  const int64_t blocks = (n_words + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_ARG, "normal1_dequant_unpack_rows: too many words");
  hipLaunchKernelGGL((dequant_rows_kernel<1, true, true>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t *)code, co, cr, (const half_t *)stdv, (const half_t *)meanv, so, sr,
                     (half_t *)out, oo, orow, n_rows, L / 32, n_words);
  return check_launch("dequant_rows_kernel");
}

// Every wave reduces its 64 inputs with the DPP / lane-row-swap reductions the attention kernels use and
// with the plain shuffle butterfly; out holds (sum, max, butterfly sum, butterfly max) per wave.
__global__ __launch_bounds__(256) void selftest_wave_reduce_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                                   int n_waves) {
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (w >= n_waves) return;  // whole waves leave together
  const float v = in[(int64_t)w * 64 + lane];
  const float s = wave_sum(v), m = wave_max(v);
  float bs = v, bm = v;
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1) {
    bs += xor_f(bs, k);
    bm = fmaxf(bm, xor_f(bm, k));
  }
  if (lane == 0) {
    out[w * 4 + 0] = s;
    out[w * 4 + 1] = m;
    out[w * 4 + 2] = bs;
    out[w * 4 + 3] = bm;
  }
}

extern "C" int hqekv_selftest_wave_reduce(const void *in, void *out, int64_t n_waves, void *stream) {
  if (n_waves < 0 || n_waves > 0x7fffffffLL) return fail(HQEKV_E_ARG, "selftest_wave_reduce: bad n_waves");
  if (n_waves == 0) return HQEKV_OK;
  if (!in || !out) return fail(HQEKV_E_ARG, "selftest_wave_reduce: null pointer");
  hipLaunchKernelGGL(selftest_wave_reduce_kernel, dim3((unsigned)((n_waves + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     (const float *)in, (float *)out, (int)n_waves);
  return check_launch("selftest_wave_reduce_kernel");
}

// Yardstick: a launch that does nothing but read `bytes` bytes, as wide and as deep as the hardware likes them
// (16 bytes per lane, eight requests in flight per lane, every CU busy).  What this takes, launch included, is the
// floor for any kernel that has to read the same bytes once.  `sum` receives one word per workgroup (so that the
// loads cannot be dropped).
namespace hq {
constexpr int SR_THREADS = 256, SR_UNROLL = 8;
__global__ __launch_bounds__(SR_THREADS) void stream_read_kernel(const uint4 *__restrict__ p, int64_t n16, uint32_t *__restrict__ sum) {
  uint32_t acc = 0;
  const int64_t stride = (int64_t)gridDim.x * SR_THREADS * SR_UNROLL;
  for (int64_t i = (int64_t)blockIdx.x * SR_THREADS * SR_UNROLL + threadIdx.x; i < n16; i += stride) {
    uint4 v[SR_UNROLL];
#pragma unroll
    for (int k = 0; k < SR_UNROLL; ++k) {
      const int64_t j = i + (int64_t)k * SR_THREADS;
      v[k] = j < n16 ? p[j] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int k = 0; k < SR_UNROLL; ++k) acc ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
  }
  for (int o = 32; o; o >>= 1) acc ^= (uint32_t)__shfl_xor((int)acc, o, HQ_WAVE);
  if ((threadIdx.x & 63) == 0) atomicXor(sum + blockIdx.x, acc);
}
}  // namespace hq

extern "C" int hqekv_selftest_stream_read(const void *src, int64_t bytes, void *sum, int64_t n_workgroups, void *stream) {
  if (!src || !sum || bytes < 0 || n_workgroups <= 0 || n_workgroups > 65535)
    return fail(HQEKV_E_ARG, "selftest_stream_read: null pointer, negative size or 0 / more than 65535 workgroups");
  if (((uintptr_t)src & 15) || (bytes & 15)) return fail(HQEKV_E_ALIGN, "selftest_stream_read: 16-byte granularity");
  if (bytes == 0) return HQEKV_OK;
  hipLaunchKernelGGL(hq::stream_read_kernel, dim3((unsigned)n_workgroups), dim3(hq::SR_THREADS), 0, (hipStream_t)stream,
                     (const uint4 *)src, bytes / 16, (uint32_t *)sum);
  return check_launch("stream_read_kernel");
}

extern "C" int hqekv_selftest_quant_division(void *counts, void *stream) {
  if (!counts) return fail(HQEKV_E_ARG, "selftest_quant_division: null pointer");
  if ((uintptr_t)counts & 7) return fail(HQEKV_E_ALIGN, "selftest_quant_division: counts must be 8-byte aligned");
  hipLaunchKernelGGL(selftest_division_kernel, dim3(65536), dim3(256), 0, (hipStream_t)stream,
                     (unsigned long long *)counts);
  return check_launch("selftest_division_kernel");
}

extern "C" int hqekv_dequant_unpack_rows(const void *code, int64_t co, int64_t cr, const void *scale,
                                         const void *zero, int64_t so, int64_t sr, void *out,
                                         int64_t oo, int64_t orow, int64_t n_outer, int64_t n_rows,
                                         int64_t L, int bits, void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "dequant_unpack_rows: bits must be 1, 2, 4 or 8 (got %d)", bits);
  const int pf = 32 / bits;
  if (n_outer < 0 || n_rows < 0 || L < 0 || L % pf != 0 || (scale && L % 32 != 0))
    return fail(HQEKV_E_ARG, "dequant_unpack_rows: bad L=%lld", (long long)L);
  const int64_t n_words = n_outer * n_rows * (L / pf);
  if (n_words == 0) return HQEKV_OK;
  if (!code || !out || (scale && !zero)) return fail(HQEKV_E_ARG, "dequant_unpack_rows: null pointer");
  if (((uintptr_t)out & 7) || (oo % 4) || (orow % 4))
    return fail(HQEKV_E_ALIGN, "dequant_unpack_rows: out rows must be 8-byte aligned");
  const int64_t blocks = (n_words + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_ARG, "dequant_unpack_rows: too many words");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(256);
#define LAUNCH(B_, DQ_)                                                                          \
  hipLaunchKernelGGL((dequant_rows_kernel<B_, DQ_>), grid, block, 0, st, (const uint32_t *)code, \
                     co, cr, (const half_t *)scale, (const half_t *)zero, so, sr, (half_t *)out, \
                     oo, orow, n_rows, L / pf, n_words)
  if (scale) {
    if (bits == 1) LAUNCH(1, true); else if (bits == 2) LAUNCH(2, true); else if (bits == 4) LAUNCH(4, true); else LAUNCH(8, true);
  } else {
    if (bits == 1) LAUNCH(1, false); else if (bits == 2) LAUNCH(2, false); else if (bits == 4) LAUNCH(4, false); else LAUNCH(8, false);
  }
#undef LAUNCH
  return check_launch("dequant_rows_kernel");
}

extern "C" int hqekv_pack_i32(const void *q, void *code, int64_t n_rows, int64_t L, int bits,
                              void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "pack_i32: bits must be 1, 2, 4 or 8 (got %d)", bits);
  const int pf = 32 / bits;
  if (n_rows < 0 || L < 0 || L % pf != 0) return fail(HQEKV_E_ARG, "pack_i32: L %% pf != 0");
  const int64_t n_words = n_rows * (L / pf);
  if (n_words == 0) return HQEKV_OK;
  if (!q || !code) return fail(HQEKV_E_ARG, "pack_i32: null pointer");
  const int64_t blocks = (n_words + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_ARG, "pack_i32: too many words");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(256);
  if (bits == 1) hipLaunchKernelGGL(pack_i32_kernel<1>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  else if (bits == 2) hipLaunchKernelGGL(pack_i32_kernel<2>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  else if (bits == 4) hipLaunchKernelGGL(pack_i32_kernel<4>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  else hipLaunchKernelGGL(pack_i32_kernel<8>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  return check_launch("pack_i32_kernel");
}
