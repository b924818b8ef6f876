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

namespace hq {

template <int BITS>
__device__ __forceinline__ uint32_t quant_one(half_t x, float mn, float scale_f) {
  constexpr float QMAX = (float)((1 << BITS) - 1);
  const float u = (float)(half_t)((float)x - mn);
  float v = (float)(half_t)(u / scale_f);
  // fmaxf/fminf drop a NaN operand: NaN -> 0, which is what the float->int conversion of the
  // reference path yields for a constant group.
  v = fminf(fmaxf(v, 0.0f), QMAX);
  return (uint32_t)(int)__builtin_rintf(v);
}

// ---------------------------------------------------------------- rows: groups along a contiguous axis
// 4 lanes per 32-element group, 8 contiguous fp16 (one 128-bit load) per lane.
template <int BITS>
__global__ __launch_bounds__(256) void quant_rows_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xr, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ scale, half_t *__restrict__ zero, int64_t so, int64_t sr,
    int64_t n_rows, int64_t groups_per_row, int64_t n_groups) {
  constexpr int PF = 32 / BITS;
  constexpr float INV_QMAX = 1.0f / (float)((1 << BITS) - 1);
  const int64_t gid = (int64_t)blockIdx.x * 64 + (threadIdx.x >> 2);
  const int sub = threadIdx.x & 3;
  if (gid >= n_groups) return;  // the four lanes of a group leave together
  const int64_t g = gid % groups_per_row;
  const int64_t rr = gid / groups_per_row;
  const int64_t r = rr % n_rows;
  const int64_t o = rr / n_rows;

  const uint4 raw = *reinterpret_cast<const uint4 *>(x + o * xo + r * xr + g * 32 + sub * 8);
  half_t v[8];
  __builtin_memcpy(v, &raw, 16);

  float mn = (float)v[0], mx = (float)v[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    mn = fminf(mn, (float)v[i]);
    mx = fmaxf(mx, (float)v[i]);
  }
  mn = fminf(mn, xor_f(mn, 1));
  mx = fmaxf(mx, xor_f(mx, 1));
  mn = fminf(mn, xor_f(mn, 2));
  mx = fmaxf(mx, xor_f(mx, 2));

  const half_t d = (half_t)(mx - mn);
  const half_t sc = (half_t)((float)d * INV_QMAX);
  const float sc_f = (float)sc;

  uint32_t c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = quant_one<BITS>(v[i], mn, sc_f);

  uint32_t *crow = code + o * co + r * cr + g * (32 / PF);
  if (BITS == 2) {
    uint32_t h = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) h |= c[i] << (2 * i);
    const uint32_t other = xor_u(h, 1);
    if ((sub & 1) == 0) crow[sub >> 1] = h | (other << 16);
  } else if (BITS == 4) {
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) w |= c[i] << (4 * i);
    crow[sub] = w;
  } else {
    crow[sub * 2 + 0] = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
    crow[sub * 2 + 1] = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
  }
  if (sub == 0) {
    scale[o * so + r * sr + g] = sc;
    zero[o * so + r * sr + g] = (half_t)mn;
  }
}

// ---------------------------------------------------------------- K handed over token-major
// One wavefront per (32-token group, outer slab); a lane owns two adjacent channels and keeps the
// 32 x 2 fp16 tile in registers, so a token row (D fp16) is read as one coalesced 4-byte-per-lane load.
template <int BITS>
__global__ __launch_bounds__(64) void quant_k_tokenmajor_kernel(
    const half_t *__restrict__ x, int64_t xo, int64_t xt, uint32_t *__restrict__ code, int64_t co,
    int64_t cr, half_t *__restrict__ scale, half_t *__restrict__ zero, int64_t so, int64_t sr,
    int64_t D) {
  constexpr int PF = 32 / BITS;
  constexpr int WPG = 32 / PF;  // words per group
  constexpr float INV_QMAX = 1.0f / (float)((1 << BITS) - 1);
  const int64_t g = blockIdx.x;
  const int64_t o = blockIdx.y;
  const half_t *xb = x + o * xo + g * 32 * xt;
  for (int64_t cp = threadIdx.x; cp * 2 < D; cp += 64) {
    half2_t t[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) t[k] = *reinterpret_cast<const half2_t *>(xb + k * xt + cp * 2);
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      float mn = (float)t[0][ch], mx = (float)t[0][ch];
#pragma unroll
      for (int k = 1; k < 32; ++k) {
        mn = fminf(mn, (float)t[k][ch]);
        mx = fmaxf(mx, (float)t[k][ch]);
      }
      const half_t d = (half_t)(mx - mn);
      const half_t sc = (half_t)((float)d * INV_QMAX);
      const float sc_f = (float)sc;
      const int64_t c_idx = cp * 2 + ch;
      uint32_t *crow = code + o * co + c_idx * cr + g * WPG;
#pragma unroll
      for (int wj = 0; wj < WPG; ++wj) {
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < PF; ++i) w |= quant_one<BITS>(t[wj * PF + i][ch], mn, sc_f) << (i * BITS);
        crow[wj] = w;
      }
      scale[o * so + c_idx * sr + g] = sc;
      zero[o * so + c_idx * sr + g] = (half_t)mn;
    }
  }
}

// ---------------------------------------------------------------- unpack (+ dequantise)
// One packed word per thread.  out = rnd16(rnd16(c * scale) + zero) (quant/pack_unpack.py:331-332).
template <int BITS, bool DEQUANT>
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
  float s = 1.0f, z = 0.0f;
  if (DEQUANT) {
    const int64_t g = (j * PF) / 32;
    s = (float)scale[o * so + r * sr + g];
    z = (float)zero[o * so + r * sr + g];
  }
  half_t vals[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const float c = (float)code_at<BITS>(w, i);
    if (DEQUANT) {
      const half_t m = (half_t)(c * s);  // exact product, one rounding
      vals[i] = (half_t)((float)m + z);  // second rounding
    } else {
      vals[i] = (half_t)c;
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

static inline bool bits_ok(int bits) { return bits == 2 || bits == 4 || bits == 8; }

}  // namespace hq

using namespace hq;

extern "C" int hqekv_quant_pack_rows(const void *x, int64_t xo, int64_t xr, void *code, int64_t co,
                                     int64_t cr, void *scale, void *zero, int64_t so, int64_t sr,
                                     int64_t n_outer, int64_t n_rows, int64_t L, int bits,
                                     void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "quant_pack_rows: bits must be 2, 4 or 8 (got %d)", bits);
  if (n_outer < 0 || n_rows < 0 || L < 0 || L % 32 != 0)
    return fail(HQEKV_E_ARG, "quant_pack_rows: L=%lld must be a non-negative multiple of 32", (long long)L);
  const int64_t n_groups = n_outer * n_rows * (L / 32);
  if (n_groups == 0) return HQEKV_OK;
  if (!x || !code || !scale || !zero) return fail(HQEKV_E_ARG, "quant_pack_rows: null pointer");
  if (((uintptr_t)x & 15) || (xo % 8) || (xr % 8))
    return fail(HQEKV_E_ALIGN, "quant_pack_rows: x rows must be 16-byte aligned");
  const int64_t blocks = (n_groups + 63) / 64;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_ARG, "quant_pack_rows: too many groups");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(256);
#define LAUNCH(B_)                                                                              \
  hipLaunchKernelGGL(quant_rows_kernel<B_>, grid, block, 0, st, (const half_t *)x, xo, xr,     \
                     (uint32_t *)code, co, cr, (half_t *)scale, (half_t *)zero, so, sr, n_rows, \
                     L / 32, n_groups)
  if (bits == 2) LAUNCH(2); else if (bits == 4) LAUNCH(4); else LAUNCH(8);
#undef LAUNCH
  return check_launch("quant_rows_kernel");
}

extern "C" int hqekv_quant_pack_k_tokenmajor(const void *x, int64_t xo, int64_t xt, void *code,
                                             int64_t co, int64_t cr, void *scale, void *zero,
                                             int64_t so, int64_t sr, int64_t n_outer, int64_t T,
                                             int64_t D, int bits, void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: bits must be 2, 4 or 8 (got %d)", bits);
  if (n_outer < 0 || T < 0 || T % 32 != 0 || D <= 0 || D % 2 != 0)
    return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: need T %% 32 == 0 and even D (T=%lld D=%lld)",
                (long long)T, (long long)D);
  if (n_outer == 0 || T == 0) return HQEKV_OK;
  if (!x || !code || !scale || !zero) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: null pointer");
  if (((uintptr_t)x & 3) || (xo % 2) || (xt % 2))
    return fail(HQEKV_E_ALIGN, "quant_pack_k_tokenmajor: x rows must be 4-byte aligned");
  if (n_outer > 65535) return fail(HQEKV_E_ARG, "quant_pack_k_tokenmajor: n_outer > 65535");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)(T / 32), (unsigned)n_outer), block(64);
#define LAUNCH(B_)                                                                                  \
  hipLaunchKernelGGL(quant_k_tokenmajor_kernel<B_>, grid, block, 0, st, (const half_t *)x, xo, xt, \
                     (uint32_t *)code, co, cr, (half_t *)scale, (half_t *)zero, so, sr, D)
  if (bits == 2) LAUNCH(2); else if (bits == 4) LAUNCH(4); else LAUNCH(8);
#undef LAUNCH
  return check_launch("quant_k_tokenmajor_kernel");
}

extern "C" int hqekv_dequant_unpack_rows(const void *code, int64_t co, int64_t cr, const void *scale,
                                         const void *zero, int64_t so, int64_t sr, void *out,
                                         int64_t oo, int64_t orow, int64_t n_outer, int64_t n_rows,
                                         int64_t L, int bits, void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "dequant_unpack_rows: bits must be 2, 4 or 8 (got %d)", bits);
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
    if (bits == 2) LAUNCH(2, true); else if (bits == 4) LAUNCH(4, true); else LAUNCH(8, true);
  } else {
    if (bits == 2) LAUNCH(2, false); else if (bits == 4) LAUNCH(4, false); else LAUNCH(8, false);
  }
#undef LAUNCH
  return check_launch("dequant_rows_kernel");
}

extern "C" int hqekv_pack_i32(const void *q, void *code, int64_t n_rows, int64_t L, int bits,
                              void *stream) {
  if (!bits_ok(bits)) return fail(HQEKV_E_ARG, "pack_i32: bits must be 2, 4 or 8 (got %d)", bits);
  const int pf = 32 / bits;
  if (n_rows < 0 || L < 0 || L % pf != 0) return fail(HQEKV_E_ARG, "pack_i32: L %% pf != 0");
  const int64_t n_words = n_rows * (L / pf);
  if (n_words == 0) return HQEKV_OK;
  if (!q || !code) return fail(HQEKV_E_ARG, "pack_i32: null pointer");
  const int64_t blocks = (n_words + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_ARG, "pack_i32: too many words");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(256);
  if (bits == 2) hipLaunchKernelGGL(pack_i32_kernel<2>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  else if (bits == 4) hipLaunchKernelGGL(pack_i32_kernel<4>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  else hipLaunchKernelGGL(pack_i32_kernel<8>, grid, block, 0, st, (const int32_t *)q, (uint32_t *)code, n_words);
  return check_launch("pack_i32_kernel");
}
