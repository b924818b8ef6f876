// Decode attention over the hybrid fp16 / 8 / 4 / 2-bit cache: fused dequantize-GEMV for q.K^T,
// scale+mask+clamp+softmax, fused dequantize-GEMV for p.V with a deterministic split-K combine.
//
// Arithmetic.  The reference defines a correct result as "dequantise with the library's own
// unpack, then matmul" (quant/cuda_hq_test.py:82,242), and its dequantiser rounds twice in fp16
// (quant/pack_unpack.py:331-332).  The kernels reproduce exactly those values in registers:
//     x = rnd16(rnd16(c * scale) + zero)           two packed-fp16 VALU ops for two codes
// and feed them to v_dot2_f32_f16 against (q_d, q_d+1) resp. (p_t, p_t+1): products are exact in
// fp32, accumulation is fp32, and the only further rounding is the final conversion to fp16.
// Codes become fp16 integers without a shift or an int->float convert: a byte permute lines up the
// same byte of two rows in the two 16-bit halves of a register, one AND-OR drops a code field into
// the mantissa of 2^(10-pos) (giving 2^(10-pos) + c exactly) and one packed subtract removes the bias.
// No MFMA and no packed-fp32 instructions are used.
//
// Layouts are consumed exactly as the cache stores them:
//   K class: code (B,Hkv,D,T/pf) -- a lane owns one packed word (pf tokens) and walks the D rows two
//            at a time, so the reduction over d needs no cross-lane traffic; 4 waves split D and meet
//            in LDS.
//   V class: code (B,Hkv,T,D/pf) -- D/pf lanes cover one token row and walk the tokens two at a time;
//            scale/zero and the gathered probabilities of a 512-token block are staged in LDS in
//            pair-interleaved order; lanes are reduced by butterflies, waves through LDS, workgroups
//            through fp32 partials summed in a fixed order.
#include "common.h"

#pragma clang fp contract(off)  // the two fp16 roundings of the dequantiser must stay separate

namespace hq {

struct SegDev {
  const void *data;
  const half_t *scale;
  const half_t *zero;
  const int64_t *idx;
  int64_t pos_base;
  int64_t n_tokens;
  int32_t bits;
  int32_t token_major;
  int32_t unit_begin;  // first tile (q.K^T) or chunk (p.V) of this segment in the launch
  int32_t pad_;
};

struct SegTable {
  SegDev seg[HQEKV_MAX_SEGS];
  int32_t nseg;
  int32_t total_units;
};

__device__ __forceinline__ int find_seg(const SegTable &tb, int unit) {
  int s = 0;
#pragma unroll
  for (int k = 1; k < HQEKV_MAX_SEGS; ++k)
    if (k < tb.nseg && unit >= tb.seg[k].unit_begin) s = k;
  return s;
}

__device__ __forceinline__ half2_t as_h2(uint32_t u) {
  half2_t h;
  __builtin_memcpy(&h, &u, 4);
  return h;
}
__device__ __forceinline__ uint32_t as_u32(half2_t h) {
  uint32_t u;
  __builtin_memcpy(&u, &h, 4);
  return u;
}
__device__ __forceinline__ half2_t pack_h2(half_t a, half_t b) {
  half2_t h;
  h[0] = a;
  h[1] = b;
  return h;
}

// [lo.byte_k, 0, hi.byte_k, 0]: byte k of two packed words side by side in the 16-bit halves
template <int K>
__device__ __forceinline__ uint32_t byte_pair(uint32_t lo, uint32_t hi) {
  return __builtin_amdgcn_perm(hi, lo, 0x0c040c00u + (uint32_t)K * 0x00010001u);
}
// (lo.half_H, hi.half_H) of two registers holding fp16 pairs
template <int H>
__device__ __forceinline__ half2_t half_pair(uint32_t lo, uint32_t hi) {
  return as_h2(__builtin_amdgcn_perm(hi, lo, H == 0 ? 0x05040100u : 0x07060302u));
}

// Field I (of 8/BITS) of the byte pair `u` as two exact fp16 integers.
template <int BITS, int I>
__device__ __forceinline__ half2_t field_pair(uint32_t u) {
  constexpr int POS = I * BITS;                         // bit position inside the byte
  constexpr uint32_t FMASK = ((1u << BITS) - 1u) << POS;
  constexpr uint32_t MASK = FMASK | (FMASK << 16);
  constexpr uint32_t EXPO = (uint32_t)(10 - POS + 15) << 10;  // fp16 bits of 2^(10-POS)
  constexpr uint32_t MAGIC = EXPO | (EXPO << 16);
  const half2_t biased = as_h2((u & MASK) | MAGIC);     // 2^(10-POS) + c, exact
  const half2_t bias = as_h2(MAGIC);
  return biased - bias;                                 // c, exact
}

// the reference dequantiser's two roundings (quant/pack_unpack.py:331-332) on a pair of codes
__device__ __forceinline__ half2_t dequant_pair(half2_t c, half2_t s2, half2_t z2) {
  const half2_t m = c * s2;
  return m + z2;
}

// Consume one byte pair: 8/BITS dequantised pairs, each dotted with NREP operand pairs.
template <int BITS, int NREP, int PF>
__device__ __forceinline__ void consume_byte(uint32_t u, half2_t s2, half2_t z2, const half2_t (&a2)[NREP],
                                             float (&acc)[NREP][PF], int tok0) {
  constexpr int FPB = 8 / BITS;
#define HQ_FIELD(I_)                                                                     \
  if constexpr (I_ < FPB) {                                                                      \
    const half2_t x2 = dequant_pair(field_pair<BITS, (I_ < FPB ? I_ : 0)>(u), s2, z2);  \
    _Pragma("unroll") for (int h = 0; h < NREP; ++h)                                     \
        acc[h][tok0 + I_] = __builtin_amdgcn_fdot2(x2, a2[h], acc[h][tok0 + I_], false); \
  }
  HQ_FIELD(0)
  HQ_FIELD(1)
  HQ_FIELD(2)
  HQ_FIELD(3)
#undef HQ_FIELD
}

template <int BITS, int NREP, int PF>
__device__ __forceinline__ void consume_words(uint32_t w0, uint32_t w1, half2_t s2, half2_t z2,
                                              const half2_t (&a2)[NREP], float (&acc)[NREP][PF]) {
  constexpr int FPB = 8 / BITS;
  consume_byte<BITS, NREP, PF>(byte_pair<0>(w0, w1), s2, z2, a2, acc, 0 * FPB);
  consume_byte<BITS, NREP, PF>(byte_pair<1>(w0, w1), s2, z2, a2, acc, 1 * FPB);
  consume_byte<BITS, NREP, PF>(byte_pair<2>(w0, w1), s2, z2, a2, acc, 2 * FPB);
  consume_byte<BITS, NREP, PF>(byte_pair<3>(w0, w1), s2, z2, a2, acc, 3 * FPB);
}

// =============================================================================== q.K^T
constexpr int QK_THREADS = 256;
constexpr int QK_WAVES = 4;

__host__ __device__ inline int64_t qk_tile_tokens(int bits, int token_major) {
  if (bits == 16) return token_major ? 64 : 128;
  return 64 * (32 / bits);
}

// cross-wave sum of PF accumulators per lane, one query head at a time (keeps LDS at 3*PF*256 B)
template <int PF>
__device__ __forceinline__ void qk_reduce_head(float (&a)[PF], float *red, int wave, int lane) {
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < PF; ++i) red[((wave - 1) * PF + i) * 64 + lane] = a[i];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < PF; ++i)
      a[i] += red[(0 * PF + i) * 64 + lane] + red[(1 * PF + i) * 64 + lane] + red[(2 * PF + i) * 64 + lane];
  }
  __syncthreads();
}

template <int NREP, int PF>
__device__ __forceinline__ void qk_store(const SegDev &sg, float (&acc)[NREP][PF], int64_t t0, int b, int hkv,
                                         int Hq, int64_t Tall, half_t *__restrict__ scores) {
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    if (t0 + i < sg.n_tokens) {
      const int64_t pos = sg.idx ? sg.idx[t0 + i] : sg.pos_base + t0 + i;
#pragma unroll
      for (int h = 0; h < NREP; ++h)
        scores[((int64_t)b * Hq + hkv * NREP + h) * Tall + pos] = (half_t)acc[h][i];
    }
  }
}

template <int BITS, int NREP>
__device__ __forceinline__ void qk_quant_tile(const SegDev &sg, int tile, int bh, int b, int hkv, int D,
                                              int Hq, int64_t Tall, const half2_t *q2s, float *red,
                                              half_t *__restrict__ scores) {
  constexpr int PF = 32 / BITS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t wpr = sg.n_tokens / PF;  // words per row
  const int64_t gpr = sg.n_tokens / 32;  // groups per row
  const int64_t jw = (int64_t)tile * 64 + lane;
  const bool valid = jw < wpr;
  const int64_t jws = valid ? jw : 0;
  const int64_t g = (jws * PF) >> 5;
  const uint32_t *code = (const uint32_t *)sg.data + (int64_t)bh * D * wpr + jws;
  const half_t *sc = sg.scale + (int64_t)bh * D * gpr + g;
  const half_t *zr = sg.zero + (int64_t)bh * D * gpr + g;
  const int DP = D >> 1;

  float acc[NREP][PF];
#pragma unroll
  for (int h = 0; h < NREP; ++h)
#pragma unroll
    for (int i = 0; i < PF; ++i) acc[h][i] = 0.f;

#pragma unroll 2
  for (int dp = wave; dp < DP; dp += QK_WAVES) {
    const int64_t d = 2 * dp;
    const uint32_t w0 = code[d * wpr];
    const uint32_t w1 = code[(d + 1) * wpr];
    const half2_t s2 = pack_h2(sc[d * gpr], sc[(d + 1) * gpr]);
    const half2_t z2 = pack_h2(zr[d * gpr], zr[(d + 1) * gpr]);
    half2_t q2[NREP];
#pragma unroll
    for (int h = 0; h < NREP; ++h) q2[h] = q2s[h * DP + dp];
    consume_words<BITS, NREP, PF>(w0, w1, s2, z2, q2, acc);
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) qk_reduce_head<PF>(acc[h], red, wave, lane);
  if (wave == 0 && valid) qk_store<NREP, PF>(sg, acc, jw * PF, b, hkv, Hq, Tall, scores);
}

// fp16 class stored channel-major (B,Hkv,D,T): a lane owns two adjacent tokens
template <int NREP>
__device__ __forceinline__ void qk_f16_cm_tile(const SegDev &sg, int tile, int bh, int b, int hkv, int D,
                                               int Hq, int64_t Tall, const half2_t *q2s, float *red,
                                               half_t *__restrict__ scores) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = sg.n_tokens;
  const int64_t t0 = ((int64_t)tile * 64 + lane) * 2;
  const bool v0 = t0 < n, v1 = t0 + 1 < n;
  const half_t *kp = (const half_t *)sg.data + (int64_t)bh * D * n + (v0 ? t0 : 0);
  const bool pair = (n & 1) == 0;  // rows stay 4-byte aligned
  const int DP = D >> 1;
  float acc[NREP][2];
#pragma unroll
  for (int h = 0; h < NREP; ++h) acc[h][0] = acc[h][1] = 0.f;
#pragma unroll 2
  for (int dp = wave; dp < DP; dp += QK_WAVES) {
    const int64_t d = 2 * dp;
    uint32_t r0, r1;  // (k[d][t0], k[d][t0+1]) and the same for row d+1
    if (pair) {
      r0 = *reinterpret_cast<const uint32_t *>(kp + d * n);
      r1 = *reinterpret_cast<const uint32_t *>(kp + (d + 1) * n);
    } else {
      r0 = as_u32(pack_h2(kp[d * n], v1 ? kp[d * n + 1] : (half_t)0));
      r1 = as_u32(pack_h2(kp[(d + 1) * n], v1 ? kp[(d + 1) * n + 1] : (half_t)0));
    }
    const half2_t ka = half_pair<0>(r0, r1);  // token t0:   (k[d], k[d+1])
    const half2_t kb = half_pair<1>(r0, r1);  // token t0+1
#pragma unroll
    for (int h = 0; h < NREP; ++h) {
      const half2_t q2 = q2s[h * DP + dp];
      acc[h][0] = __builtin_amdgcn_fdot2(ka, q2, acc[h][0], false);
      acc[h][1] = __builtin_amdgcn_fdot2(kb, q2, acc[h][1], false);
    }
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) qk_reduce_head<2>(acc[h], red, wave, lane);
  if (wave == 0 && v0) qk_store<NREP, 2>(sg, acc, t0, b, hkv, Hq, Tall, scores);
}

// fp16 residual stored token-major (B,Hkv,T,D): a wave walks tokens, lanes split the channels
template <int NREP>
__device__ __forceinline__ void qk_f16_tm_tile(const SegDev &sg, int tile, int bh, int b, int hkv, int D,
                                               int Hq, int64_t Tall, const half2_t *q2s,
                                               half_t *__restrict__ scores) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = sg.n_tokens;
  const half_t *kb = (const half_t *)sg.data + (int64_t)bh * n * D;
  const int DP = D >> 1;
  for (int k = 0; k < 16; ++k) {
    const int64_t t = (int64_t)tile * 64 + wave * 16 + k;
    if (t >= n) break;  // uniform per wave
    float part[NREP];
#pragma unroll
    for (int h = 0; h < NREP; ++h) part[h] = 0.f;
    for (int dp = lane; dp < DP; dp += 64) {
      const half2_t kk = *reinterpret_cast<const half2_t *>(kb + t * D + 2 * dp);
#pragma unroll
      for (int h = 0; h < NREP; ++h) part[h] = __builtin_amdgcn_fdot2(kk, q2s[h * DP + dp], part[h], false);
    }
#pragma unroll
    for (int h = 0; h < NREP; ++h) part[h] = wave_sum(part[h]);
    if (lane == 0) {
      const int64_t pos = sg.idx ? sg.idx[t] : sg.pos_base + t;
#pragma unroll
      for (int h = 0; h < NREP; ++h)
        scores[((int64_t)b * Hq + hkv * NREP + h) * Tall + pos] = (half_t)part[h];
    }
  }
}

template <int NREP>
__global__ __launch_bounds__(QK_THREADS) void qk_hybrid_kernel(SegTable tb, const half_t *__restrict__ q,
                                                               half_t *__restrict__ scores, int Hq,
                                                               int Hkv, int D, int64_t Tall) {
  extern __shared__ float smem[];
  float *red = smem;                                          // 3 * 16 * 64 floats
  half2_t *q2s = reinterpret_cast<half2_t *>(smem + 3 * 16 * 64);  // NREP * D/2 pairs (q[d], q[d+1])
  const int bh = blockIdx.y;
  const int b = bh / Hkv, hkv = bh % Hkv;
  const uint32_t *qsrc = reinterpret_cast<const uint32_t *>(q + ((int64_t)b * Hq + hkv * NREP) * D);
  for (int k = threadIdx.x; k < NREP * (D >> 1); k += QK_THREADS) q2s[k] = as_h2(qsrc[k]);
  __syncthreads();
  const int s = find_seg(tb, blockIdx.x);
  const SegDev &sg = tb.seg[s];
  const int tile = blockIdx.x - sg.unit_begin;
  switch (sg.bits) {
    case 2: qk_quant_tile<2, NREP>(sg, tile, bh, b, hkv, D, Hq, Tall, q2s, red, scores); break;
    case 4: qk_quant_tile<4, NREP>(sg, tile, bh, b, hkv, D, Hq, Tall, q2s, red, scores); break;
    case 8: qk_quant_tile<8, NREP>(sg, tile, bh, b, hkv, D, Hq, Tall, q2s, red, scores); break;
    default:
      if (sg.token_major) qk_f16_tm_tile<NREP>(sg, tile, bh, b, hkv, D, Hq, Tall, q2s, scores);
      else qk_f16_cm_tile<NREP>(sg, tile, bh, b, hkv, D, Hq, Tall, q2s, red, scores);
  }
}

// =============================================================================== softmax
constexpr int SM_THREADS = 1024;

__device__ __forceinline__ float block_reduce(float v, float *sh, bool is_max) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();  // sh may still be read from a previous reduction
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  float r = sh[0];
  for (int k = 1; k < SM_THREADS / 64; ++k) r = is_max ? fmaxf(r, sh[k]) : r + sh[k];
  return r;
}

// x = max(rnd16(rnd16(s * inv_sqrt_d) + mask), -65504) -- the fp16 steps of quant_matmul_hq.py:100-102
__device__ __forceinline__ float sm_logit(half_t s, const half_t *mask, int64_t t, float inv) {
  half_t x = (half_t)((float)s * inv);
  if (mask) x = (half_t)((float)x + (float)mask[t]);
  return fmaxf((float)x, -65504.0f);
}

__global__ __launch_bounds__(SM_THREADS) void scale_softmax_kernel(half_t *__restrict__ scores,
                                                                   const half_t *__restrict__ mask,
                                                                   int64_t mask_row_stride, int64_t Tall,
                                                                   float inv) {
  __shared__ float sh[SM_THREADS / 64];
  half_t *row = scores + (int64_t)blockIdx.x * Tall;
  const half_t *mrow = mask ? mask + (int64_t)blockIdx.x * mask_row_stride : nullptr;
  float m = -INFINITY;
  for (int64_t t = threadIdx.x; t < Tall; t += SM_THREADS) m = fmaxf(m, sm_logit(row[t], mrow, t, inv));
  m = block_reduce(m, sh, true);
  float l = 0.f;
  for (int64_t t = threadIdx.x; t < Tall; t += SM_THREADS) l += expf(sm_logit(row[t], mrow, t, inv) - m);
  l = block_reduce(l, sh, false);
  for (int64_t t = threadIdx.x; t < Tall; t += SM_THREADS)
    row[t] = (half_t)(expf(sm_logit(row[t], mrow, t, inv) - m) / l);
}

// =============================================================================== p.V
constexpr int PV_THREADS = 256;
constexpr int PV_WAVES = 4;
constexpr int PV_BLOCK = 512;  // tokens staged in LDS at a time (256 token pairs)

// LDS block: per token pair {s2, z2} for each of the D/32 groups, and p2 for each query head
template <int NREP, int NG>
struct PvStage {
  uint2 sz[PV_BLOCK / 2][NG];
  half2_t p2[PV_BLOCK / 2][NREP];
};

// stage p (gathered through idx) and, for quantised classes, scale/zero of tokens [t0, t0+nt)
template <int NREP, int NG, bool QUANT>
__device__ __forceinline__ void pv_stage(const SegDev &sg, int64_t t0, int nt, int bh,
                                         const half_t *const (&prow)[NREP], PvStage<NREP, NG> &st) {
  const int ntp = (nt + 1) >> 1;
  for (int k = threadIdx.x; k < ntp * NREP; k += PV_THREADS) {
    const int tp = k / NREP, h = k % NREP;
    const int64_t ta = t0 + 2 * tp;
    const bool has_b = 2 * tp + 1 < nt;
    const int64_t pa = sg.idx ? sg.idx[ta] : sg.pos_base + ta;
    const int64_t pb = has_b ? (sg.idx ? sg.idx[ta + 1] : sg.pos_base + ta + 1) : pa;
    st.p2[tp][h] = pack_h2(prow[h][pa], has_b ? prow[h][pb] : (half_t)0);
  }
  if (QUANT) {  // n_tokens is a multiple of 32, so pairs are always complete
    const half_t *sc = sg.scale + ((int64_t)bh * sg.n_tokens + t0) * NG;
    const half_t *zr = sg.zero + ((int64_t)bh * sg.n_tokens + t0) * NG;
    for (int k = threadIdx.x; k < ntp * NG; k += PV_THREADS) {
      const int tp = k / NG, g = k % NG;
      uint2 v;
      v.x = as_u32(pack_h2(sc[(2 * tp) * NG + g], sc[(2 * tp + 1) * NG + g]));
      v.y = as_u32(pack_h2(zr[(2 * tp) * NG + g], zr[(2 * tp + 1) * NG + g]));
      st.sz[tp][g] = v;
    }
  }
}

template <int BITS, int NREP, int D>
__device__ __forceinline__ void pv_quant_chunk(const SegDev &sg, int64_t c0, int64_t c1, int bh,
                                               const half_t *const (&prow)[NREP], PvStage<NREP, D / 32> &st,
                                               float *red) {
  constexpr int PF = 32 / BITS;
  constexpr int WT = D / PF;    // words (lanes) per token row
  constexpr int TPW = 64 / WT;  // token pairs per wave step
  static_assert(WT >= 1 && WT <= 64 && (WT & (WT - 1)) == 0, "D/pf must be a power of two <= 64");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int jl = lane % WT, tl = lane / WT;
  const int g = (jl * PF) / 32;
  const uint32_t *code = (const uint32_t *)sg.data + (int64_t)bh * sg.n_tokens * WT + jl;

  float acc[NREP][PF];
#pragma unroll
  for (int h = 0; h < NREP; ++h)
#pragma unroll
    for (int i = 0; i < PF; ++i) acc[h][i] = 0.f;

  for (int64_t t0 = c0; t0 < c1; t0 += PV_BLOCK) {
    const int nt = (int)min((int64_t)PV_BLOCK, c1 - t0);
    __syncthreads();
    pv_stage<NREP, D / 32, true>(sg, t0, nt, bh, prow, st);
    __syncthreads();
    const int ntp = nt >> 1;
#pragma unroll 2
    for (int tp = wave * TPW + tl; tp < ntp; tp += PV_WAVES * TPW) {
      const int64_t t = t0 + 2 * tp;
      const uint32_t w0 = code[t * WT];
      const uint32_t w1 = code[(t + 1) * WT];
      const uint2 sz = st.sz[tp][g];
      half2_t p2[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) p2[h] = st.p2[tp][h];
      consume_words<BITS, NREP, PF>(w0, w1, as_h2(sz.x), as_h2(sz.y), p2, acc);
    }
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      float v = acc[h][i];
#pragma unroll
      for (int m = WT; m < 64; m <<= 1) v += xor_f(v, m);
      if (tl == 0) red[(wave * NREP + h) * D + jl * PF + i] = v;
    }
  }
}

template <int NREP, int D>
__device__ __forceinline__ void pv_f16_chunk(const SegDev &sg, int64_t c0, int64_t c1, int bh,
                                             const half_t *const (&prow)[NREP], PvStage<NREP, D / 32> &st,
                                             float *red) {
  constexpr int LPT = D / 2;     // lanes per token row (a lane owns two channels)
  constexpr int TPW = 64 / LPT;  // token pairs per wave step
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int jl = lane % LPT, tl = lane / LPT;
  const half_t *vb = (const half_t *)sg.data + (int64_t)bh * sg.n_tokens * D + jl * 2;
  float acc[NREP][2];
#pragma unroll
  for (int h = 0; h < NREP; ++h) acc[h][0] = acc[h][1] = 0.f;
  for (int64_t t0 = c0; t0 < c1; t0 += PV_BLOCK) {
    const int nt = (int)min((int64_t)PV_BLOCK, c1 - t0);
    __syncthreads();
    pv_stage<NREP, D / 32, false>(sg, t0, nt, bh, prow, st);
    __syncthreads();
    const int ntp = (nt + 1) >> 1;
#pragma unroll 2
    for (int tp = wave * TPW + tl; tp < ntp; tp += PV_WAVES * TPW) {
      const int64_t t = t0 + 2 * tp;
      const uint32_t r0 = *reinterpret_cast<const uint32_t *>(vb + t * D);
      const uint32_t r1 = (2 * tp + 1 < nt) ? *reinterpret_cast<const uint32_t *>(vb + (t + 1) * D) : 0u;
      const half2_t va = half_pair<0>(r0, r1);  // channel 2*jl:   (v[t], v[t+1])
      const half2_t vc = half_pair<1>(r0, r1);  // channel 2*jl+1
#pragma unroll
      for (int h = 0; h < NREP; ++h) {
        const half2_t p2 = st.p2[tp][h];
        acc[h][0] = __builtin_amdgcn_fdot2(va, p2, acc[h][0], false);
        acc[h][1] = __builtin_amdgcn_fdot2(vc, p2, acc[h][1], false);
      }
    }
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float v = acc[h][i];
#pragma unroll
      for (int m = LPT; m < 64; m <<= 1) v += xor_f(v, m);
      if (tl == 0) red[(wave * NREP + h) * D + jl * 2 + i] = v;
    }
  }
}

template <int NREP, int D>
__global__ __launch_bounds__(PV_THREADS) void pv_hybrid_kernel(SegTable tb, const half_t *__restrict__ p,
                                                               float *__restrict__ partial, int Hq, int Hkv,
                                                               int64_t Tall, int64_t chunk_tokens,
                                                               int64_t n_bhq) {
  __shared__ float red[PV_WAVES * NREP * D];
  __shared__ PvStage<NREP, D / 32> st;
  const int bh = blockIdx.y;
  const int b = bh / Hkv, hkv = bh % Hkv;
  const int s = find_seg(tb, blockIdx.x);
  const SegDev &sg = tb.seg[s];
  const int64_t c0 = (int64_t)(blockIdx.x - sg.unit_begin) * chunk_tokens;
  const int64_t c1 = min(c0 + chunk_tokens, sg.n_tokens);
  const half_t *prow[NREP];
#pragma unroll
  for (int h = 0; h < NREP; ++h) prow[h] = p + ((int64_t)b * Hq + hkv * NREP + h) * Tall;
  switch (sg.bits) {
    case 2: pv_quant_chunk<2, NREP, D>(sg, c0, c1, bh, prow, st, red); break;
    case 4: pv_quant_chunk<4, NREP, D>(sg, c0, c1, bh, prow, st, red); break;
    case 8: pv_quant_chunk<8, NREP, D>(sg, c0, c1, bh, prow, st, red); break;
    default: pv_f16_chunk<NREP, D>(sg, c0, c1, bh, prow, st, red);
  }
  __syncthreads();
  for (int k = threadIdx.x; k < NREP * D; k += PV_THREADS) {
    const float v = red[k] + red[NREP * D + k] + red[2 * NREP * D + k] + red[3 * NREP * D + k];
    const int h = k / D, d = k % D;
    partial[((int64_t)blockIdx.x * n_bhq + (int64_t)b * Hq + hkv * NREP + h) * D + d] = v;
  }
}

// fixed-order sum over chunks: deterministic replacement for the reference's half atomics
// (quant/csrc/gemv_cuda_wv_uniform.cu:110)
__global__ void pv_combine_kernel(const float *__restrict__ partial, half_t *__restrict__ out, int n_chunks,
                                  int64_t n_bhq, int D) {
  const int64_t r = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = 0.f;
    for (int c = 0; c < n_chunks; ++c) v += partial[((int64_t)c * n_bhq + r) * D + d];
    out[r * D + d] = (half_t)v;
  }
}

// =============================================================================== host side

static int build_table(const hqekv_seg *segs, int nseg, bool is_k, int64_t D, int64_t chunk_tokens,
                       int64_t Tall, SegTable *tb, const char *who) {
  if (nseg < 0 || nseg > HQEKV_MAX_SEGS) return fail(HQEKV_E_ARG, "%s: nseg=%d out of range", who, nseg);
  if (nseg > 0 && !segs) return fail(HQEKV_E_ARG, "%s: null segment table", who);
  int64_t units = 0;
  int m = 0;
  for (int k = 0; k < nseg; ++k) {
    const hqekv_seg &s = segs[k];
    if (s.n_tokens < 0) return fail(HQEKV_E_ARG, "%s: segment %d has negative n_tokens", who, k);
    if (s.n_tokens == 0) continue;
    if (!(s.bits == 16 || s.bits == 8 || s.bits == 4 || s.bits == 2))
      return fail(HQEKV_E_ARG, "%s: segment %d bits=%d (must be 16, 8, 4 or 2)", who, k, s.bits);
    if (!s.data) return fail(HQEKV_E_ARG, "%s: segment %d has null data", who, k);
    if (s.bits != 16) {
      if (!s.scale || !s.zero) return fail(HQEKV_E_ARG, "%s: segment %d lacks scale/zero", who, k);
      if (s.n_tokens % 32 != 0)
        return fail(HQEKV_E_ARG, "%s: segment %d n_tokens=%lld not a multiple of 32", who, k, (long long)s.n_tokens);
    }
    if (!s.idx && (s.pos_base < 0 || s.pos_base + s.n_tokens > Tall))
      return fail(HQEKV_E_ARG, "%s: segment %d positions [%lld,%lld) outside [0,%lld)", who, k,
                  (long long)s.pos_base, (long long)(s.pos_base + s.n_tokens), (long long)Tall);
    if ((uintptr_t)s.data & 3) return fail(HQEKV_E_ALIGN, "%s: segment %d data not 4-byte aligned", who, k);
    SegDev &d = tb->seg[m++];
    d.data = s.data;
    d.scale = (const half_t *)s.scale;
    d.zero = (const half_t *)s.zero;
    d.idx = s.idx;
    d.pos_base = s.pos_base;
    d.n_tokens = s.n_tokens;
    d.bits = s.bits;
    d.token_major = is_k ? (s.bits == 16 && s.token_major) : 0;
    d.unit_begin = (int32_t)units;
    d.pad_ = 0;
    const int64_t per = is_k ? qk_tile_tokens(s.bits, d.token_major) : chunk_tokens;
    units += (s.n_tokens + per - 1) / per;
    if (units > 0x3fffffff) return fail(HQEKV_E_ARG, "%s: too many work units", who);
  }
  tb->nseg = m;
  tb->total_units = (int32_t)units;
  (void)D;
  return HQEKV_OK;
}

static int check_heads(const char *who, int64_t B, int64_t Hq, int64_t Hkv, int64_t D) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
    return fail(HQEKV_E_ARG, "%s: need B>0 and Hq %% Hkv == 0 (B=%lld Hq=%lld Hkv=%lld)", who, (long long)B,
                (long long)Hq, (long long)Hkv);
  const int64_t nrep = Hq / Hkv;
  if (!(nrep == 1 || nrep == 2 || nrep == 4 || nrep == 8))
    return fail(HQEKV_E_UNSUPPORTED, "%s: Hq/Hkv=%lld (supported: 1, 2, 4, 8)", who, (long long)nrep);
  if (B * Hkv > 65535) return fail(HQEKV_E_ARG, "%s: B*Hkv > 65535", who);
  if (D <= 0 || D % 32 != 0) return fail(HQEKV_E_ARG, "%s: D=%lld must be a positive multiple of 32", who, (long long)D);
  return HQEKV_OK;
}

static int launch_qk(const SegTable &tb, const void *q, void *scores, int64_t B, int64_t Hq, int64_t Hkv,
                     int64_t D, int64_t Tall, hipStream_t st) {
  if (tb.total_units == 0) return HQEKV_OK;
  const int nrep = (int)(Hq / Hkv);
  dim3 grid((unsigned)tb.total_units, (unsigned)(B * Hkv)), block(QK_THREADS);
  const size_t shmem = (size_t)(nrep * D + 3 * 16 * 64) * sizeof(float);
#define LAUNCH(N_)                                                                                    \
  hipLaunchKernelGGL(qk_hybrid_kernel<N_>, grid, block, shmem, st, tb, (const half_t *)q, (half_t *)scores, \
                     (int)Hq, (int)Hkv, (int)D, Tall)
  switch (nrep) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 4: LAUNCH(4); break;
    default: LAUNCH(8);
  }
#undef LAUNCH
  return check_launch("qk_hybrid_kernel");
}

// chunk length for the p.V split-K: aim for a few workgroups per CU, never below 64 tokens
static int64_t pv_chunk_tokens(int64_t total_tokens, int64_t BHkv) {
  const int64_t target_wgs = 256 * 4;
  int64_t chunks_per_bh = (target_wgs + BHkv - 1) / BHkv;
  if (chunks_per_bh < 1) chunks_per_bh = 1;
  int64_t c = (total_tokens + chunks_per_bh - 1) / chunks_per_bh;
  c = (c + 63) / 64 * 64;
  if (c < 64) c = 64;
  if (c > 4096) c = 4096;
  return c;
}

static int64_t seg_total_tokens(const hqekv_seg *segs, int nseg) {
  int64_t n = 0;
  for (int k = 0; k < nseg; ++k) n += segs[k].n_tokens > 0 ? segs[k].n_tokens : 0;
  return n;
}

static int launch_pv(const SegTable &tb, int64_t chunk, const void *p, void *out, float *partial, int64_t B,
                     int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall, hipStream_t st) {
  const int nrep = (int)(Hq / Hkv);
  const int64_t n_bhq = B * Hq;
  if (tb.total_units > 0) {
    dim3 grid((unsigned)tb.total_units, (unsigned)(B * Hkv)), block(PV_THREADS);
#define LAUNCH(N_, D_)                                                                                   \
  hipLaunchKernelGGL((pv_hybrid_kernel<N_, D_>), grid, block, 0, st, tb, (const half_t *)p, partial, (int)Hq, \
                     (int)Hkv, Tall, chunk, n_bhq)
#define LAUNCH_D(N_) \
  if (D == 128) LAUNCH(N_, 128); else LAUNCH(N_, 64)
    switch (nrep) {
      case 1: LAUNCH_D(1); break;
      case 2: LAUNCH_D(2); break;
      case 4: LAUNCH_D(4); break;
      default: LAUNCH_D(8);
    }
#undef LAUNCH_D
#undef LAUNCH
    int rc = check_launch("pv_hybrid_kernel");
    if (rc) return rc;
  }
  hipLaunchKernelGGL(pv_combine_kernel, dim3((unsigned)n_bhq), dim3((unsigned)(D < 64 ? 64 : D)), 0, st, partial,
                     (half_t *)out, (int)tb.total_units, n_bhq, (int)D);
  return check_launch("pv_combine_kernel");
}

}  // namespace hq

using namespace hq;

extern "C" int hqekv_qk_hybrid(const hqekv_seg *segs, int nseg, const void *q, void *scores, int64_t B,
                               int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall, void *stream) {
  int rc = check_heads("qk_hybrid", B, Hq, Hkv, D);
  if (rc) return rc;
  if (D > 1024) return fail(HQEKV_E_UNSUPPORTED, "qk_hybrid: D=%lld > 1024", (long long)D);
  if (!q || !scores || Tall <= 0) return fail(HQEKV_E_ARG, "qk_hybrid: null pointer or Tall <= 0");
  SegTable tb{};
  rc = build_table(segs, nseg, true, D, 0, Tall, &tb, "qk_hybrid");
  if (rc) return rc;
  return launch_qk(tb, q, scores, B, Hq, Hkv, D, Tall, (hipStream_t)stream);
}

extern "C" int hqekv_scale_softmax(void *scores, const void *mask, int64_t mask_row_stride, int64_t n_rows,
                                   int64_t Tall, float inv_sqrt_d, void *stream) {
  if (n_rows < 0 || Tall <= 0 || n_rows > 0x7fffffffLL) return fail(HQEKV_E_ARG, "scale_softmax: bad shape");
  if (n_rows == 0) return HQEKV_OK;
  if (!scores) return fail(HQEKV_E_ARG, "scale_softmax: null scores");
  hipLaunchKernelGGL(scale_softmax_kernel, dim3((unsigned)n_rows), dim3(SM_THREADS), 0, (hipStream_t)stream,
                     (half_t *)scores, (const half_t *)mask, mask_row_stride, Tall, inv_sqrt_d);
  return check_launch("scale_softmax_kernel");
}

extern "C" int64_t hqekv_pv_workspace_bytes(const hqekv_seg *segs, int nseg, int64_t B, int64_t Hq,
                                            int64_t Hkv, int64_t D) {
  if (nseg < 0 || nseg > HQEKV_MAX_SEGS || (nseg > 0 && !segs) || B <= 0 || Hq <= 0 || Hkv <= 0) return -1;
  const int64_t chunk = pv_chunk_tokens(seg_total_tokens(segs, nseg), B * Hkv);
  int64_t chunks = 0;
  for (int k = 0; k < nseg; ++k)
    if (segs[k].n_tokens > 0) chunks += (segs[k].n_tokens + chunk - 1) / chunk;
  if (chunks == 0) chunks = 1;
  return chunks * B * Hq * D * (int64_t)sizeof(float);
}

extern "C" int hqekv_pv_hybrid(const hqekv_seg *segs, int nseg, const void *p, void *out, int64_t B, int64_t Hq,
                               int64_t Hkv, int64_t D, int64_t Tall, void *workspace, int64_t workspace_bytes,
                               void *stream) {
  int rc = check_heads("pv_hybrid", B, Hq, Hkv, D);
  if (rc) return rc;
  if (!(D == 128 || D == 64)) return fail(HQEKV_E_UNSUPPORTED, "pv_hybrid: D=%lld (supported: 64, 128)", (long long)D);
  if (!p || !out || Tall <= 0) return fail(HQEKV_E_ARG, "pv_hybrid: null pointer or Tall <= 0");
  const int64_t chunk = pv_chunk_tokens(seg_total_tokens(segs, nseg), B * Hkv);
  SegTable tb{};
  rc = build_table(segs, nseg, false, D, chunk, Tall, &tb, "pv_hybrid");
  if (rc) return rc;
  const int64_t need = (int64_t)(tb.total_units > 0 ? tb.total_units : 1) * B * Hq * D * (int64_t)sizeof(float);
  if (!workspace || workspace_bytes < need)
    return fail(HQEKV_E_WORKSPACE, "pv_hybrid: workspace %lld bytes < %lld needed", (long long)workspace_bytes,
                (long long)need);
  if ((uintptr_t)workspace & 15) return fail(HQEKV_E_ALIGN, "pv_hybrid: workspace not 16-byte aligned");
  return launch_pv(tb, chunk, p, out, (float *)workspace, B, Hq, Hkv, D, Tall, (hipStream_t)stream);
}

extern "C" int hqekv_decode_attn(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                                 const void *q, const void *mask, int64_t mask_row_stride, void *attn_weights,
                                 void *attn_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall,
                                 void *workspace, int64_t workspace_bytes, void *stream) {
  int rc = hqekv_qk_hybrid(k_segs, n_k, q, attn_weights, B, Hq, Hkv, D, Tall, stream);
  if (rc) return rc;
  const float inv = 1.0f / (float)sqrt((double)D);
  rc = hqekv_scale_softmax(attn_weights, mask, mask_row_stride, B * Hq, Tall, inv, stream);
  if (rc) return rc;
  return hqekv_pv_hybrid(v_segs, n_v, attn_weights, attn_out, B, Hq, Hkv, D, Tall, workspace, workspace_bytes,
                         stream);
}

// ------------------------------------------------------------------ per-class GEMV on the same kernels
static bool gemv_is_pv_shape(int64_t K, int64_t N) { return (N == 64 || N == 128) && K % 32 == 0 && K > N; }

extern "C" int64_t hqekv_gemv_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N, int bits) {
  (void)bits;
  if (!gemv_is_pv_shape(K, N)) return 0;
  hqekv_seg s{};
  s.bits = 2;
  s.n_tokens = K;
  return hqekv_pv_workspace_bytes(&s, 1, B, Hq, Hkv, N);
}

extern "C" int hqekv_gemv_uniform_group(const void *fA, const void *code, const void *scale, const void *zero,
                                        void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N,
                                        int bits, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!(bits == 2 || bits == 4 || bits == 8)) return fail(HQEKV_E_ARG, "gemv_uniform_group: bits=%d", bits);
  if (K <= 0 || N <= 0 || N % 32 != 0) return fail(HQEKV_E_ARG, "gemv_uniform_group: need N %% 32 == 0, K > 0");
  hqekv_seg s{};
  s.bits = bits;
  s.data = code;
  s.scale = scale;
  s.zero = zero;
  s.idx = nullptr;
  s.pos_base = 0;
  if (gemv_is_pv_shape(K, N)) {  // p.V: reduce over tokens, N = head_dim
    s.n_tokens = K;
    return hqekv_pv_hybrid(&s, 1, fA, out, B, Hq, Hkv, N, K, workspace, workspace_bytes, stream);
  }
  // q.K^T: reduce over the K rows, N = tokens
  if (K % 32 != 0) return fail(HQEKV_E_UNSUPPORTED, "gemv_uniform_group: K=%lld must be a multiple of 32", (long long)K);
  s.n_tokens = N;
  return hqekv_qk_hybrid(&s, 1, fA, out, B, Hq, Hkv, K, N, stream);
}
