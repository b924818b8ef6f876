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
// With four query heads per KV head the products of those values with the query (or the probabilities) run as
// 4x4x4 fp16 matrix instructions (same dequantised bits, exact products, fp32 accumulation; HQEKV_DOT_VALU keeps them
// on the vector ALU).  No packed-fp32 instructions are used.
//
// Layouts are consumed exactly as the cache stores them:
//   K class: code (B,Hkv,D,T/pf) -- a lane owns one packed word (pf tokens) and walks the D rows two
//            at a time, so the reduction over d needs no cross-lane traffic; 4 waves split D and meet
//            in LDS.
//   V class: code (B,Hkv,T,D/pf) -- D/pf lanes cover one token row and walk the tokens two at a time;
//            scale/zero and the gathered probabilities of a 512-token block are staged in LDS in
//            pair-interleaved order; lanes are reduced by butterflies, waves through LDS, workgroups
//            through fp32 partials summed in a fixed order.
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "common.h"

#pragma clang fp contract(off)  // the two fp16 roundings of the dequantiser must stay separate

#ifndef HQ_DEFAULT_DOT_MFMA
#define HQ_DEFAULT_DOT_MFMA true   // the form of the dot products for calls that name neither (see dot_on_matrix_cores)
#endif

namespace hq {

struct SegDev {
  const void *data;
  const half_t *scale;
  const half_t *zero;
  const int64_t *idx;
  int64_t pos_base;
  int64_t n_tokens;
  int32_t bits;
  int32_t layout;      // HQEKV_LAYOUT_*: 1 = fp16 K stored token-major, 2 = 1-bit normal-quantile coding
  int32_t unit_begin;  // first chunk of this segment in the p.V partial buffer
  int32_t n_units;     // tiles (q.K^T) or chunks (p.V) of this segment
  int64_t slab_tokens; // token rows between two (b, kv head) slabs of a token-major segment (>= n_tokens)
};

struct SegTable {
  SegDev seg[HQEKV_MAX_SEGS];
  int32_t nseg;
  int32_t total_units;
  int32_t max_units;   // the largest n_units of any segment
  int32_t pad_;
  int32_t begin[HQEKV_MAX_SEGS];  // first grid.y index of every segment (INT32_MAX past nseg): one scalar load finds a workgroup's segment
};

// grid.y enumerates the units of all segments back to back (no idle workgroups): unit u belongs to the last
// segment whose first unit is <= u.  Branch-free on the eight begins, which arrive in one scalar load.
__device__ __forceinline__ int seg_of_unit(const SegTable &tb, int u) {
  int s = -1;
#pragma unroll
  for (int k = 0; k < HQEKV_MAX_SEGS; ++k) s += (u >= tb.begin[k]) ? 1 : 0;
  return s;
}
// begin[s] without a second, dependent load from the argument segment
__device__ __forceinline__ int begin_of_seg(const SegTable &tb, int s) {
  int b = 0;
#pragma unroll
  for (int k = 0; k < HQEKV_MAX_SEGS; ++k) b += (k == s) ? tb.begin[k] : 0;
  return b;
}

// Optional fusion of the softmax into the two GEMV launches (valid when no mask is added and the K
// classes as well as the V classes each cover every position exactly once):
//   q.K^T stores the scaled fp16 logit instead of the raw score and one (max, sum exp) pair per tile and
//   head; p.V turns a logit into its probability while staging it and writes it back for the caller.
// The split-K partials are summed by the LAST p.V workgroup of each (b, kv head) to finish, when there are few
// enough of them; otherwise by a small launch of their own.  Nobody waits for anybody: a workgroup stores its
// partial rows write-through (agent-scope relaxed stores go past the per-XCD L2), waits for the stores to be
// acknowledged, and bumps one relaxed agent-scope counter; whoever reads the final count adds the rows up with
// loads that bypass the L2 as well, in the fixed order of the separate launch.  No release / acquire fences are
// involved: those write back and invalidate the whole L2 on this chip (the step went from 39 to 146 us with them).
struct FuseArgs {
  float2 *stats;       // (B*Hq, n_stat) pairs (m, l); nullptr = unfused
  int32_t n_stat;      // tiles per row of stats = number of q.K^T tiles per (b, kv head)
  float inv_sqrt_d;
  // Folded combine (independent of the softmax fusion): one arrival counter per (b, kv head), zeroed by the q.K^T
  // launch of the same call; nullptr = the split-K partials are summed by a launch of their own.
  uint32_t *arrive;
  half_t *out;         // (B*Hq, D) attention output, written by the last workgroup of each (b, kv head)
  int32_t two_step;    // never fold the bias removal of a code into its multiply (HQEKV_TWO_STEP_DEQUANT)
};
// More than eight query heads per KV head are served in slices of at most eight, one launch each: the launch's NREP
// heads are heads `off` .. `off` + NREP - 1 of the `group` query heads of their KV head (a launch that covers all
// heads: group = NREP, off = 0).  Group and offset ride in the upper half of the kernels' head-count argument,
// hq_slice = Hq | group << 16 | off << 24, and are used without a branch: as two members at the end of FuseArgs, or
// behind a test for "no slices", the kernel's other scalar loads ended up behind a first, dependent one -- half a
// microsecond in every workgroup -- and even one more plain argument moved the launches by a quarter.
// -> first query head (inside its batch row) that a workgroup of KV head `hkv` works on
__device__ __forceinline__ int first_head(int hq_slice, int hkv) { return hkv * ((hq_slice >> 16) & 0xff) + (int)((uint32_t)hq_slice >> 24); }
__host__ __device__ constexpr int hq_with_slice(int Hq, int group, int off) { return Hq | group << 16 | off << 24; }

// What the caller of a decode step does next to the attention (model/llama_hqe.py:131-133, 200), folded into the
// step's last launch: the row of the importance ring -- the probabilities summed over the batch, rounded to fp16,
// then summed over the heads and rounded again (model/public_func.py:243-257: attn_weights.sum(0).sum(0)) -- and
// the copies that append the step's key and value rows to the fp16 residual.
struct StepEpilogue {
  const half_t *weights;   // (B, Hq, Tall) probabilities
  half_t *ring_line;       // (Tall) or nullptr
  int64_t Tall;
  int32_t B, Hq;
  int32_t ring_by;         // threads torch's reduction deals the head rows to for this shape: 1 or 2
  int32_t app_rows;        // token rows to append per (b, kv head); 0 = none
  int32_t app_row_elems;   // head_dim
  int32_t app_bh;          // B * Hkv
  const half_t *app_src[2];
  half_t *app_dst[2];          // first destination row of slab 0
  int64_t app_src_slab[2];     // elements between two (b, kv head) slabs
  int64_t app_dst_slab[2];
};

// A workgroup learns its segment and its tile/chunk from its block id with two scalar loads at the top of
// the kernel: the eight unit begins, then the segment's 64-byte entry (a scalar load that misses costs about
// a microsecond; walking the table entry by entry would chain several of them).

// Workgroups are handed to the 8 XCDs round-robin in launch order, and each XCD has its own L2.
// Neighbouring tiles of one (b, kv head) slab share cache lines (a tile's row segment is shorter than a
// line, its scale/zero rows are a quarter of one), so the (b, kv head) index is the FASTEST grid
// dimension: with B*Hkv a multiple of 8, every tile of a slab runs on the same XCD, neighbours meet in
// one L2, and the eight XCDs get equal work.  (Tile-fastest order fetched every line 2x on average.)

// keep every load issued above this point ahead of the arithmetic below it (the scheduler would
// otherwise sink loads next to their uses to save registers, serialising the memory latency)
#define HQ_LOADS_ABOVE()                     \
  do {                                       \
    asm volatile("" ::: "memory");           \
    __builtin_amdgcn_sched_barrier(0);       \
  } while (0)

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
  // (u & MASK) | MAGIC in one VALU op; the mask rides in a scalar register, the magic in a vector one
  uint32_t r;
  const uint32_t magic_v = MAGIC;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(u), "s"(MASK), "v"(magic_v));
  const half2_t biased = as_h2(r);                      // 2^(10-POS) + c, exact
  const half2_t bias = as_h2(MAGIC);
  return biased - bias;                                 // c, exact
}

// The same field still carrying its bias: 2^(10-POS) + c.
template <int BITS, int I>
__device__ __forceinline__ half2_t field_pair_biased(uint32_t u) {
  constexpr int POS = I * BITS;
  constexpr uint32_t FMASK = ((1u << BITS) - 1u) << POS;
  constexpr uint32_t MASK = FMASK | (FMASK << 16);
  constexpr uint32_t EXPO = (uint32_t)(10 - POS + 15) << 10;
  constexpr uint32_t MAGIC = EXPO | (EXPO << 16);
  uint32_t r;
  const uint32_t magic_v = MAGIC;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(u), "s"(MASK), "v"(magic_v));
  return as_h2(r);
}
// -2^(10-POS) * s for field I: with it rnd16(c * s) is ONE fused multiply-add on the biased field,
// (2^(10-POS) + c) * s - 2^(10-POS) * s = c * s before the single rounding -- exactly the product the reference
// rounds -- provided 2^(10-POS) * s is itself an fp16 number, i.e. |s| < 64 at POS = 0 (scaling by a power of two
// is exact short of overflow).  Callers take this route only after checking the scales of the whole tile.
template <int BITS, int I>
__device__ __forceinline__ half2_t bias_times_scale(half2_t s2) {
  constexpr _Float16 NB = (_Float16)(-(float)(1 << (10 - I * BITS)));
  return s2 * (half2_t){NB, NB};
}

// the reference dequantiser's two roundings (quant/pack_unpack.py:331-332) on a pair of codes
__device__ __forceinline__ half2_t dequant_pair(half2_t c, half2_t s2, half2_t z2) {
  const half2_t m = c * s2;
  return m + z2;
}

// 1-bit normal-quantile coding (quant/pack_unpack.py:371-375): x = rnd16(rnd16(centre[c] * std) + mean)
// with centre = -+k, k = fp16(0.6745).  rnd16(-+k * std) = -+a with a = rnd16(k * std), so with a2 formed
// once per group the value is the single rounding of (2c - 1) * a + mean: two packed fused ops.
#define HQ_NORMAL1_CENTER ((_Float16)0.67431640625f)  // fp16(norm.ppf(0.75))
__device__ __forceinline__ half2_t normal1_spread(half2_t std2) {
  return std2 * (half2_t){HQ_NORMAL1_CENTER, HQ_NORMAL1_CENTER};
}
__device__ __forceinline__ half2_t dequant_pair_normal1(half2_t c, half2_t a2, half2_t mean2) {
  const half2_t t = __builtin_elementwise_fma(c, (half2_t){(_Float16)2, (_Float16)2}, (half2_t){(_Float16)-1, (_Float16)-1});
  return __builtin_elementwise_fma(t, a2, mean2);
}

// Consume one byte pair: 8/BITS dequantised pairs, each dotted with NREP operand pairs.
// NORMAL (1 bit only): s2 is the spread a2 = rnd16(k * std), z2 the mean.
template <int BITS, int NREP, int PF, bool NORMAL = false, int NFIELD = 8 / BITS>
__device__ __forceinline__ void consume_byte(uint32_t u, half2_t s2, half2_t z2, const half2_t (&a2)[NREP],
                                             float (&acc)[NREP][PF], int tok0) {
  constexpr int FPB = NFIELD;   // fields taken, from the low end of the byte
#define HQ_FIELD(I_)                                                                     \
  if constexpr (I_ < FPB) {                                                                      \
    const half2_t c2_ = field_pair<BITS, (I_ < FPB ? I_ : 0)>(u);                        \
    const half2_t x2 = NORMAL ? dequant_pair_normal1(c2_, s2, z2) : dequant_pair(c2_, s2, z2);  \
    _Pragma("unroll") for (int h = 0; h < NREP; ++h)                                     \
        acc[h][tok0 + I_] = __builtin_amdgcn_fdot2(x2, a2[h], acc[h][tok0 + I_], false); \
  }
  HQ_FIELD(0)
  HQ_FIELD(1)
  HQ_FIELD(2)
  HQ_FIELD(3)
  HQ_FIELD(4)
  HQ_FIELD(5)
  HQ_FIELD(6)
  HQ_FIELD(7)
#undef HQ_FIELD
}

// The same with the bias removal folded into the multiply (see bias_times_scale): nb[I] = -2^(10-POS_I) * s2.
template <int BITS, int NREP, int PF, int NFIELD>
__device__ __forceinline__ void consume_byte_fused_bias(uint32_t u, half2_t s2, half2_t z2, const half2_t (&nb)[8 / BITS],
                                                        const half2_t (&a2)[NREP], float (&acc)[NREP][PF], int tok0) {
#define HQ_FIELD(I_)                                                                      \
  if constexpr (I_ < NFIELD) {                                                            \
    const half2_t b2_ = field_pair_biased<BITS, (I_ < NFIELD ? I_ : 0)>(u);               \
    const half2_t m2_ = __builtin_elementwise_fma(b2_, s2, nb[I_ < NFIELD ? I_ : 0]);     \
    const half2_t x2 = m2_ + z2;                                                          \
    _Pragma("unroll") for (int h = 0; h < NREP; ++h)                                      \
        acc[h][tok0 + I_] = __builtin_amdgcn_fdot2(x2, a2[h], acc[h][tok0 + I_], false);  \
  }
  HQ_FIELD(0)
  HQ_FIELD(1)
  HQ_FIELD(2)
  HQ_FIELD(3)
  HQ_FIELD(4)
  HQ_FIELD(5)
  HQ_FIELD(6)
  HQ_FIELD(7)
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

// ------------------------------------------------------------------------------- matrix-core form of the dot products
// With four query heads per KV head the inner product is a 4 x 4 x 4 matrix product per lane group: heads x
// (four elements of the reduction axis) x (the four lanes' tokens or channels).  v_mfma_f32_4x4x4_16b_f16 runs sixteen
// such blocks per wave, a block per four consecutive lanes: lane l supplies row l % 4 of its block's A (four fp16) and
// column l % 4 of its block's B, and receives column l % 4 of D (four fp32).  A holds the query (or the probabilities)
// of head l % 4, B the lane's own dequantised values -- bit for bit the ones the vector-ALU form feeds to its
// dot products -- so D is (4 heads) x (this lane's token or channel): one instruction on the matrix pipe in place of
// eight two-element dot products on the vector ALU.  Products are exact in fp32, accumulation is fp32; only the order
// of the additions differs from the vector-ALU form.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f4_t mfma_4x4x4(half2_t a01, half2_t a23, half2_t b01, half2_t b23, f4_t c) {
  const half4_t a = __builtin_shufflevector(a01, a23, 0, 1, 2, 3);
  const half4_t b = __builtin_shufflevector(b01, b23, 0, 1, 2, 3);
  return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 0, 0, 0);
}

template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// field I of a byte pair, dequantised with the reference's two roundings
template <int BITS, int I, bool NORMAL>
__device__ __forceinline__ half2_t dequant_field(uint32_t u, half2_t s2, half2_t z2) {
  const half2_t c2 = field_pair<BITS, I>(u);
  return NORMAL ? dequant_pair_normal1(c2, s2, z2) : dequant_pair(c2, s2, z2);
}
// the same with the bias removal folded into the multiply: nb = bias_times_scale<BITS, I>(s2)
template <int BITS, int I>
__device__ __forceinline__ half2_t dequant_field_fused_bias(uint32_t u, half2_t s2, half2_t z2, half2_t nb) {
  const half2_t m2 = __builtin_elementwise_fma(field_pair_biased<BITS, I>(u), s2, nb);
  return m2 + z2;
}

// Matrix-core form of consume_byte: byte pair `ua` belongs to elements 0, 1 of the reduction axis (a row pair of K, a
// token pair of V), `ub` to elements 2, 3; (a01, a23) is the A operand for those four elements.
template <int BITS, bool NORMAL, int NFIELD, int N>
__device__ __forceinline__ void consume_bytes_mfma(uint32_t ua, uint32_t ub, half2_t sa, half2_t za, half2_t sb, half2_t zb,
                                                   half2_t a01, half2_t a23, f4_t (&acc)[N], int tok0) {
  static_for<NFIELD>([&](auto I_) {
    constexpr int I = decltype(I_)::value;
    const half2_t xa = dequant_field<BITS, I, NORMAL>(ua, sa, za);
    const half2_t xb = dequant_field<BITS, I, NORMAL>(ub, sb, zb);
    acc[tok0 + I] = mfma_4x4x4(a01, a23, xa, xb, acc[tok0 + I]);
  });
}
template <int BITS, int NFIELD, int N>
__device__ __forceinline__ void consume_bytes_mfma_fused_bias(uint32_t ua, uint32_t ub, half2_t sa, half2_t za, half2_t sb,
                                                              half2_t zb, const half2_t (&nba)[8 / BITS],
                                                              const half2_t (&nbb)[8 / BITS], half2_t a01, half2_t a23,
                                                              f4_t (&acc)[N], int tok0) {
  static_for<NFIELD>([&](auto I_) {
    constexpr int I = decltype(I_)::value;
    const half2_t xa = dequant_field_fused_bias<BITS, I>(ua, sa, za, nba[I]);
    const half2_t xb = dequant_field_fused_bias<BITS, I>(ub, sb, zb, nbb[I]);
    acc[tok0 + I] = mfma_4x4x4(a01, a23, xa, xb, acc[tok0 + I]);
  });
}
__device__ __forceinline__ uint32_t byte_pair_at(uint32_t lo, uint32_t hi, int k) {  // byte_pair<k>, k known after unrolling
  return k == 0 ? byte_pair<0>(lo, hi) : k == 1 ? byte_pair<1>(lo, hi) : k == 2 ? byte_pair<2>(lo, hi) : byte_pair<3>(lo, hi);
}

// =============================================================================== q.K^T
// A tile is worked on by W = 8 waves (small launches: shortest critical path per tile) or W = 4 waves
// (large launches: more independent workgroups per CU, so one tile's load and reduce phases overlap
// another's arithmetic).
constexpr int QK_TPL = 8;               // tokens per lane in every channel-major class
constexpr int QK_TILE = 64 * QK_TPL;    // tokens per workgroup tile
// row pairs per register block (two blocks of loads are in flight per wave): 2 with 8 waves per tile, where
// the smaller blocks keep the kernel at 4 waves per SIMD; 4 with 4 waves per tile
__host__ __device__ constexpr int qk_unr(int waves) { return waves == 8 ? 2 : 4; }


// What a lane holds of one block of QK_UNR row pairs of a quantised class (32-bit members only: a struct
// with 16-bit members is not kept in registers).
template <int BITS, int QK_UNR>
struct QkBlock {
  static constexpr int NW = BITS == 8 ? 2 : 1;  // packed words per lane per row
  uint32_t w0[QK_UNR][NW], w1[QK_UNR][NW];
  uint32_t s0[QK_UNR], s1[QK_UNR], z0[QK_UNR], z1[QK_UNR];  // fp16 bit patterns, zero-extended
};

// Accumulate one quantised tile: 512 tokens x D channels.  A lane owns 8 consecutive tokens: a byte of a
// packed word at 1 bit (four lanes read the same word), half a word at 2 bits, one word at 4 bits, two
// words at 8 bits.  The loads of a wave's first block are issued before the query is staged (stage_q ends
// with the workgroup barrier), and each later block is requested while the previous one is consumed, so a
// wave always has one block of loads in flight; the rolled loop keeps the code small enough to stay in the
// instruction cache from one launch to the next.
template <int BITS, int NREP, int QK_WAVES, bool NORMAL, bool MF, typename StageQ>
__device__ __forceinline__ void qk_quant_accumulate(const SegDev &sg, uint32_t ts, int bh, int D, int wave,
                                                    StageQ &&stage_q, const half2_t *q2s,
                                                    float (&acc)[NREP][QK_TPL]) {
  static_assert(!MF || NREP == 4, "the matrix-core form is a 4-head product");
  constexpr int PF = 32 / BITS;
  constexpr int QK_UNR = qk_unr(QK_WAVES);
  using Block = QkBlock<BITS, QK_UNR>;
  constexpr int NW = Block::NW;
  const uint32_t n = (uint32_t)sg.n_tokens;
  const uint32_t wpr = n / PF;   // words per row
  const uint32_t gpr = n >> 5;   // groups per row
  const uint32_t wofs = (ts / PF) * 4u;  // byte offset of this lane's first word inside a row
  const uint32_t gofs = (ts >> 5) * 2u;  // byte offset of this lane's group inside a scale/zero row
  const int sh2 = (BITS == 2) ? (int)((ts >> 3) & 1) * 16      // which half of the 2-bit word
                  : (BITS == 1) ? (int)((ts >> 3) & 3) * 8     // which byte of the 1-bit word
                                : 0;
  const rsrc_t rc = make_rsrc((const uint32_t *)sg.data + (int64_t)bh * D * wpr, (uint32_t)D * wpr * 4u);
  const rsrc_t rs = make_rsrc(sg.scale + (int64_t)bh * D * gpr, (uint32_t)D * gpr * 2u);
  const rsrc_t rz = make_rsrc(sg.zero + (int64_t)bh * D * gpr, (uint32_t)D * gpr * 2u);
  const int DP = D >> 1;

  auto load = [&](int dp0, Block &r) {
#pragma unroll
    for (int k = 0; k < QK_UNR; ++k) {
      const int dpk = dp0 + QK_WAVES * k;
      const uint32_t d = 2u * (uint32_t)(dpk < DP ? dpk : dp0);  // uniform; past-the-end pairs reload dp0
      const uint32_t crow = d * wpr * 4u, grow = d * gpr * 2u;   // scalar row offsets
#pragma unroll
      for (int j = 0; j < NW; ++j) {
        r.w0[k][j] = buf_u32(rc, wofs + 4 * j, crow);
        r.w1[k][j] = buf_u32(rc, wofs + 4 * j, crow + wpr * 4u);
      }
      r.s0[k] = buf_u16(rs, gofs, grow);
      r.s1[k] = buf_u16(rs, gofs, grow + gpr * 2u);
      r.z0[k] = buf_u16(rz, gofs, grow);
      r.z1[k] = buf_u16(rz, gofs, grow + gpr * 2u);
    }
  };
  f4_t av[QK_TPL];  // matrix-core form: (4 heads) per token of this lane
#pragma unroll
  for (int i = 0; i < QK_TPL; ++i) av[i] = (f4_t){0.f, 0.f, 0.f, 0.f};
  const int hl = threadIdx.x & 3;  // the head whose query this lane supplies to the matrix product
  // two row pairs = four channels per matrix product (head_dim is a multiple of 32, so a block's row pairs all exist)
  auto compute_mf = [&](int dp0, const Block &r) {
#pragma unroll
    for (int k = 0; k < QK_UNR; k += 2) {
      const int dpa = dp0 + QK_WAVES * k, dpb = dpa + QK_WAVES;
      const half2_t qa = q2s[dpa * NREP + hl], qb = q2s[dpb * NREP + hl];
      half2_t sa = half_pair<0>(r.s0[k], r.s1[k]), sb = half_pair<0>(r.s0[k + 1], r.s1[k + 1]);
      const half2_t za = half_pair<0>(r.z0[k], r.z1[k]), zb = half_pair<0>(r.z0[k + 1], r.z1[k + 1]);
      if (NORMAL) {
        sa = normal1_spread(sa);
        sb = normal1_spread(sb);
      }
      constexpr int FPB = 8 / BITS;
      constexpr int NBYTE = BITS;            // bytes that hold a lane's 8 codes of one row
      constexpr int NF = BITS == 1 ? 8 : FPB;
#pragma unroll
      for (int j = 0; j < NBYTE; ++j) {
        const int sh = BITS <= 2 ? sh2 : 0;
        const uint32_t ua = byte_pair_at(r.w0[k][j / 4] >> sh, r.w1[k][j / 4] >> sh, j % 4);
        const uint32_t ub = byte_pair_at(r.w0[k + 1][j / 4] >> sh, r.w1[k + 1][j / 4] >> sh, j % 4);
        consume_bytes_mfma<BITS, NORMAL, NF, QK_TPL>(ua, ub, sa, za, sb, zb, qa, qb, av, j * FPB);
      }
    }
  };
  auto compute_valu = [&](int dp0, const Block &r) {
#pragma unroll
    for (int k = 0; k < QK_UNR; ++k) {
      const int dp = dp0 + QK_WAVES * k;
      if (dp >= DP) break;  // uniform
      half2_t q2[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) q2[h] = q2s[dp * NREP + h];
      half2_t s2 = half_pair<0>(r.s0[k], r.s1[k]);
      const half2_t z2 = half_pair<0>(r.z0[k], r.z1[k]);
      if (NORMAL) s2 = normal1_spread(s2);
      if (BITS == 1) {
        const uint32_t a0 = r.w0[k][0] >> sh2, a1 = r.w1[k][0] >> sh2;
        consume_byte<1, NREP, QK_TPL, NORMAL>(byte_pair<0>(a0, a1), s2, z2, q2, acc, 0);
      } else if (BITS == 2) {
        const uint32_t a0 = r.w0[k][0] >> sh2, a1 = r.w1[k][0] >> sh2;
        consume_byte<2, NREP, QK_TPL>(byte_pair<0>(a0, a1), s2, z2, q2, acc, 0);
        consume_byte<2, NREP, QK_TPL>(byte_pair<1>(a0, a1), s2, z2, q2, acc, 4);
      } else if (BITS == 4) {
        consume_byte<4, NREP, QK_TPL>(byte_pair<0>(r.w0[k][0], r.w1[k][0]), s2, z2, q2, acc, 0);
        consume_byte<4, NREP, QK_TPL>(byte_pair<1>(r.w0[k][0], r.w1[k][0]), s2, z2, q2, acc, 2);
        consume_byte<4, NREP, QK_TPL>(byte_pair<2>(r.w0[k][0], r.w1[k][0]), s2, z2, q2, acc, 4);
        consume_byte<4, NREP, QK_TPL>(byte_pair<3>(r.w0[k][0], r.w1[k][0]), s2, z2, q2, acc, 6);
      } else {
#pragma unroll
        for (int j = 0; j < NW; ++j) {
          consume_byte<8, NREP, QK_TPL>(byte_pair<0>(r.w0[k][j], r.w1[k][j]), s2, z2, q2, acc, 4 * j + 0);
          consume_byte<8, NREP, QK_TPL>(byte_pair<1>(r.w0[k][j], r.w1[k][j]), s2, z2, q2, acc, 4 * j + 1);
          consume_byte<8, NREP, QK_TPL>(byte_pair<2>(r.w0[k][j], r.w1[k][j]), s2, z2, q2, acc, 4 * j + 2);
          consume_byte<8, NREP, QK_TPL>(byte_pair<3>(r.w0[k][j], r.w1[k][j]), s2, z2, q2, acc, 4 * j + 3);
        }
      }
    }
  };

  auto compute = [&](int dp0, const Block &r) {
    if constexpr (MF) compute_mf(dp0, r);
    else compute_valu(dp0, r);
  };
  // two register blocks in turn: while one is consumed the other one's loads are in flight
  constexpr int STEP = QK_WAVES * QK_UNR;
  Block ba, bb;
  load(wave, ba);
  stage_q();
#pragma unroll 1
  for (int dp0 = wave; dp0 < DP; dp0 += 2 * STEP) {  // every condition below is uniform
    if (dp0 + STEP < DP) load(dp0 + STEP, bb);
    HQ_LOADS_ABOVE();
    compute(dp0, ba);
    if (dp0 + 2 * STEP < DP) load(dp0 + 2 * STEP, ba);
    HQ_LOADS_ABOVE();
    if (dp0 + STEP < DP) compute(dp0 + STEP, bb);
  }
  if constexpr (MF) {
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int i = 0; i < QK_TPL; ++i) acc[h][i] = av[i][h];
  }
}

// fp16 class stored channel-major (B,Hkv,D,T): a lane owns 8 adjacent tokens of each row
template <int NREP, int QK_WAVES, bool MF, typename StageQ>
__device__ __forceinline__ void qk_f16_cm_accumulate(const SegDev &sg, uint32_t t0, int bh, int D, int wave,
                                                     StageQ &&stage_q, const half2_t *q2s,
                                                     float (&acc)[NREP][QK_TPL]) {
  static_assert(!MF || NREP == 4, "the matrix-core form is a 4-head product");
  const uint32_t n = (uint32_t)sg.n_tokens;
  const half_t *kp = (const half_t *)sg.data + (int64_t)bh * D * n;
  const bool vec = (n & 7) == 0 && (((uintptr_t)kp) & 15) == 0 && t0 < n;  // rows stay 16-byte aligned
  const int DP = D >> 1;
  auto load8 = [&](const half_t *row, uint32_t (&r)[4]) {
    if (vec) {
      const uint4 v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(row) + t0 * 2u);
      r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t ta = t0 + 2 * i, tb = ta + 1;
        r[i] = as_u32(pack_h2(ta < n ? row[ta] : (half_t)0, tb < n ? row[tb] : (half_t)0));
      }
    }
  };
  constexpr int UNR = 2;
  struct Rows {
    uint32_t r0[UNR][4], r1[UNR][4];
  };
  auto load = [&](int dp0, Rows &r) {
#pragma unroll
    for (int k = 0; k < UNR; ++k) {
      const int dpk = dp0 + QK_WAVES * k;
      const uint32_t d = 2u * (uint32_t)(dpk < DP ? dpk : dp0);
      load8(kp + (size_t)d * n, r.r0[k]);
      load8(kp + (size_t)(d + 1) * n, r.r1[k]);
    }
  };
  f4_t av[QK_TPL];
#pragma unroll
  for (int i = 0; i < QK_TPL; ++i) av[i] = (f4_t){0.f, 0.f, 0.f, 0.f};
  const int hl = threadIdx.x & 3;
  auto compute = [&](int dp0, const Rows &r) {
    if constexpr (MF) {   // the block's two row pairs = four channels per matrix product
      static_assert(UNR == 2, "one matrix product per token and block");
      const int dpa = dp0, dpb = dp0 + QK_WAVES;
      const half2_t qa = q2s[dpa * NREP + hl], qb = q2s[dpb * NREP + hl];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[2 * i] = mfma_4x4x4(qa, qb, half_pair<0>(r.r0[0][i], r.r1[0][i]), half_pair<0>(r.r0[1][i], r.r1[1][i]), av[2 * i]);
        av[2 * i + 1] = mfma_4x4x4(qa, qb, half_pair<1>(r.r0[0][i], r.r1[0][i]), half_pair<1>(r.r0[1][i], r.r1[1][i]), av[2 * i + 1]);
      }
    } else {
#pragma unroll
      for (int k = 0; k < UNR; ++k) {
        const int dp = dp0 + QK_WAVES * k;
        if (dp >= DP) break;  // uniform
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const half2_t ka = half_pair<0>(r.r0[k][i], r.r1[k][i]);  // token 2i:   (k[d], k[d+1])
          const half2_t kb = half_pair<1>(r.r0[k][i], r.r1[k][i]);  // token 2i+1
#pragma unroll
          for (int h = 0; h < NREP; ++h) {
            const half2_t q2 = q2s[dp * NREP + h];
            acc[h][2 * i] = __builtin_amdgcn_fdot2(ka, q2, acc[h][2 * i], false);
            acc[h][2 * i + 1] = __builtin_amdgcn_fdot2(kb, q2, acc[h][2 * i + 1], false);
          }
        }
      }
    }
  };
  constexpr int STEP = QK_WAVES * UNR;
  Rows ba, bb;
  load(wave, ba);
  stage_q();
#pragma unroll 1
  for (int dp0 = wave; dp0 < DP; dp0 += 2 * STEP) {  // every condition below is uniform
    if (dp0 + STEP < DP) load(dp0 + STEP, bb);
    HQ_LOADS_ABOVE();
    compute(dp0, ba);
    if (dp0 + 2 * STEP < DP) load(dp0 + 2 * STEP, ba);
    HQ_LOADS_ABOVE();
    if (dp0 + STEP < DP) compute(dp0 + STEP, bb);
  }
  if constexpr (MF) {
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int i = 0; i < QK_TPL; ++i) acc[h][i] = av[i][h];
  }
}

// fp16 residual stored token-major (B,Hkv,T,D), one 64-token tile per workgroup.
// D == 128: a wave takes 8 tokens at a time, 8 lanes per token, 16 channels (two 128-bit loads) per lane, so
// all of a wave's loads are in flight together and a token's dot product is reduced across 8 lanes.
// Other D: a wave walks its tokens one by one, lanes split the channels.
template <int NREP, int QK_WAVES>
__device__ __forceinline__ void qk_f16_tm_tile(const SegDev &sg, int tile, int bh, int b, int head0, int D,
                                               int Hq, int64_t Tall, int wave, int lane, const half2_t *q2s,
                                               half_t *__restrict__ scores, const FuseArgs &fz, float *red) {
  const int64_t n = sg.n_tokens;
  const half_t *kb = (const half_t *)sg.data + (int64_t)bh * sg.slab_tokens * D;
  const int DP = D >> 1;
  constexpr int TPW = 64 / QK_WAVES;  // tokens per wave
  float m_run[NREP], l_run[NREP];  // running softmax statistics of this wave's tokens (fused mode)
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
    m_run[h] = -INFINITY;
    l_run[h] = 0.f;
  }
  if (D == 128) {
    const int lg = lane & 7, tsub = lane >> 3;
#pragma unroll 2
    for (int r = 0; r < TPW / 8; ++r) {
      const int64_t t = (int64_t)tile * 64 + wave * TPW + r * 8 + tsub;
      const bool valid = t < n;
      const int64_t tc = valid ? t : n - 1;
      const uint4 *src = reinterpret_cast<const uint4 *>(kb + tc * 128 + lg * 16);
      const uint4 lo = src[0], hi = src[1];
      const uint32_t pos = sg.idx ? reinterpret_cast<const uint32_t *>(sg.idx)[2 * tc] : (uint32_t)(sg.pos_base + tc);
      const uint32_t kw[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      float part[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) part[h] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int h = 0; h < NREP; ++h)
          part[h] = __builtin_amdgcn_fdot2(as_h2(kw[j]), q2s[(lg * 8 + j) * NREP + h], part[h], false);
#pragma unroll
      for (int h = 0; h < NREP; ++h) {
        float v = part[h];  // the token's 8 lanes: two quad permutes, then the half-row mirror joins the quads
        v += dpp_f<0xB1>(v);
        v += dpp_f<0x4E>(v);
        v += dpp_f<0x141>(v);
        half_t rr = (half_t)v;
        if (fz.stats) {
          rr = (half_t)((float)rr * fz.inv_sqrt_d);
          const float x = valid ? (float)rr : -INFINITY;
          const float mn = fmaxf(m_run[h], wave_max(x));
          const float e = (valid && lg == 0) ? __expf(x - mn) : 0.f;
          const float keep = (m_run[h] == mn) ? 1.f : __expf(m_run[h] - mn);  // also covers -inf == -inf
          l_run[h] = l_run[h] * keep + wave_sum(e);
          m_run[h] = mn;
        }
        if (valid && lg == 0) scores[((int64_t)b * Hq + head0 + h) * Tall + pos] = rr;
      }
    }
  } else {
#pragma unroll 1
    for (int k = 0; k < TPW; ++k) {
      const int64_t t = (int64_t)tile * 64 + wave * TPW + k;
      if (t >= n) break;  // uniform per wave
      float part[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) part[h] = 0.f;
      for (int dp = lane; dp < DP; dp += 64) {
        const half2_t kk = *reinterpret_cast<const half2_t *>(kb + t * D + 2 * dp);
#pragma unroll
        for (int h = 0; h < NREP; ++h) part[h] = __builtin_amdgcn_fdot2(kk, q2s[dp * NREP + h], part[h], false);
      }
      const int64_t pos = sg.idx ? sg.idx[t] : sg.pos_base + t;
#pragma unroll
      for (int h = 0; h < NREP; ++h) {
        half_t r = (half_t)wave_sum(part[h]);
        if (fz.stats) {
          r = (half_t)((float)r * fz.inv_sqrt_d);
          const float x = (float)r, mn = fmaxf(m_run[h], x);
          l_run[h] = l_run[h] * __expf(m_run[h] - mn) + __expf(x - mn);
          m_run[h] = mn;
        }
        if (lane == 0) scores[((int64_t)b * Hq + head0 + h) * Tall + pos] = r;
      }
    }
  }
  if (fz.stats) {  // one (m, l) pair per head for the whole 64-token tile
    if (lane == 0) {
#pragma unroll
      for (int h = 0; h < NREP; ++h) {
        red[(wave * NREP + h) * 2 + 0] = m_run[h];
        red[(wave * NREP + h) * 2 + 1] = l_run[h];
      }
    }
    __syncthreads();
    if (threadIdx.x < NREP) {
      const int h = threadIdx.x;
      float m = -INFINITY, l = 0.f;
      for (int w = 0; w < QK_WAVES; ++w) m = fmaxf(m, red[(w * NREP + h) * 2]);
      for (int w = 0; w < QK_WAVES; ++w) {
        const float lw = red[(w * NREP + h) * 2 + 1];
        if (lw > 0.f) l += lw * __expf(red[(w * NREP + h) * 2] - m);
      }
      fz.stats[((int64_t)b * Hq + head0 + h) * fz.n_stat + sg.unit_begin + tile] = make_float2(m, l);
    }
  }
}

// heads reduced per pass of the cross-wave reduction: the largest of 4 (four waves per tile only), 2, 1 that divides
// the heads of the launch; at most 32 KB of LDS per pass
__host__ __device__ constexpr int qk_reduce_heads(int nrep, int waves) {
  return (waves == 4 && nrep % 4 == 0) ? 4 : (nrep % 2 == 0 ? 2 : 1);
}
template <int NREP, int QK_WAVES>
struct QkReduce {
  static constexpr int RH = qk_reduce_heads(NREP, QK_WAVES);
  static constexpr int VPT = RH * QK_TILE / (QK_WAVES * 64);  // values a thread sums and stores per pass
  static constexpr int WPH = QK_WAVES / RH;                    // waves that share a head in a pass
  static_assert(VPT >= 1 && VPT <= QK_TPL && WPH >= 1, "reduction shape");
};

// One workgroup = one tile of one class for one (b, kv head).  The class-specific code is only the
// accumulation; the cross-wave reduction and the (scattered) store are shared by every class.
//
template <int NREP, int QK_WAVES, bool MF = false>
__global__ __launch_bounds__(QK_WAVES * 64, NREP <= 4 ? 16 / QK_WAVES : 1) void qk_hybrid_kernel(SegTable tb, const half_t *__restrict__ q,
                                                               half_t *__restrict__ scores, int hq_slice,
                                                               int Hkv, int D, int64_t Tall, FuseArgs fz, int tpw) {
  using R = QkReduce<NREP, QK_WAVES>;
  constexpr int RH = R::RH, VPT = R::VPT, WPH = R::WPH;
  extern __shared__ float smem[];
  float *red = smem;                                                              // QK_WAVES * RH * 512 floats
  half2_t *q2s = reinterpret_cast<half2_t *>(smem + QK_WAVES * RH * QK_TILE);      // D/2 x NREP pairs (q[d], q[d+1])
  __shared__ float2 wave_ml[NREP][QK_WAVES];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int bh = blockIdx.x;
  const int b = bh / Hkv, hkv = bh % Hkv;
  const int Hq = hq_slice & 0xffff, head0 = first_head(hq_slice, hkv);
  if (fz.arrive && blockIdx.y == 0 && threadIdx.x == 0) fz.arrive[bh] = 0;  // for the p.V launch that follows
  // grid.y counts workgroups; a workgroup takes `tpw` consecutive tiles of one class (1 unless the
  // environment asks for more: longer-lived workgroups stage the query once, but measured no faster)
  const int si = seg_of_unit(tb, blockIdx.y);
  const SegDev sg = tb.seg[si];  // by value: one batch of scalar loads, no lazy re-reads
  const int tile_begin = ((int)blockIdx.y - begin_of_seg(tb, si)) * tpw;
  const int tile_end = min(tile_begin + tpw, (int)sg.n_units);
  const bool tm = sg.bits == 16 && sg.layout == HQEKV_LAYOUT_TOKEN_MAJOR;
  const uint32_t n = (uint32_t)sg.n_tokens;
  const uint32_t *qsrc = reinterpret_cast<const uint32_t *>(q + ((int64_t)b * Hq + head0) * D);
  // The query is staged by the first tile only; for every tile the call is the workgroup barrier between
  // "first loads requested" and "arithmetic starts", and between two tiles' uses of the reduction buffer.
  bool staged = false;
  auto stage_q = [&]() {
    if (!staged) {
      for (int k = threadIdx.x; k < NREP * (D >> 1); k += QK_WAVES * 64) {
        const int h = k / (D >> 1), dp = k % (D >> 1);
        q2s[dp * NREP + h] = as_h2(qsrc[k]);  // [dp][h]: one 16-byte LDS read fetches a row pair for 4 heads
      }
      staged = true;
    }
    __syncthreads();
  };
  if (tm) {
#pragma unroll 1
    for (int tile = tile_begin; tile < tile_end; ++tile) {
      stage_q();
      qk_f16_tm_tile<NREP, QK_WAVES>(sg, tile, bh, b, head0, D, Hq, Tall, wave, lane, q2s, scores, fz, red);
    }
    return;
  }

  // The tile loop lives inside each class's branch (instantiated once per class by the generic lambda), so
  // what a class keeps in registers across tiles is its own and not the union over all classes.
  auto run_tiles = [&](auto accumulate) {
#pragma unroll 1
    for (int tile = tile_begin; tile < tile_end; ++tile) {
      const uint32_t t0 = (uint32_t)tile * QK_TILE + lane * QK_TPL;
      const uint32_t ts = t0 < n ? t0 : 0;  // lanes past the end recompute token 0 and store nothing
      // the VPT values this thread reduces and stores in every pass: head hl of the pass, tokens tok .. tok+VPT-1
      const int hl = (int)(threadIdx.x * VPT) / QK_TILE;
      const uint32_t tok = (uint32_t)tile * QK_TILE + (threadIdx.x * VPT) % QK_TILE;
      // their positions: requested first (branch-free, so the loads overlap), used last.  Positions are below
      // 2^31 (they index a row of Tall fp16 scores), so the low word of each int64 index is enough.
      uint32_t pos[VPT];
      {
        const uint32_t *ip = reinterpret_cast<const uint32_t *>(sg.idx);
        const bool has_idx = ip != nullptr;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
          const uint32_t t = min(tok + i, n - 1);
          pos[i] = (uint32_t)sg.pos_base + t;
          if (has_idx) pos[i] = ip[2 * t];
        }
      }
      float acc[NREP][QK_TPL];
#pragma unroll
      for (int h = 0; h < NREP; ++h)
#pragma unroll
        for (int i = 0; i < QK_TPL; ++i) acc[h][i] = 0.f;
      accumulate(ts, t0, acc);

      // Cross-wave reduction, RH heads per pass.  Every wave parks its partial rows (token-contiguous, two
      // 128-bit LDS writes per head); then ALL threads share the summation: a thread adds the QK_WAVES
      // partials of VPT adjacent tokens of one head (one vector LDS read per partial, conflict-free), rounds,
      // and stores them, so a wave writes 128 * VPT contiguous bytes of a score row.
      bool contig = (tok + VPT <= n);
#pragma unroll
      for (int i = 1; i < VPT; ++i) contig = contig && (pos[i] == pos[0] + i);
#pragma unroll
      for (int h0 = 0; h0 < NREP; h0 += RH) {
        if (h0 > 0) __syncthreads();
#pragma unroll
        for (int j = 0; j < RH; ++j) {
          // a partial row is parked as two planes -- tokens 0-3 and tokens 4-7 of every lane -- so that the lanes of
          // a wave write adjacent 16-byte pieces (one plane of [lane][8] would put them 32 bytes apart: two-way
          // bank conflicts on every 128-bit access)
          float *row = red + (wave * RH + j) * QK_TILE;
          *reinterpret_cast<float4 *>(row + lane * 4) = make_float4(acc[h0 + j][0], acc[h0 + j][1], acc[h0 + j][2], acc[h0 + j][3]);
          *reinterpret_cast<float4 *>(row + QK_TILE / 2 + lane * 4) = make_float4(acc[h0 + j][4], acc[h0 + j][5], acc[h0 + j][6], acc[h0 + j][7]);
        }
        __syncthreads();
        const int h = h0 + hl;
        float a[VPT];
#pragma unroll
        for (int i = 0; i < VPT; ++i) a[i] = 0.f;
        constexpr int PIECE = VPT < 4 ? VPT : 4;                 // adjacent tokens that lie together in a plane
        const int tk = (int)(threadIdx.x * VPT) % QK_TILE;       // first of this thread's tokens inside the tile
#pragma unroll
        for (int w = 0; w < QK_WAVES; ++w) {
          const float *row = red + (w * RH + hl) * QK_TILE;
          float part[VPT];
#pragma unroll
          for (int i0 = 0; i0 < VPT; i0 += PIECE) {
            const int t = tk + i0;  // token t = 8 * lane + i sits at plane i / 4, [lane][i % 4]
            __builtin_memcpy(part + i0, row + ((t & 4) ? QK_TILE / 2 : 0) + (t >> 3) * 4 + (t & 3), PIECE * 4);
          }
#pragma unroll
          for (int i = 0; i < VPT; ++i) a[i] += part[i];
        }
        half_t v[VPT];
        float m_lane = -INFINITY;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
          v[i] = (half_t)a[i];
          if (fz.stats) {  // the fp16 steps of the reference epilogue: round the score, scale, round again
            v[i] = (half_t)((float)v[i] * fz.inv_sqrt_d);
            if (tok + i < n) m_lane = fmaxf(m_lane, (float)v[i]);
          }
        }
        if (fz.stats) {  // (max, sum exp) of this wave's 64 * VPT tokens; merged per head after the last pass
          const float m = wave_max(m_lane);
          float l_lane = 0.f;
#pragma unroll
          for (int i = 0; i < VPT; ++i)
            if (tok + i < n) l_lane += __expf((float)v[i] - m);
          const float l = wave_sum(l_lane);
          if (lane == 0) wave_ml[h][wave - hl * WPH] = make_float2(m, l);
        }
        if (tok < n) {
          half_t *srow = scores + ((int64_t)b * Hq + head0 + h) * Tall;
          // consecutive positions (classes are made of 32-token blocks) and an aligned destination: one
          // vector store; otherwise 2-byte scatters through idx
          if (contig && (((uintptr_t)(srow + pos[0])) & (VPT * 2 - 1)) == 0) {
            __builtin_memcpy(__builtin_assume_aligned(srow + pos[0], VPT * 2), v, VPT * 2);
          } else {
#pragma unroll
            for (int i = 0; i < VPT; ++i)
              if (tok + i < n) srow[pos[i]] = v[i];
          }
        }
      }
      if (fz.stats) {
        __syncthreads();
        if (threadIdx.x < NREP) {
          const int h = threadIdx.x;
          float m = -INFINITY, l = 0.f;
#pragma unroll
          for (int w = 0; w < WPH; ++w) m = fmaxf(m, wave_ml[h][w].x);
#pragma unroll
          for (int w = 0; w < WPH; ++w)
            if (wave_ml[h][w].y > 0.f) l += wave_ml[h][w].y * __expf(wave_ml[h][w].x - m);
          fz.stats[((int64_t)b * Hq + head0 + h) * fz.n_stat + sg.unit_begin + tile] = make_float2(m, l);
        }
      }
    }
  };
  using Acc = float (&)[NREP][QK_TPL];
  switch (sg.bits) {
    case 1:
      if (sg.layout == HQEKV_LAYOUT_NORMAL1)
        run_tiles([&](uint32_t ts, uint32_t, Acc acc) { qk_quant_accumulate<1, NREP, QK_WAVES, true, MF>(sg, ts, bh, D, wave, stage_q, q2s, acc); });
      else
        run_tiles([&](uint32_t ts, uint32_t, Acc acc) { qk_quant_accumulate<1, NREP, QK_WAVES, false, MF>(sg, ts, bh, D, wave, stage_q, q2s, acc); });
      break;
    case 2: run_tiles([&](uint32_t ts, uint32_t, Acc acc) { qk_quant_accumulate<2, NREP, QK_WAVES, false, MF>(sg, ts, bh, D, wave, stage_q, q2s, acc); }); break;
    case 4: run_tiles([&](uint32_t ts, uint32_t, Acc acc) { qk_quant_accumulate<4, NREP, QK_WAVES, false, MF>(sg, ts, bh, D, wave, stage_q, q2s, acc); }); break;
    case 8: run_tiles([&](uint32_t ts, uint32_t, Acc acc) { qk_quant_accumulate<8, NREP, QK_WAVES, false, MF>(sg, ts, bh, D, wave, stage_q, q2s, acc); }); break;
    default: run_tiles([&](uint32_t, uint32_t t0, Acc acc) { qk_f16_cm_accumulate<NREP, QK_WAVES, MF>(sg, t0, bh, D, wave, stage_q, q2s, acc); });
  }
}

// =============================================================================== q.K^T, one wave per tile
// The tiling for launches with many tiles.  A workgroup is ONE wave that owns its tokens across all of
// head_dim: a lane keeps 8 adjacent tokens and walks the channel rows two at a time, so the sum over d never
// leaves the lane -- no partial rows parked in LDS, no workgroup barrier, no second pass over the scores.
// Per tile the wave first requests its first block of code words, then stages the query ([row pair][head]
// pairs) and the tile's scale/zero rows in LDS: the rows are fetched with wide loads (a tile's groups of one
// row are contiguous) and stored pair-interleaved -- {(s_d, s_d+1), (z_d, z_d+1)} per (row pair, group) -- so
// the inner loop reads both with one 8-byte LDS access and pairs nothing itself.
// TPL = 8 tokens per lane: tile = 512 tokens, least fixed work per code; 128 registers and 9 KB of LDS per wave
//         allow four waves per SIMD.
// TPL = 4 tokens per lane: tile = 256 tokens, half the accumulators and half the staged scale/zero rows: eight
//         waves per SIMD hide the memory latency that four leave exposed, at the price of the per-tile work
//         (query staging, statistics, stores) being spread over half as many codes.
// head_dim is 128 here; the host sends other sizes to the tilings above.
template <int TPL>
struct QwGeom {
  static constexpr int TILE = 64 * TPL;    // tokens per tile
  static constexpr int NG = TILE / 32;     // scale/zero groups per tile and row
  static constexpr int LPG = 32 / TPL;     // lanes that share a group
  static constexpr int RP = 64;            // row pairs a lane walks
  static constexpr int GPI = 8;            // groups one staging item covers (16 bytes per row)
};
__host__ __device__ constexpr int qw_tile(int tpl) { return 64 * tpl; }

__device__ __forceinline__ uint4 buf_u128(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_off, (int)row_off, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 buf_u64(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  typedef uint32_t v2u __attribute__((ext_vector_type(2)));
  const v2u v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_off, (int)row_off, 0);
  return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t buf_u8(rsrc_t r, uint32_t lane_off, uint32_t row_off) {
  return (uint32_t)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(r, (int)lane_off, (int)row_off, 0);
}

// the TPL codes of one row a lane owns: TPL * BITS bits, fetched with the narrowest load that holds them (at
// 1 bit and 4 tokens per lane two lanes share a byte and each takes its nibble)
template <int BITS, int TPL>
struct QwRow {
  uint32_t w[TPL * BITS > 32 ? 2 : 1];
};
template <int BITS, int TPL>
__device__ __forceinline__ QwRow<BITS, TPL> qw_load_row(rsrc_t rc, uint32_t lane_off, uint32_t row_off) {
  constexpr int NB = TPL * BITS;  // bits per lane and row
  QwRow<BITS, TPL> r;
  if constexpr (NB == 64) {
    const uint2 v = buf_u64(rc, lane_off, row_off);
    r.w[0] = v.x;
    r.w[1] = v.y;
  } else if constexpr (NB == 32) {
    r.w[0] = buf_u32(rc, lane_off, row_off);
  } else if constexpr (NB == 16) {
    r.w[0] = buf_u16(rc, lane_off, row_off);
  } else {
    r.w[0] = buf_u8(rc, lane_off, row_off);
  }
  return r;
}

// Stage the scale/zero rows of one tile: sz[dp * NG + g] = {(s[2dp][g], s[2dp+1][g]), (z[2dp][g], z[2dp+1][g])}.
// Groups past the end of the class read whatever follows (the next row, or zero past the slab): only lanes
// whose tokens do not exist look at them.
// Returns true when every scale this lane staged is finite and below 32 in magnitude.
template <int TPL, bool NORMAL>
__device__ __forceinline__ bool qw_stage_sz(const SegDev &sg, int tile, int bh, int lane, uint2 *sz) {
  using G = QwGeom<TPL>;
  constexpr int NG = G::NG, GPI = G::GPI;
  constexpr int ITEMS = 64 * NG / GPI;   // (row pair, part of the tile's groups)
  const uint32_t gpr = (uint32_t)(sg.n_tokens >> 5);
  const rsrc_t rs = make_rsrc(sg.scale + (int64_t)bh * 128 * gpr, 128u * gpr * 2u);
  const rsrc_t rz = make_rsrc(sg.zero + (int64_t)bh * 128 * gpr, 128u * gpr * 2u);
  const uint32_t g0 = (uint32_t)tile * NG;
  uint32_t big = 0;  // bit 15 / 31 set once an |scale| >= 32 (fp16 0x5000), an infinity or a NaN has been seen
#pragma unroll 1   // one item's sixteen registers at a time: the accumulators are live across this
  for (int k = 0; k < ITEMS / 64; ++k) {
    const int it = lane + 64 * k;
    const int dp = it / (NG / GPI), part = it % (NG / GPI);
    const uint32_t off = ((uint32_t)(2 * dp) * gpr + g0 + (uint32_t)part * GPI) * 2u;
    uint32_t sa[GPI / 2], sb[GPI / 2], za[GPI / 2], zb[GPI / 2];
    const uint32_t gb = g0 + (uint32_t)part * GPI;   // first group of this item
    if (gb + GPI > gpr) {
      // the last tile of a class: the item's window hangs over the end of the row (and, in the last row, over
      // the end of the slab, where a wide load is dropped whole).  Element loads with the group clamped.
#pragma unroll
      for (int j = 0; j < GPI / 2; ++j) {
        const uint32_t ga = min(gb + 2 * j, gpr - 1), gc = min(gb + 2 * j + 1, gpr - 1);
        const uint32_t ra = ((uint32_t)(2 * dp) * gpr + ga) * 2u, rb = ((uint32_t)(2 * dp) * gpr + gc) * 2u;
        sa[j] = buf_u16(rs, ra, 0) | (buf_u16(rs, rb, 0) << 16);
        sb[j] = buf_u16(rs, ra, gpr * 2u) | (buf_u16(rs, rb, gpr * 2u) << 16);
        za[j] = buf_u16(rz, ra, 0) | (buf_u16(rz, rb, 0) << 16);
        zb[j] = buf_u16(rz, ra, gpr * 2u) | (buf_u16(rz, rb, gpr * 2u) << 16);
      }
    } else if constexpr (GPI == 8) {
      const uint4 a = buf_u128(rs, off, 0), b = buf_u128(rs, off, gpr * 2u);
      const uint4 c = buf_u128(rz, off, 0), d = buf_u128(rz, off, gpr * 2u);
      sa[0] = a.x; sa[1] = a.y; sa[2] = a.z; sa[3] = a.w;
      sb[0] = b.x; sb[1] = b.y; sb[2] = b.z; sb[3] = b.w;
      za[0] = c.x; za[1] = c.y; za[2] = c.z; za[3] = c.w;
      zb[0] = d.x; zb[1] = d.y; zb[2] = d.z; zb[3] = d.w;
    } else {
      const uint2 a = buf_u64(rs, off, 0), b = buf_u64(rs, off, gpr * 2u);
      const uint2 c = buf_u64(rz, off, 0), d = buf_u64(rz, off, gpr * 2u);
      sa[0] = a.x; sa[1] = a.y;
      sb[0] = b.x; sb[1] = b.y;
      za[0] = c.x; za[1] = c.y;
      zb[0] = d.x; zb[1] = d.y;
    }
    uint4 *dst = reinterpret_cast<uint4 *>(sz + dp * NG + part * GPI);
#pragma unroll
    for (int j = 0; j < GPI / 2; ++j) {
      big |= ((sa[j] & 0x7fff7fffu) + 0x30003000u) | ((sb[j] & 0x7fff7fffu) + 0x30003000u);
      half2_t s_lo = half_pair<0>(sa[j], sb[j]), s_hi = half_pair<1>(sa[j], sb[j]);
      if (NORMAL) {  // the spread a = rnd16(k * std) once per group instead of once per use
        s_lo = normal1_spread(s_lo);
        s_hi = normal1_spread(s_hi);
      }
      dst[j] = make_uint4(as_u32(s_lo), as_u32(half_pair<0>(za[j], zb[j])), as_u32(s_hi), as_u32(half_pair<1>(za[j], zb[j])));
    }
  }
  return (big & 0x80008000u) == 0;
}

// Register blocks per wave (one is consumed, the others are in flight).  Deeper rings and larger blocks were measured
// on the matrix-core form (rings of 4, blocks of 1-4 KB, 2-4 waves per SIMD): no gain, the launch is not bound by the
// depth of a wave's load queue.
__host__ __device__ constexpr int qw_ring_blocks(bool) { return 2; }
__host__ __device__ constexpr int qw_rows_per_block(int nb, int tpl, bool) {
  return (nb == 64 || tpl == 4) ? 2 : 4;
}

// matrix-core form: the query is staged head-major, q2s[h * QW_QH_STRIDE + row pair], so that a lane reads the four (or
// two) row pairs of a register block for its head, lane % 4, with one LDS access; the stride keeps the four heads' reads
// in distinct banks and 16-byte aligned
constexpr int QW_QH_STRIDE = 68;

template <int BITS, int NREP, int TPL, bool NORMAL, bool MF, typename Stage>
__device__ __forceinline__ void qw_quant_accumulate(const SegDev &sg, uint32_t ts, int bh, int lane, Stage &&stage,
                                                    const half2_t *q2s, const uint2 *sz, float (&acc)[NREP][TPL]) {
  static_assert(!MF || NREP == 4, "the matrix-core form is a 4-head product");
  using G = QwGeom<TPL>;
  using Row = QwRow<BITS, TPL>;
  constexpr int NB = TPL * BITS;                    // bits per lane and row
  // row pairs per register block (two blocks of loads are in flight): short blocks where registers are scarce --
  // the wide rows of the 8-bit class, and the 256-token tile, whose extra waves hide latency instead.
  constexpr int U = qw_rows_per_block(NB, TPL, MF);
  const uint32_t n = (uint32_t)sg.n_tokens;
  const uint32_t rowb = n / 8u * BITS;              // bytes per channel row
  const uint32_t lane_off = ts * BITS / 8u;         // (two lanes share a byte when a lane owns 4 bits)
  const int nib = (NB == 4) ? (int)(ts & 4u) : 0;   // ... and the odd one takes the upper nibble
  const rsrc_t rc = make_rsrc((const char *)sg.data + (int64_t)bh * 128 * rowb, 128u * rowb);
  const uint2 *sp = sz + lane / G::LPG;
  struct Block {
    Row r0[U], r1[U];
  };
  auto load = [&](int i0, Block &b) {
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t row = (uint32_t)(2 * (i0 + k)) * rowb;  // uniform
      b.r0[k] = qw_load_row<BITS, TPL>(rc, lane_off, row);
      b.r1[k] = qw_load_row<BITS, TPL>(rc, lane_off, row + rowb);
    }
  };
  f4_t av[TPL];  // matrix-core form: (4 heads) per token of this lane
#pragma unroll
  for (int i = 0; i < TPL; ++i) av[i] = (f4_t){0.f, 0.f, 0.f, 0.f};
  const half2_t *qh = q2s + (lane & 3) * QW_QH_STRIDE;  // the head whose query this lane supplies
  auto compute_mf = [&](int i0, const Block &b, auto fused_bias) {
    constexpr bool FB = decltype(fused_bias)::value;
    constexpr int FPB = 8 / BITS;                 // codes per byte
    constexpr int NBYTE = (NB + 7) / 8;           // bytes per lane and row
    constexpr int NF = NB < 8 ? NB / BITS : FPB;  // codes taken from a byte
    half2_t qa[U];
#pragma unroll
    for (int k = 0; k < U; k += 4) {
      if constexpr (U % 4 == 0) {
        const uint4 v = *reinterpret_cast<const uint4 *>(qh + i0 + k);
        qa[k] = as_h2(v.x); qa[k + 1] = as_h2(v.y); qa[k + 2] = as_h2(v.z); qa[k + 3] = as_h2(v.w);
      } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(qh + i0 + k);
        qa[k] = as_h2(v.x); qa[k + 1] = as_h2(v.y);
      }
    }
#pragma unroll
    for (int k = 0; k < U; k += 2) {   // two row pairs = four channels per matrix product
      const uint2 sza = sp[(i0 + k) * G::NG], szb = sp[(i0 + k + 1) * G::NG];
      const half2_t sa = as_h2(sza.x), za = as_h2(sza.y), sb = as_h2(szb.x), zb = as_h2(szb.y);
      half2_t nba[FPB], nbb[FPB];
      if constexpr (FB) {
        static_for<NF>([&](auto I_) {
          constexpr int I = decltype(I_)::value;
          nba[I] = bias_times_scale<BITS, I>(sa);
          nbb[I] = bias_times_scale<BITS, I>(sb);
        });
      }
#pragma unroll
      for (int j = 0; j < NBYTE; ++j) {
        uint32_t a0 = b.r0[k].w[j / 4], a1 = b.r1[k].w[j / 4], c0 = b.r0[k + 1].w[j / 4], c1 = b.r1[k + 1].w[j / 4];
        if (NB == 4) {
          a0 >>= nib; a1 >>= nib; c0 >>= nib; c1 >>= nib;
        }
        const uint32_t ua = byte_pair_at(a0, a1, j % 4), ub = byte_pair_at(c0, c1, j % 4);
        if constexpr (FB) consume_bytes_mfma_fused_bias<BITS, NF, TPL>(ua, ub, sa, za, sb, zb, nba, nbb, qa[k], qa[k + 1], av, j * FPB);
        else consume_bytes_mfma<BITS, NORMAL, NF, TPL>(ua, ub, sa, za, sb, zb, qa[k], qa[k + 1], av, j * FPB);
      }
    }
  };
  auto compute_valu = [&](int i0, const Block &b, auto fused_bias) {
    constexpr bool FB = decltype(fused_bias)::value;
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int i = i0 + k;
      half2_t q2[NREP];
#pragma unroll
      for (int h = 0; h < NREP; ++h) q2[h] = q2s[i * NREP + h];
      const uint2 szv = sp[i * G::NG];
      const half2_t s2 = as_h2(szv.x), z2 = as_h2(szv.y);
      constexpr int FPB = 8 / BITS;                 // codes per byte
      constexpr int NBYTE = (NB + 7) / 8;           // bytes per lane and row
      constexpr int NF = NB < 8 ? NB / BITS : FPB;  // codes taken from a byte
      half2_t nb[FPB];
      if constexpr (FB) {   // -2^(10-pos) * s for every field position, once per row pair
#define HQ_NB(I_) \
  if constexpr (I_ < NF) nb[I_ < FPB ? I_ : 0] = bias_times_scale<BITS, (I_ < FPB ? I_ : 0)>(s2);
        HQ_NB(0) HQ_NB(1) HQ_NB(2) HQ_NB(3) HQ_NB(4) HQ_NB(5) HQ_NB(6) HQ_NB(7)
#undef HQ_NB
      }
#pragma unroll
      for (int j = 0; j < NBYTE; ++j) {
        uint32_t a0 = b.r0[k].w[j / 4], a1 = b.r1[k].w[j / 4];
        if (NB == 4) {
          a0 >>= nib;
          a1 >>= nib;
        }
        const uint32_t u = (j % 4 == 0)   ? byte_pair<0>(a0, a1)
                           : (j % 4 == 1) ? byte_pair<1>(a0, a1)
                           : (j % 4 == 2) ? byte_pair<2>(a0, a1)
                                          : byte_pair<3>(a0, a1);
        if constexpr (FB) consume_byte_fused_bias<BITS, NREP, TPL, NF>(u, s2, z2, nb, q2, acc, j * FPB);
        else consume_byte<BITS, NREP, TPL, NORMAL, NF>(u, s2, z2, q2, acc, j * FPB);
      }
    }
  };
  auto compute = [&](int i0, const Block &b, auto fused_bias) {
    if constexpr (MF) compute_mf(i0, b, fused_bias);
    else compute_valu(i0, b, fused_bias);
  };
  // A ring of NBLK register blocks: block b is requested NBLK - 1 blocks of arithmetic before it is consumed.
  constexpr int NBLK = qw_ring_blocks(MF);
  static_assert(G::RP % (NBLK * U) == 0, "the ring loop covers the row pairs exactly");
  Block ring[NBLK];
#pragma unroll
  for (int j = 0; j < NBLK - 1; ++j) load(j * U, ring[j]);   // in flight across the staging
  // Query and scale/zero into LDS; the staging also says whether every scale of the tile is small enough for the
  // multiply that removes the bias on the way (one packed op fewer per pair of codes).  Worth it where a lane has
  // more codes per row pair than field positions: 8, 4 and 2 bits.
  const bool small_scales = stage();
  auto finish = [&]() {
    if constexpr (MF) {
#pragma unroll
      for (int h = 0; h < NREP; ++h)
#pragma unroll
        for (int i = 0; i < TPL; ++i) acc[h][i] = av[i][h];
    }
  };
  auto run = [&](auto fused_bias) {
#pragma unroll 1
    for (int i0 = 0; i0 < G::RP; i0 += NBLK * U) {
#pragma unroll
      for (int j = 0; j < NBLK; ++j) {
        const int nxt = i0 + (j + NBLK - 1) * U;   // the block whose turn it is NBLK - 1 blocks from now
        if (nxt < G::RP) load(nxt, ring[(j + NBLK - 1) % NBLK]);   // uniform
        HQ_LOADS_ABOVE();
        compute(i0 + j * U, ring[j], fused_bias);
      }
    }
  };
  if constexpr (!NORMAL && BITS != 1) {
    if (__builtin_amdgcn_ballot_w64(!small_scales) == 0) {
      run(std::true_type{});
      finish();
      return;
    }
  }
  run(std::false_type{});
  finish();
}

// fp16 class stored channel-major (B,Hkv,128,T), T a multiple of 8: a lane reads its TPL tokens of a row as 16 or 8 bytes
template <int NREP, int TPL, bool MF, typename Stage>
__device__ __forceinline__ void qw_f16_accumulate(const SegDev &sg, uint32_t ts, int bh, int lane, Stage &&stage,
                                                  const half2_t *q2s, float (&acc)[NREP][TPL]) {
  static_assert(!MF || NREP == 4, "the matrix-core form is a 4-head product");
  using G = QwGeom<TPL>;
  constexpr int U = 2, NW = TPL / 2;   // words per lane and row
  const uint32_t n = (uint32_t)sg.n_tokens;
  const uint32_t rowb = n * 2u;
  const uint32_t lane_off = ts * 2u;
  const rsrc_t rc = make_rsrc((const char *)sg.data + (int64_t)bh * 128 * rowb, 128u * rowb);
  struct Block {
    uint32_t r0[U][NW], r1[U][NW];
  };
  auto load_row = [&](uint32_t row, uint32_t (&w)[NW]) {
    if constexpr (NW == 4) {
      const uint4 v = buf_u128(rc, lane_off, row);
      w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else {
      const uint2 v = buf_u64(rc, lane_off, row);
      w[0] = v.x; w[1] = v.y;
    }
  };
  auto load = [&](int i0, Block &b) {
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t row = (uint32_t)(2 * (i0 + k)) * rowb;
      load_row(row, b.r0[k]);
      load_row(row + rowb, b.r1[k]);
    }
  };
  f4_t av[TPL];
#pragma unroll
  for (int i = 0; i < TPL; ++i) av[i] = (f4_t){0.f, 0.f, 0.f, 0.f};
  const half2_t *qh = q2s + (lane & 3) * QW_QH_STRIDE;
  auto compute = [&](int i0, const Block &b) {
    if constexpr (MF) {   // the block's two row pairs = four channels per matrix product
      static_assert(U == 2, "one matrix product per token and block");
      const uint2 qv = *reinterpret_cast<const uint2 *>(qh + i0);
      const half2_t qa = as_h2(qv.x), qb = as_h2(qv.y);
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        av[2 * i] = mfma_4x4x4(qa, qb, half_pair<0>(b.r0[0][i], b.r1[0][i]), half_pair<0>(b.r0[1][i], b.r1[1][i]), av[2 * i]);
        av[2 * i + 1] = mfma_4x4x4(qa, qb, half_pair<1>(b.r0[0][i], b.r1[0][i]), half_pair<1>(b.r0[1][i], b.r1[1][i]), av[2 * i + 1]);
      }
    } else {
#pragma unroll
      for (int k = 0; k < U; ++k) {
        half2_t q2[NREP];
#pragma unroll
        for (int h = 0; h < NREP; ++h) q2[h] = q2s[(i0 + k) * NREP + h];
#pragma unroll
        for (int i = 0; i < NW; ++i) {
          const half2_t ka = half_pair<0>(b.r0[k][i], b.r1[k][i]);  // token 2i:   (k[d], k[d+1])
          const half2_t kb = half_pair<1>(b.r0[k][i], b.r1[k][i]);  // token 2i+1
#pragma unroll
          for (int h = 0; h < NREP; ++h) {
            acc[h][2 * i] = __builtin_amdgcn_fdot2(ka, q2[h], acc[h][2 * i], false);
            acc[h][2 * i + 1] = __builtin_amdgcn_fdot2(kb, q2[h], acc[h][2 * i + 1], false);
          }
        }
      }
    }
  };
  constexpr int NBLK = qw_ring_blocks(MF);
  static_assert(G::RP % (NBLK * U) == 0, "the ring loop covers the row pairs exactly");
  Block ring[NBLK];
#pragma unroll
  for (int j = 0; j < NBLK - 1; ++j) load(j * U, ring[j]);
  stage();
#pragma unroll 1
  for (int i0 = 0; i0 < G::RP; i0 += NBLK * U) {
#pragma unroll
    for (int j = 0; j < NBLK; ++j) {
      const int nxt = i0 + (j + NBLK - 1) * U;
      if (nxt < G::RP) load(nxt, ring[(j + NBLK - 1) % NBLK]);   // uniform
      HQ_LOADS_ABOVE();
      compute(i0 + j * U, ring[j]);
    }
  }
  if constexpr (MF) {
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int i = 0; i < TPL; ++i) acc[h][i] = av[i][h];
  }
}

template <int NREP, int TPL, bool MF = false>
__global__ __launch_bounds__(64, NREP <= 4 ? (TPL == 8 ? 4 : 6) : 2) void qk_wave_kernel(SegTable tb, const half_t *__restrict__ q,
                                                                              half_t *__restrict__ scores, int hq_slice, int Hkv,
                                                                              int64_t Tall, FuseArgs fz) {
  using G = QwGeom<TPL>;
  // [row pair][head]: (q[d], q[d+1]); matrix-core form: [head][row pair], QW_QH_STRIDE pairs per head
  __shared__ __align__(16) half2_t q2s[MF ? NREP * QW_QH_STRIDE : 64 * NREP];
  __shared__ __align__(16) uint2 sz[64 * G::NG];      // [row pair][group]: {(s_d, s_d+1), (z_d, z_d+1)}
  __shared__ float red[2 * NREP];
  const int lane = threadIdx.x;
  const int bh = blockIdx.x;
  const int b = bh / Hkv, hkv = bh % Hkv;
  const int Hq = hq_slice & 0xffff, head0 = first_head(hq_slice, hkv);
  if (fz.arrive && blockIdx.y == 0 && lane == 0) fz.arrive[bh] = 0;  // for the p.V launch that follows
  const int si = seg_of_unit(tb, blockIdx.y);
  const SegDev sg = tb.seg[si];
  const int tile = (int)blockIdx.y - begin_of_seg(tb, si);

  const uint32_t *qsrc = reinterpret_cast<const uint32_t *>(q + ((int64_t)b * Hq + head0) * 128);
  auto stage_q_pairs = [&]() {
#pragma unroll
    for (int h = 0; h < NREP; ++h) q2s[lane * NREP + h] = as_h2(qsrc[h * 64 + lane]);
  };
  auto stage_q = [&]() {
    if constexpr (MF) {
#pragma unroll
      for (int h = 0; h < NREP; ++h) q2s[h * QW_QH_STRIDE + lane] = as_h2(qsrc[h * 64 + lane]);
    } else {
      stage_q_pairs();
    }
  };
  if (sg.bits == 16 && sg.layout == HQEKV_LAYOUT_TOKEN_MAJOR) {
    stage_q_pairs();
    __syncthreads();
    qk_f16_tm_tile<NREP, 1>(sg, tile, bh, b, head0, 128, Hq, Tall, 0, lane, q2s, scores, fz, red);
    return;
  }
  const uint32_t n = (uint32_t)sg.n_tokens;
  const uint32_t t0 = (uint32_t)tile * G::TILE + (uint32_t)lane * TPL;
  const bool valid = t0 < n;           // class lengths are multiples of 8: a lane's tokens exist or do not
  const uint32_t ts = valid ? t0 : 0;  // lanes past the end recompute the first tokens and store nothing
  float acc[NREP][TPL];
#pragma unroll
  for (int h = 0; h < NREP; ++h)
#pragma unroll
    for (int i = 0; i < TPL; ++i) acc[h][i] = 0.f;

  auto stage_quant = [&](auto normal) {
    stage_q();
    const bool small_scales = qw_stage_sz<TPL, decltype(normal)::value>(sg, tile, bh, lane, sz);
    __syncthreads();
    return small_scales && !fz.two_step;
  };
  auto stage_plain = [&]() {
    stage_q();
    __syncthreads();
  };
  using T = std::true_type;
  using F = std::false_type;
  switch (sg.bits) {
    case 1:
      if (sg.layout == HQEKV_LAYOUT_NORMAL1)
        qw_quant_accumulate<1, NREP, TPL, true, MF>(sg, ts, bh, lane, [&]() { return stage_quant(T{}); }, q2s, sz, acc);
      else
        qw_quant_accumulate<1, NREP, TPL, false, MF>(sg, ts, bh, lane, [&]() { return stage_quant(F{}); }, q2s, sz, acc);
      break;
    case 2: qw_quant_accumulate<2, NREP, TPL, false, MF>(sg, ts, bh, lane, [&]() { return stage_quant(F{}); }, q2s, sz, acc); break;
    case 4: qw_quant_accumulate<4, NREP, TPL, false, MF>(sg, ts, bh, lane, [&]() { return stage_quant(F{}); }, q2s, sz, acc); break;
    case 8: qw_quant_accumulate<8, NREP, TPL, false, MF>(sg, ts, bh, lane, [&]() { return stage_quant(F{}); }, q2s, sz, acc); break;
    default: qw_f16_accumulate<NREP, TPL, MF>(sg, ts, bh, lane, stage_plain, q2s, acc);
  }

  // positions of the lane's tokens (they index a row of Tall < 2^31 scores, so the low word of each int64 entry
  // is enough); requested here, used after the conversions below
  uint32_t pos[TPL];
  if (sg.idx) {
    const uint4 *ip = reinterpret_cast<const uint4 *>(sg.idx + ts);
#pragma unroll
    for (int i = 0; i < TPL / 2; ++i) {
      const uint4 v = ip[i];
      pos[2 * i] = v.x;
      pos[2 * i + 1] = v.z;
    }
  } else {
#pragma unroll
    for (int i = 0; i < TPL; ++i) pos[i] = (uint32_t)sg.pos_base + ts + i;
  }
  bool contig = true;
#pragma unroll
  for (int i = 1; i < TPL; ++i) contig = contig && (pos[i] == pos[0] + i);
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
    half_t v[TPL];
    float m_lane = -INFINITY;
#pragma unroll
    for (int i = 0; i < TPL; ++i) {
      v[i] = (half_t)acc[h][i];
      if (fz.stats) {  // the fp16 steps of the reference epilogue: round the score, scale, round again
        v[i] = (half_t)((float)v[i] * fz.inv_sqrt_d);
        m_lane = fmaxf(m_lane, (float)v[i]);
      }
    }
    if (fz.stats) {  // (max, sum exp) of the tile
      if (!valid) m_lane = -INFINITY;
      const float m = wave_max(m_lane);
      float l_lane = 0.f;
#pragma unroll
      for (int i = 0; i < TPL; ++i) l_lane += __expf((float)v[i] - m);
      if (!valid) l_lane = 0.f;
      const float l = wave_sum(l_lane);
      if (lane == 0)
        fz.stats[((int64_t)b * Hq + head0 + h) * fz.n_stat + sg.unit_begin + tile] = make_float2(m, l);
    }
    if (valid) {
      half_t *srow = scores + ((int64_t)b * Hq + head0 + h) * Tall;
      // consecutive positions (classes are made of 32-token blocks) and an aligned destination: one vector
      // store; otherwise 2-byte scatters through idx
      if (contig && (((uintptr_t)(srow + pos[0])) & (2 * TPL - 1)) == 0) {
        __builtin_memcpy(__builtin_assume_aligned(srow + pos[0], 2 * TPL), v, 2 * TPL);
      } else {
#pragma unroll
        for (int i = 0; i < TPL; ++i) srow[pos[i]] = v[i];
      }
    }
  }
}

// =============================================================================== softmax
constexpr int SM_THREADS = 1024;

__device__ __forceinline__ float block_reduce(float v, float *sh, bool is_max) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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

// Generic three-pass kernel: any row length, scalar accesses.
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

// Register-resident kernel: the row is read once with 128-bit accesses aligned to memory (a row of
// odd length does not start on a 16-byte boundary, so vector j covers elements [8j-off, 8j-off+8) and
// the two edge vectors fall back to predicated scalar accesses), kept as fp16 logits in registers for
// the max / sum / normalise passes, and written once.  NV <= 8 vectors per thread cover up to 65536 elements;
// longer rows take the generic kernel.
template <int NV>
__global__ __launch_bounds__(SM_THREADS) void scale_softmax_reg_kernel(half_t *__restrict__ scores,
                                                                       const half_t *__restrict__ mask,
                                                                       int64_t mask_row_stride, int64_t Tall,
                                                                       float inv) {
  __shared__ float sh[SM_THREADS / 64];
  half_t *row = scores + (int64_t)blockIdx.x * Tall;
  const half_t *mrow = mask ? mask + (int64_t)blockIdx.x * mask_row_stride : nullptr;
  const int off = (int)(((uintptr_t)row >> 1) & 7);  // elements between the previous 16-byte boundary and row[0]
  half_t x[NV][8];
  float m = -INFINITY;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t e0 = ((int64_t)k * SM_THREADS + threadIdx.x) * 8 - off;  // first element of this vector
    if (e0 >= 0 && e0 + 8 <= Tall) {
      const uint4 raw = *reinterpret_cast<const uint4 *>(row + e0);
      __builtin_memcpy(x[k], &raw, 16);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[k][i] = (e0 + i >= 0 && e0 + i < Tall) ? row[e0 + i] : (half_t)0;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t t = e0 + i;
      if (t >= 0 && t < Tall) {
        half_t v = (half_t)((float)x[k][i] * inv);
        if (mrow) v = (half_t)((float)v + (float)mrow[t]);
        v = (half_t)fmaxf((float)v, -65504.0f);
        x[k][i] = v;
        m = fmaxf(m, (float)v);
      }
    }
  }
  m = block_reduce(m, sh, true);
  // exp(x - m) is evaluated once (hardware exp2; its error is far below one fp16 ulp of the result)
  // and kept in registers for the normalisation
  float e[NV][8];
  float l = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t e0 = ((int64_t)k * SM_THREADS + threadIdx.x) * 8 - off;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool in = e0 + i >= 0 && e0 + i < Tall;
      e[k][i] = in ? __expf((float)x[k][i] - m) : 0.f;
      l += e[k][i];
    }
  }
  l = block_reduce(l, sh, false);
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t e0 = ((int64_t)k * SM_THREADS + threadIdx.x) * 8 - off;
    if (e0 >= Tall || e0 + 8 <= 0) continue;
    half_t y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (half_t)(e[k][i] * inv_l);
    if (e0 >= 0 && e0 + 8 <= Tall) {
      uint4 raw;
      __builtin_memcpy(&raw, y, 16);
      *reinterpret_cast<uint4 *>(row + e0) = raw;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (e0 + i >= 0 && e0 + i < Tall) row[e0 + i] = y[i];
    }
  }
}

// =============================================================================== p.V
constexpr int CB_CH = 32;      // combine: channels per workgroup
constexpr int CB_SLICES = 32;  // combine: chunk slices, slice s adds chunks s, s + 32, ...
constexpr int CB_FOLD_MAX = 64;  // most chunks per (b, kv head) the last p.V workgroup adds up itself
constexpr int64_t CB_FOLD_MIN_TOKEN_ROWS = 2 << 20;  // ... and the least V token rows (tokens x B x Hkv) for which it pays
constexpr int PV_THREADS = 256;
constexpr int PV_WAVES = 4;
constexpr int PV_CPL = 8;                        // channels per lane
constexpr int PV_BLOCK = 512;                    // tokens staged in LDS at a time (256 token pairs)
constexpr int PV_UNR = 4;                        // word pairs per lane in flight together (steps = 4 / words per token)
#ifndef HQ_PV_MF_UNR
#define HQ_PV_MF_UNR 4                           // the same for the matrix-core form
#endif

// LDS block, pair-interleaved: per token pair {s2, z2} for each of the D/32 groups and p2 for each
// query head, so one 8-byte and one 4*NREP-byte LDS read feed a whole step of a lane.
template <int NREP, int NG>
struct PvStage {
  uint2 sz[PV_BLOCK / 2][NG];
  half2_t p2[PV_BLOCK / 2][NREP];
};

// What thread t fetches for token pair t of a 512-token block: positions, the two logits/probabilities
// of every query head, and the pair's scale/zero rows.  Fetching and committing are separate so that the
// requests of the next block (and of the first block, at kernel start) overlap with other work.
template <int NREP, int NG>
struct PvPair {
  int64_t pa, pb;        // positions of the pair's tokens
  int64_t ta;            // token a inside the class; token b is `second` rows on (0: there is none, a is read twice)
  int32_t second;
  half_t va[NREP], vb[NREP];
  uint2 sa, sb, za, zb;  // 4 fp16 scales / zeros of token a and of token b (NG == 4)
  bool valid, has_b;
};

// The fetch has two dependent halves -- the positions, then what sits at the positions -- so that a caller with
// something else to wait for can put it between them.
template <int NREP, int NG>
__device__ __forceinline__ void pv_fetch_positions(const SegDev &sg, int64_t t0, int nt, PvPair<NREP, NG> &pr) {
  const int tp = threadIdx.x;
  pr.valid = 2 * tp < nt;
  pr.has_b = 2 * tp + 1 < nt;
  pr.ta = t0 + (pr.valid ? 2 * tp : 0);
  pr.second = pr.has_b ? 1 : 0;
  pr.pa = sg.pos_base + pr.ta;
  pr.pb = pr.pa + pr.second;
  if (sg.idx) {
    pr.pa = sg.idx[pr.ta];
    pr.pb = sg.idx[pr.ta + pr.second];
  }
}

template <int NREP, int NG, bool QUANT>
__device__ __forceinline__ void pv_fetch_values(const SegDev &sg, int bh, half_t *const (&prow)[NREP],
                                                PvPair<NREP, NG> &pr) {
  static_assert(NG == 4, "a token's scale row is read as one 8-byte load");
  if (QUANT) {  // a V class may hold any number of tokens: the last pair of an odd count reads row a twice
    const uint2 *sc = reinterpret_cast<const uint2 *>(sg.scale + ((int64_t)bh * sg.slab_tokens + pr.ta) * NG);
    const uint2 *zr = reinterpret_cast<const uint2 *>(sg.zero + ((int64_t)bh * sg.slab_tokens + pr.ta) * NG);
    pr.sa = sc[0];
    pr.sb = sc[pr.second];
    pr.za = zr[0];
    pr.zb = zr[pr.second];
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
    pr.va[h] = prow[h][pr.pa];
    pr.vb[h] = prow[h][pr.pb];
  }
}

template <int NREP, int NG, bool QUANT>
__device__ __forceinline__ void pv_fetch(const SegDev &sg, int64_t t0, int nt, int bh, half_t *const (&prow)[NREP],
                                         PvPair<NREP, NG> &pr) {
  pv_fetch_positions<NREP, NG>(sg, t0, nt, pr);
  pv_fetch_values<NREP, NG, QUANT>(sg, bh, prow, pr);
}

template <int NREP, int NG, bool QUANT, bool ZERO_FILL = false>
__device__ __forceinline__ void pv_commit(const PvPair<NREP, NG> &pr, half_t *const (&prow)[NREP],
                                          PvStage<NREP, NG> &st, bool fused, const float *sm_ml) {
  const int tp = threadIdx.x;
  if (!pr.valid) {
    // The matrix-core form runs whole step blocks without looking at the pair count: a pair that does not exist
    // carries p = 0 and scale = zero = 0, so whatever code words its lanes hold turn into exact zeros.
    if (ZERO_FILL) {
#pragma unroll
      for (int h = 0; h < NREP; ++h) st.p2[tp][h] = pack_h2((half_t)0, (half_t)0);
      if (QUANT) {
#pragma unroll
        for (int g = 0; g < NG; ++g) st.sz[tp][g] = make_uint2(0u, 0u);
      }
    }
    return;
  }
  half_t va[NREP], vb[NREP];
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
    va[h] = pr.va[h];
    vb[h] = pr.vb[h];
  }
  if (fused) {
    // the row holds scaled logits: p = rnd16(exp(x - M) / L), written back for the caller.  Every
    // position belongs to exactly one token of exactly one V class, so nobody else touches it.
#pragma unroll
    for (int h = 0; h < NREP; ++h) {
      const float M = sm_ml[2 * h], invL = sm_ml[2 * h + 1];
      va[h] = (half_t)(__expf((float)va[h] - M) * invL);
      vb[h] = (half_t)(__expf((float)vb[h] - M) * invL);
      prow[h][pr.pa] = va[h];
      if (pr.has_b) prow[h][pr.pb] = vb[h];
    }
  }
#pragma unroll
  for (int h = 0; h < NREP; ++h) st.p2[tp][h] = pack_h2(va[h], pr.has_b ? vb[h] : (half_t)0);
  if (QUANT) {
    // (s_a[g], s_b[g]) pairs: halves 2g of the two rows
    const uint32_t sa[2] = {pr.sa.x, pr.sa.y}, sb[2] = {pr.sb.x, pr.sb.y};
    const uint32_t za[2] = {pr.za.x, pr.za.y}, zb[2] = {pr.zb.x, pr.zb.y};
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      uint2 v;
      v.x = (g & 1) ? as_u32(half_pair<1>(sa[g >> 1], sb[g >> 1])) : as_u32(half_pair<0>(sa[g >> 1], sb[g >> 1]));
      v.y = (g & 1) ? as_u32(half_pair<1>(za[g >> 1], zb[g >> 1])) : as_u32(half_pair<0>(za[g >> 1], zb[g >> 1]));
      st.sz[tp][g] = v;
    }
  }
}

// One class chunk.  16 lanes cover a token row (8 channels each: a byte of a packed word at 1 bit, half a
// word at 2 bits, one word at 4 bits, two words at 8 bits, 16 bytes of fp16), 4 token pairs per wave step, so the reduction over
// tokens needs only two butterfly steps across lanes.  Code words are requested one step-block ahead of
// their use, and the staging requests of a block are issued before the previous block is consumed.
template <int BITS, int NREP, int D, bool NORMAL = false, bool MF = false>
__device__ __forceinline__ void pv_chunk(const SegDev &sg, int64_t c0, int64_t c1, int bh, int wave, int lane,
                                         half_t *const (&prow)[NREP], PvStage<NREP, D / 32> &st,
                                         float (&acc)[NREP][PV_CPL], bool fused, const float *sm_ml,
                                         const PvPair<NREP, D / 32> &first) {
  static_assert(D == 128, "16 lanes x 8 channels cover one token row");
  static_assert(!MF || NREP == 4, "the matrix-core form is a 4-head product");
  constexpr int NG = D / 32;
  constexpr bool QUANT = BITS != 16;
  constexpr int WPL = BITS == 16 ? 4 : (BITS == 8 ? 2 : 1);  // 32-bit words per lane per token
  constexpr int ROWB = D * BITS / 8;                          // bytes per token row
  // wave steps per block: 8 words in flight per lane; the matrix-core form takes two token pairs (steps) per product
  // and, its arithmetic no longer hiding the memory latency, keeps more words in flight
  // (fp16 rows fill a lane's registers with one token pair per step: there a product takes one pair and two zeros)
  constexpr int UNR = MF ? ((HQ_PV_MF_UNR / WPL < 1) ? 1 : HQ_PV_MF_UNR / WPL) : PV_UNR / WPL;
  const int cl = lane & 15, tl = lane >> 4;
  const int g = cl >> 2;
  const int sh2 = (BITS == 2) ? (cl & 1) * 16 : (BITS == 1) ? (cl & 3) * 8 : 0;
  const uint32_t wofs = (BITS == 1 ? (cl >> 2) : BITS == 2 ? (cl >> 1) : cl * WPL) * 4u;  // byte offset inside a token row
  const rsrc_t rc = make_rsrc((const char *)sg.data + (int64_t)bh * sg.slab_tokens * ROWB,
                              (uint32_t)(sg.n_tokens * ROWB));
  const uint32_t lane_off = (uint32_t)(2 * tl) * ROWB + wofs;   // this lane's first token of a step + word

  struct Words {
    uint32_t w0[UNR][WPL], w1[UNR][WPL];
  };
  // the step-block starting at wave step s0 of the 512-token block at t0 (uniform offsets in scalars)
  auto load_steps = [&](int64_t t0, int nt, int s0, Words &r) {
#pragma unroll
    for (int k = 0; k < UNR; ++k) {
      const uint32_t tok = (uint32_t)(t0 + 8 * ((s0 + k) * PV_WAVES + wave));  // uniform: first token of the step
      const bool odd_tail = (int)(8 * ((s0 + k) * PV_WAVES + wave) + 2 * tl + 1) >= nt;  // pair without a second token
      const uint32_t row = tok * ROWB;
#pragma unroll
      for (int j = 0; j < WPL; ++j) {
        r.w0[k][j] = buf_u32(rc, lane_off + 4 * j, row);
        r.w1[k][j] = buf_u32(rc, lane_off + (odd_tail ? 0u : (uint32_t)ROWB) + 4 * j, row);
      }
    }
  };

  f4_t av[PV_CPL];  // matrix-core form: (4 heads) per channel of this lane
#pragma unroll
  for (int i = 0; i < PV_CPL; ++i) av[i] = (f4_t){0.f, 0.f, 0.f, 0.f};
  PvPair<NREP, NG> pr = first;   // the first block's positions were requested at the top of the kernel
  Words cur;
  {
    const int nt0 = (int)min((int64_t)PV_BLOCK, c1 - c0);
    pv_fetch_values<NREP, NG, QUANT>(sg, bh, prow, pr);
    load_steps(c0, nt0, 0, cur);
  }
  for (int64_t t0 = c0; t0 < c1; t0 += PV_BLOCK) {
    const int nt = (int)min((int64_t)PV_BLOCK, c1 - t0);
    const int ntp = (nt + 1) >> 1;
    const int nsteps = (ntp + 4 * PV_WAVES - 1) / (4 * PV_WAVES);
    const bool more = t0 + PV_BLOCK < c1;
    const int nt_next = more ? (int)min((int64_t)PV_BLOCK, c1 - t0 - PV_BLOCK) : 0;
    __syncthreads();  // previous block fully consumed (and sm_ml published)
    pv_commit<NREP, NG, QUANT, MF>(pr, prow, st, fused, sm_ml);
    if (more) pv_fetch<NREP, NG, QUANT>(sg, t0 + PV_BLOCK, nt_next, bh, prow, pr);
    __syncthreads();
#pragma unroll 1
    for (int s0 = 0; s0 < nsteps; s0 += UNR) {
      Words nxt;
      if (s0 + UNR < nsteps) load_steps(t0, nt, s0 + UNR, nxt);
      else if (more) load_steps(t0 + PV_BLOCK, nt_next, 0, nxt);
      HQ_LOADS_ABOVE();
      if constexpr (MF && UNR == 1) {
        // one token pair per step block (fp16 rows): the product's other two tokens are zeros
        static_assert(!(MF && UNR == 1) || BITS == 16, "only fp16 rows have single-pair step blocks");
        const int tpa = 4 * (s0 * PV_WAVES + wave) + tl;
        const half2_t pa = st.p2[tpa][lane & 3], zero2 = (half2_t){(_Float16)0, (_Float16)0};
#pragma unroll
        for (int j = 0; j < (BITS == 16 ? 4 : 0); ++j) {
          av[2 * j] = mfma_4x4x4(pa, zero2, half_pair<0>(cur.w0[0][j], cur.w1[0][j]), zero2, av[2 * j]);
          av[2 * j + 1] = mfma_4x4x4(pa, zero2, half_pair<1>(cur.w0[0][j], cur.w1[0][j]), zero2, av[2 * j + 1]);
        }
      } else if constexpr (MF) {
        // two token pairs = four tokens per matrix product; pairs past the end of the block were staged as zeros
#pragma unroll
        for (int k = 0; k + 1 < UNR; k += 2) {
          const int tpa = 4 * ((s0 + k) * PV_WAVES + wave) + tl, tpb = tpa + 4 * PV_WAVES;
          const half2_t pa = st.p2[tpa][lane & 3], pb = st.p2[tpb][lane & 3];
          if constexpr (BITS == 16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              av[2 * j] = mfma_4x4x4(pa, pb, half_pair<0>(cur.w0[k][j], cur.w1[k][j]),
                                     half_pair<0>(cur.w0[k + 1][j], cur.w1[k + 1][j]), av[2 * j]);
              av[2 * j + 1] = mfma_4x4x4(pa, pb, half_pair<1>(cur.w0[k][j], cur.w1[k][j]),
                                         half_pair<1>(cur.w0[k + 1][j], cur.w1[k + 1][j]), av[2 * j + 1]);
            }
          } else {
            const uint2 sza = st.sz[tpa][g], szb = st.sz[tpb][g];
            half2_t sa = as_h2(sza.x), sb = as_h2(szb.x);
            const half2_t za = as_h2(sza.y), zb = as_h2(szb.y);
            if (NORMAL) {
              sa = normal1_spread(sa);
              sb = normal1_spread(sb);
            }
            constexpr int FPB = 8 / BITS;
            constexpr int NBYTE = BITS;   // bytes that hold a lane's 8 channels of one token
#pragma unroll
            for (int j = 0; j < NBYTE; ++j) {
              const uint32_t ua = byte_pair_at(cur.w0[k][j / 4] >> sh2, cur.w1[k][j / 4] >> sh2, j % 4);
              const uint32_t ub = byte_pair_at(cur.w0[k + 1][j / 4] >> sh2, cur.w1[k + 1][j / 4] >> sh2, j % 4);
              consume_bytes_mfma<BITS, NORMAL, FPB, PV_CPL>(ua, ub, sa, za, sb, zb, pa, pb, av, j * FPB);
            }
          }
        }
      } else {
#pragma unroll
      for (int k = 0; k < UNR; ++k) {
        const int tp = 4 * ((s0 + k) * PV_WAVES + wave) + tl;
        if (tp < ntp) {
          half2_t p2[NREP];
#pragma unroll
          for (int h = 0; h < NREP; ++h) p2[h] = st.p2[tp][h];
          if (BITS == 16) {
            // an odd tail pair has p = 0 for its second token, so the duplicated row adds nothing
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const half2_t va = half_pair<0>(cur.w0[k][j], cur.w1[k][j]);  // channel 2j:   (v[t], v[t+1])
              const half2_t vb = half_pair<1>(cur.w0[k][j], cur.w1[k][j]);  // channel 2j+1
#pragma unroll
              for (int h = 0; h < NREP; ++h) {
                acc[h][2 * j] = __builtin_amdgcn_fdot2(va, p2[h], acc[h][2 * j], false);
                acc[h][2 * j + 1] = __builtin_amdgcn_fdot2(vb, p2[h], acc[h][2 * j + 1], false);
              }
            }
          } else {
            const uint2 sz = st.sz[tp][g];
            half2_t s2 = as_h2(sz.x);
            const half2_t z2 = as_h2(sz.y);
            if (NORMAL) s2 = normal1_spread(s2);
            if (BITS == 1) {
              const uint32_t a0 = cur.w0[k][0] >> sh2, a1 = cur.w1[k][0] >> sh2;
              consume_byte<1, NREP, PV_CPL, NORMAL>(byte_pair<0>(a0, a1), s2, z2, p2, acc, 0);
            } else if (BITS == 2) {
              const uint32_t a0 = cur.w0[k][0] >> sh2, a1 = cur.w1[k][0] >> sh2;
              consume_byte<2, NREP, PV_CPL>(byte_pair<0>(a0, a1), s2, z2, p2, acc, 0);
              consume_byte<2, NREP, PV_CPL>(byte_pair<1>(a0, a1), s2, z2, p2, acc, 4);
            } else if (BITS == 4) {
              consume_byte<4, NREP, PV_CPL>(byte_pair<0>(cur.w0[k][0], cur.w1[k][0]), s2, z2, p2, acc, 0);
              consume_byte<4, NREP, PV_CPL>(byte_pair<1>(cur.w0[k][0], cur.w1[k][0]), s2, z2, p2, acc, 2);
              consume_byte<4, NREP, PV_CPL>(byte_pair<2>(cur.w0[k][0], cur.w1[k][0]), s2, z2, p2, acc, 4);
              consume_byte<4, NREP, PV_CPL>(byte_pair<3>(cur.w0[k][0], cur.w1[k][0]), s2, z2, p2, acc, 6);
            } else {
#pragma unroll
              for (int j = 0; j < (BITS == 8 ? 2 : 0); ++j) {
                consume_byte<8, NREP, PV_CPL>(byte_pair<0>(cur.w0[k][j], cur.w1[k][j]), s2, z2, p2, acc, 4 * j + 0);
                consume_byte<8, NREP, PV_CPL>(byte_pair<1>(cur.w0[k][j], cur.w1[k][j]), s2, z2, p2, acc, 4 * j + 1);
                consume_byte<8, NREP, PV_CPL>(byte_pair<2>(cur.w0[k][j], cur.w1[k][j]), s2, z2, p2, acc, 4 * j + 2);
                consume_byte<8, NREP, PV_CPL>(byte_pair<3>(cur.w0[k][j], cur.w1[k][j]), s2, z2, p2, acc, 4 * j + 3);
              }
            }
          }
        }
      }
      }
      cur = nxt;
    }
  }
  if constexpr (MF) {
#pragma unroll
    for (int h = 0; h < NREP; ++h)
#pragma unroll
      for (int i = 0; i < PV_CPL; ++i) acc[h][i] = av[i][h];
  }
}

#ifndef HQ_PV_MF_WAVES
#define HQ_PV_MF_WAVES 4   // waves per SIMD the matrix-core form is held to (its accumulators live in the AGPR half of the file)
#endif
template <int NREP, int D, bool MF = false>
__global__ __launch_bounds__(PV_THREADS, MF ? HQ_PV_MF_WAVES : 1) void pv_hybrid_kernel(SegTable tb, half_t *__restrict__ p,
                                                               float *__restrict__ partial, int hq_slice, int Hkv,
                                                               int64_t Tall, int64_t chunk_tokens,
                                                               int64_t n_bhq, FuseArgs fz) {
  __shared__ float red[PV_WAVES * NREP * D];
  __shared__ PvStage<NREP, D / 32> st;
  __shared__ float sm_ml[2 * NREP];  // fused mode: (max, 1 / sum exp) of each query head's row
  const int bh = blockIdx.x;
  const SegDev sg = tb.seg[seg_of_unit(tb, blockIdx.y)];  // by value: one batch of scalar loads
  const int ux = (int)blockIdx.y - sg.unit_begin;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = bh / Hkv, hkv = bh % Hkv;
  const int Hq = hq_slice & 0xffff, head0 = first_head(hq_slice, hkv);
  const int chunk_id = sg.unit_begin + ux;
  const int64_t c0 = (int64_t)ux * chunk_tokens;
  const int64_t c1 = min(c0 + chunk_tokens, sg.n_tokens);
  const bool fused = fz.stats != nullptr;
  half_t *prow[NREP];
#pragma unroll
  for (int h = 0; h < NREP; ++h) prow[h] = p + ((int64_t)b * Hq + head0 + h) * Tall;
  // The positions of the first block are asked for before anything else: what is read AT them (the logits) is the
  // longest chain of dependent loads at the start of a workgroup's life, and the statistics below wait in its shadow.
  PvPair<NREP, D / 32> first;
  pv_fetch_positions<NREP, D / 32>(sg, c0, (int)min((int64_t)PV_BLOCK, c1 - c0), first);
  if (fused) {
    // merge the per-tile (m, l) pairs of each head: wave w serves heads w, w+4, ...; up to 128 tiles are read once
    // and kept in registers between the maximum and the sum
    for (int h = wave; h < NREP; h += PV_WAVES) {
      const float2 *sp = fz.stats + ((int64_t)b * Hq + head0 + h) * fz.n_stat;
      const float2 none = make_float2(-INFINITY, 0.f);
      const float2 v0 = lane < fz.n_stat ? sp[lane] : none;
      const float2 v1 = lane + 64 < fz.n_stat ? sp[lane + 64] : none;
      float m = fmaxf(v0.x, v1.x);
      for (int e = lane + 128; e < fz.n_stat; e += 64) m = fmaxf(m, sp[e].x);
      m = wave_max(m);
      float l = (lane < fz.n_stat ? v0.y * __expf(v0.x - m) : 0.f) + (lane + 64 < fz.n_stat ? v1.y * __expf(v1.x - m) : 0.f);
      for (int e = lane + 128; e < fz.n_stat; e += 64) {
        const float2 v = sp[e];
        l += v.y * __expf(v.x - m);
      }
      l = wave_sum(l);
      if (lane == 0) {
        sm_ml[2 * h] = m;
        sm_ml[2 * h + 1] = 1.0f / l;
      }
    }
  }
  float acc[NREP][PV_CPL];
#pragma unroll
  for (int h = 0; h < NREP; ++h)
#pragma unroll
    for (int i = 0; i < PV_CPL; ++i) acc[h][i] = 0.f;
  switch (sg.bits) {  // (the first barrier inside pv_chunk also publishes sm_ml)
    case 1:
      if (sg.layout == HQEKV_LAYOUT_NORMAL1) pv_chunk<1, NREP, D, true, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first);
      else pv_chunk<1, NREP, D, false, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first);
      break;
    case 2: pv_chunk<2, NREP, D, false, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first); break;
    case 4: pv_chunk<4, NREP, D, false, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first); break;
    case 8: pv_chunk<8, NREP, D, false, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first); break;
    default: pv_chunk<16, NREP, D, false, MF>(sg, c0, c1, bh, wave, lane, prow, st, acc, fused, sm_ml, first);
  }
  // Lanes 16, 32 and 48 apart hold the same channels of other tokens.  Their sum is needed in lanes 0-15
  // only: two lane-row swaps on the vector ALU per value (a swap exchanges rows of 16 lanes between two
  // registers: the odd rows of the first with the even rows of the second, then the upper half of the first
  // with the lower half of the second) instead of two trips through the LDS crossbar, which 16 waves per CU
  // saturate (2.8 us of a 9 us workgroup life at 32k context).
  const int cl = lane & 15;
#pragma unroll
  for (int h = 0; h < NREP; ++h) {
    float v[PV_CPL], o[PV_CPL];
#pragma unroll
    for (int i = 0; i < PV_CPL; ++i) v[i] = o[i] = acc[h][i];
    static_assert(PV_CPL == 8, "the swap batches below name eight register pairs");
    // The swaps need idle issue slots between a vector-ALU write of their operands and themselves, and
    // between themselves and the first read of their results; the compiler does not see into the asm, so
    // each batch of eight independent swaps carries its own (generous) wait states.
#define HQ_SWAP8(OP_)                                                                                         \
  asm volatile("s_nop 7\n\t" OP_ " %0, %8\n\t" OP_ " %1, %9\n\t" OP_ " %2, %10\n\t" OP_ " %3, %11\n\t"         \
               OP_ " %4, %12\n\t" OP_ " %5, %13\n\t" OP_ " %6, %14\n\t" OP_ " %7, %15\n\ts_nop 7"               \
               : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), \
                 "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]))
    HQ_SWAP8("v_permlane16_swap_b32");  // rows 0 and 2: o = the old rows 1 and 3
#pragma unroll
    for (int i = 0; i < PV_CPL; ++i) v[i] = o[i] = v[i] + o[i];
    HQ_SWAP8("v_permlane32_swap_b32");  // row 0: o = the old row 2
#undef HQ_SWAP8
#pragma unroll
    for (int i = 0; i < PV_CPL; ++i) v[i] += o[i];
    if (lane < 16) {
      float4 *dst = reinterpret_cast<float4 *>(red + (wave * NREP + h) * D + cl * PV_CPL);
      dst[0] = make_float4(v[0], v[1], v[2], v[3]);
      dst[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
  }
  __syncthreads();
  const bool fold = fz.arrive != nullptr;
  for (int k = threadIdx.x; k < NREP * D; k += PV_THREADS) {
    const float v = red[k] + red[NREP * D + k] + red[2 * NREP * D + k] + red[3 * NREP * D + k];
    const int h = k / D, d = k % D;
    float *dst = partial + ((int64_t)chunk_id * n_bhq + (int64_t)b * Hq + head0 + h) * D + d;
    if (fold) __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // write-through
    else *dst = v;
  }
  if (!fold) return;
  // ---- the last workgroup of this (b, kv head) to get here adds up all partial rows
  // Ordering.  Every access to `partial` and to the counter on this path is an agent-scope atomic, so each one is
  // performed at the point of coherence all XCDs share and is never served from a cache line one XCD keeps to itself;
  // the wait below holds a thread until its partial stores have been acknowledged from there, the barrier
  // collects the workgroup, and only then does thread 0 count the workgroup in.  The workgroup that reads the final
  // count issues its loads after that read (barrier + branch; nothing is loaded ahead of the branch), again as
  // agent-scope atomics.  A release on the increment and an acquire fence after it would say the same in the
  // language's memory model, but on this target a release at agent scope writes the whole L2 back: measured on
  // the B=8, 52k-token launch that takes this path, 183 us instead of 103 us with the release on the increment
  // alone and 395 us with a release fence in every thread.  Hence relaxed atomics plus the explicit wait; any new
  // access to `partial` on this path has to be an agent-scope atomic as well.
  __shared__ uint32_t s_last;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial stores are acknowledged
  __syncthreads();
  const int n_chunks = tb.total_units;
  if (threadIdx.x == 0) {
    const uint32_t seen = __hip_atomic_fetch_add(&fz.arrive[bh], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (seen + 1u == (uint32_t)n_chunks) ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;
  // Same association as pv_combine_kernel: 32 slices (chunks s, s + 32, ...) each summed ascending from zero,
  // slices 2w and 2w + 1 added, the 16 pair sums added in order.  A thread owns two adjacent channels of one
  // query head (8-byte loads, which go past the L2 like the stores did).
  static_assert(D % 2 == 0, "channel pairs");
  for (int o = threadIdx.x; o < NREP * (D / 2); o += PV_THREADS) {
    const int h = o / (D / 2), d = 2 * (o % (D / 2));
    const int64_t row = (int64_t)b * Hq + head0 + h;
    const uint64_t *src = reinterpret_cast<const uint64_t *>(partial + row * D + d);
    const int64_t cstride = n_bhq * D / 2;  // in 8-byte units
    float t0 = 0.f, t1 = 0.f;
    static_assert(CB_FOLD_MAX == 2 * CB_SLICES, "a slice holds at most two chunks here");
#pragma unroll
    for (int w0 = 0; w0 < CB_SLICES / 2; w0 += 4) {
      // sixteen loads requested together (a missing chunk re-reads chunk 0 and counts as zero), then the sums
      uint64_t raw[4][2][2];
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            const int c = 2 * (w0 + k) + e + r * CB_SLICES;
            raw[k][e][r] = __hip_atomic_load(src + (int64_t)(c < n_chunks ? c : 0) * cstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float v[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          v[e][0] = v[e][1] = 0.f;
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            const int c = 2 * (w0 + k) + e + r * CB_SLICES;
            const bool in = c < n_chunks;
            v[e][0] += in ? __builtin_bit_cast(float, (uint32_t)raw[k][e][r]) : 0.f;
            v[e][1] += in ? __builtin_bit_cast(float, (uint32_t)(raw[k][e][r] >> 32)) : 0.f;
          }
        }
        const float p0 = v[0][0] + v[1][0], p1 = v[0][1] + v[1][1];
        t0 = (w0 + k == 0) ? p0 : t0 + p0;
        t1 = (w0 + k == 0) ? p1 : t1 + p1;
      }
    }
    *reinterpret_cast<half2_t *>(fz.out + row * D + d) = pack_h2((half_t)t0, (half_t)t1);
  }
  if (threadIdx.x == 0) __hip_atomic_store(&fz.arrive[bh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- the importance ring's row, in the order torch's GPU reduction adds fp16 rows in (fp32 accumulators):
// a thread of that reduction walks its rows with FOUR interleaved accumulators (its k-th row goes to accumulator
// k mod 4, each starting from zero) and adds them up as ((a0 + a1) + a2) + a3; the rows of one output are dealt
// round-robin to `by` threads whose results are added in a halving tree.  by is 1 for the sum over the batch, and for
// the sum over the 32 heads it is 2 when the row length is a multiple of 4 of at least 256 on an 8-byte aligned
// input, else 1 (measured against torch.sum on the device; the caller passes the value for its shape).
template <int NBY, typename Load>
__device__ __forceinline__ float torch_row_sum(int n_rows, Load &&load) {
  float v[NBY];
#pragma unroll
  for (int y = 0; y < NBY; ++y) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int r = y;
    for (; r + 3 * NBY < n_rows; r += 4 * NBY) {
      a0 += load(r);
      a1 += load(r + NBY);
      a2 += load(r + 2 * NBY);
      a3 += load(r + 3 * NBY);
    }
    if (r < n_rows) a0 += load(r);
    if (r + NBY < n_rows) a1 += load(r + NBY);
    if (r + 2 * NBY < n_rows) a2 += load(r + 2 * NBY);
    v[y] = ((a0 + a1) + a2) + a3;
  }
  if constexpr (NBY == 2) return v[0] + v[1];
  return v[0];
}

// torch_row_sum<1> for a row count known at compile time, fully unrolled (row k goes to accumulator k mod 4)
template <int N, typename Load>
__device__ __forceinline__ float torch_row_sum_n(Load &&load) {
  float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < N; ++r) a[r & 3] += load(r);
  return ((a[0] + a[1]) + a[2]) + a[3];
}

constexpr int RING_V = 4;                 // adjacent columns of the ring row a lane loads at a time (8 bytes)
constexpr int RING_SPAN = 64 * RING_V;    // columns a workgroup covers per pass
constexpr int RING_LDS_HEADS = 64;        // most heads whose batch sums a pass parks in LDS

// The probabilities as a pointer into global memory: the pointer arrives inside a by-value struct, where the
// compiler cannot tell its address space and would fall back to generic (flat) loads.
typedef const __attribute__((address_space(1))) half_t *ring_src_t;
struct __attribute__((packed, aligned(2))) ring_quad_t { uint64_t v; };   // RING_V probabilities at an element's alignment
static_assert(sizeof(half_t) * RING_V == sizeof(uint64_t), "a quad is one 64-bit word");
typedef const __attribute__((address_space(1))) ring_quad_t *ring_quad_src_t;

// what the ring row needs from the epilogue's description, by value (nothing here lives in memory)
struct RingShape {
  ring_src_t w;      // (B, Hq, Tall)
  int64_t Tall;
  int B, Hq, by;
};

// heads g, g + waves, ... of a lane's RING_V columns into the LDS tile, for a batch of NB rows known at compile
// time: the loads of HU heads are issued before the first sum is formed (the additions keep torch_row_sum's order)
// `shift` > 0 marks the row's last, ragged quad: its loads start `shift` columns early, so that they end with the
// row, and the wanted columns are moved down afterwards.
template <int NB>
__device__ __forceinline__ void ring_heads_to_lds(const RingShape r, ring_src_t col, int shift, int g, int waves,
                                                  half_t *tile_lane) {
  constexpr int HU = 8 / NB;   // heads in flight per thread: about eight loads
  const int64_t hs = r.Tall, bs = (int64_t)r.Hq * r.Tall;
  for (int h0 = g; h0 < r.Hq; h0 += waves * HU) {
    uint64_t raw[HU][NB];   // a quad is loaded, shifted and stored as one 64-bit word
#pragma unroll
    for (int u = 0; u < HU; ++u) {
      const int h = min(h0 + u * waves, r.Hq - 1);
#pragma unroll
      for (int b = 0; b < NB; ++b)   // 8 bytes at the alignment of an element: the target reads unaligned
        raw[u][b] = reinterpret_cast<ring_quad_src_t>(col + (int64_t)b * bs + (int64_t)h * hs)->v >> (16 * shift);
    }
#pragma unroll
    for (int u = 0; u < HU; ++u) {
      const int h = h0 + u * waves;
      uint64_t v = raw[u][0];
      if constexpr (NB > 1) {
        v = 0;
#pragma unroll
        for (int i = 0; i < RING_V; ++i) {
          const half_t s = (half_t)torch_row_sum_n<NB>(
              [&](int b) { return (float)__builtin_bit_cast(half_t, (uint16_t)(raw[u][b] >> (16 * i))); });
          v |= (uint64_t)__builtin_bit_cast(uint16_t, s) << (16 * i);
        }
      }
      if (h < r.Hq) *reinterpret_cast<uint64_t *>(tile_lane + h * RING_SPAN) = v;   // 8-byte aligned: lane * RING_V halves
    }
  }
}

// Column t for any batch size and head count, one load at a time: for the shapes the tiled path does not take.
// Kept out of line so that its registers do not add to the tiled path's.
__device__ __noinline__ float ring_column_alone(const RingShape r, int64_t t) {
  ring_src_t col = r.w + t;
  const int64_t hs = r.Tall, bs = (int64_t)r.Hq * r.Tall;
  auto head = [&](int h) -> float {
    if (r.B == 1) return (float)col[(int64_t)h * hs];
    return (float)(half_t)torch_row_sum<1>(r.B, [&](int b) { return (float)col[(int64_t)b * bs + (int64_t)h * hs]; });
  };
  return r.by == 2 ? torch_row_sum<2>(r.Hq, head) : torch_row_sum<1>(r.Hq, head);
}

// Columns [c0, c1) of the ring row, RING_SPAN per pass (c0 a multiple of RING_SPAN).  The loads are spread over the
// whole workgroup -- lane l of every wave looks at columns 4 l .. 4 l + 3 of the pass, wave g at heads g, g + waves,
// ... -- so every load is independent of the others and 8 bytes wide; the head values (fp16 by construction) meet
// in LDS, where the first RING_SPAN threads add them up in torch's order, one column each.  Every thread of the
// workgroup must call this with the same arguments; blockDim.x is a multiple of 64 and at least RING_SPAN.
__device__ __forceinline__ void ring_row_columns(const StepEpilogue &e, int64_t c0, int64_t c1, half_t *tile) {
  const RingShape r{(ring_src_t)(uintptr_t)e.weights, e.Tall, e.B, e.Hq, e.ring_by};
  half_t *const line = e.ring_line;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const bool lds = r.Hq <= RING_LDS_HEADS && r.B <= 8;
  for (int64_t t0 = c0; t0 < c1; t0 += RING_SPAN) {
    const int64_t t = t0 + threadIdx.x;   // the column this thread sums in the end (threads below RING_SPAN)
    if (lds) {
      const int64_t c = t0 + lane * RING_V;
      // the row's last quad may stick out by `shift` columns (the passes of all workgroups but the last end on a
      // multiple of RING_SPAN): it is loaded from `shift` columns earlier, which needs a row of RING_V columns at least
      const int shift = (int)max((int64_t)0, c + RING_V - c1);
      const bool mine = shift < RING_V && c - shift >= 0;
      ring_src_t col = r.w + (mine ? c - shift : 0);
      half_t *tile_lane = tile + lane * RING_V;
      switch (mine ? r.B : 0) {
        case 1: ring_heads_to_lds<1>(r, col, shift, g, waves, tile_lane); break;
        case 2: ring_heads_to_lds<2>(r, col, shift, g, waves, tile_lane); break;
        case 3: ring_heads_to_lds<3>(r, col, shift, g, waves, tile_lane); break;
        case 4: ring_heads_to_lds<4>(r, col, shift, g, waves, tile_lane); break;
        case 5: ring_heads_to_lds<5>(r, col, shift, g, waves, tile_lane); break;
        case 6: ring_heads_to_lds<6>(r, col, shift, g, waves, tile_lane); break;
        case 7: ring_heads_to_lds<7>(r, col, shift, g, waves, tile_lane); break;
        case 8: ring_heads_to_lds<8>(r, col, shift, g, waves, tile_lane); break;
        default: break;
      }
      __syncthreads();
    }
    if (threadIdx.x < RING_SPAN && t < c1) {
      float sum;
      if (lds && c1 >= RING_V) {
        auto head = [&](int h) -> float { return (float)tile[h * RING_SPAN + threadIdx.x]; };
        sum = r.by == 2 ? torch_row_sum<2>(r.Hq, head) : torch_row_sum<1>(r.Hq, head);
      } else {   // outside what the LDS tile covers: the thread walks its column alone
        sum = ring_column_alone(r, t);
      }
      line[t] = (half_t)sum;
    }
    if (lds) __syncthreads();
  }
}

// block `blk` of `nblk` of the epilogue: a share of the ring row's columns, and of the appended rows
__device__ __forceinline__ void step_epilogue_block(const StepEpilogue &e, int64_t blk, int64_t nblk, half_t *sh) {
  if (e.ring_line) {
    const int64_t per = ((e.Tall + nblk - 1) / nblk + RING_SPAN - 1) / RING_SPAN * RING_SPAN;
    ring_row_columns(e, min(e.Tall, blk * per), min(e.Tall, (blk + 1) * per), sh);
  }
  if (e.app_rows > 0) {   // 16-byte pieces of the appended rows, dealt over the blocks
    const int64_t row16 = e.app_row_elems / 8;   // pieces per row (head_dim is a multiple of 32)
    const int64_t per_side = (int64_t)e.app_bh * e.app_rows * row16;
    for (int64_t i = blk * blockDim.x + threadIdx.x; i < 2 * per_side; i += nblk * blockDim.x) {
      const int side = i >= per_side ? 1 : 0;
      const int64_t j = i - side * per_side;
      const int64_t bh = j / (e.app_rows * row16), rem = j % (e.app_rows * row16);
      const uint4 *src = reinterpret_cast<const uint4 *>(e.app_src[side] + bh * e.app_src_slab[side]) + rem;
      uint4 *dst = reinterpret_cast<uint4 *>(e.app_dst[side] + bh * e.app_dst_slab[side]) + rem;
      *dst = *src;
    }
  }
}

// fixed-order sum over chunks: deterministic replacement for the reference's half atomics
// (quant/csrc/gemv_cuda_wv_uniform.cu:110).  One workgroup per (b, hq) row and 128 channels; CB_SLICES
// slices of the chunk list are summed in parallel (strided, ascending within a slice, eight requests in
// flight per thread), then the slices in order.  Workgroups with blockIdx.z > 0 (or all of them, when there is
// nothing to combine) run the step epilogue instead.
__global__ __launch_bounds__(CB_CH * CB_SLICES) void pv_combine_kernel(const float *__restrict__ partial,
                                                                      half_t *__restrict__ out, int n_chunks,
                                                                      int64_t n_bhq, int D, StepEpilogue ep, int combine) {
  static_assert(RING_LDS_HEADS * RING_SPAN * sizeof(half_t) >= (CB_SLICES / 2) * CB_CH * sizeof(float) &&
                    CB_CH * CB_SLICES >= RING_SPAN, "one LDS array serves both roles");
  __shared__ __align__(16) half_t sh_all[RING_LDS_HEADS * RING_SPAN];
  const int z0 = combine ? 1 : 0;
  if ((int)blockIdx.z >= z0) {
    const int64_t per_z = (int64_t)gridDim.x * gridDim.y;
    step_epilogue_block(ep, ((int64_t)blockIdx.z - z0) * per_z + (int64_t)blockIdx.y * gridDim.x + blockIdx.x,
                        per_z * (gridDim.z - z0), sh_all);
    return;
  }
  float (*sh)[CB_CH] = reinterpret_cast<float (*)[CB_CH]>(sh_all);
  const int64_t r = blockIdx.x;
  const int d = threadIdx.x % CB_CH, sl = threadIdx.x / CB_CH;  // a wave holds two slices of the 32 channels
  const int d0 = blockIdx.y * CB_CH;
  const bool in = d0 + d < D;
  const float *src = partial + r * D + d0 + (in ? d : 0);
  const int64_t cstride = n_bhq * D;
  float v = 0.f;
  for (int c0 = sl; c0 < n_chunks; c0 += CB_SLICES * 4) {
    float t[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = c0 + k * CB_SLICES;
      t[k] = c < n_chunks ? src[(int64_t)c * cstride] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) v += t[k];
  }
  v += xor_f(v, 32);  // the wave's two slices (once per thread)
  if ((threadIdx.x & 63) < CB_CH) sh[threadIdx.x >> 6][d] = v;
  __syncthreads();
  if (threadIdx.x < CB_CH && in) {
    float t = sh[0][d];
#pragma unroll
    for (int k = 1; k < CB_SLICES / 2; ++k) t += sh[k][d];
    out[r * D + d0 + d] = (half_t)t;
  }
}

// =============================================================================== host side

// `unit_tokens`: tokens per work unit -- the q.K^T tile of the chosen tiling (the token-major fp16 residual
// always has 64-token tiles) or the p.V chunk.
static int build_table(const hqekv_seg *segs, int nseg, bool is_k, int64_t D, int64_t unit_tokens,
                       int64_t Tall, SegTable *tb, const char *who) {
  if (nseg < 0 || nseg > HQEKV_MAX_SEGS) return fail(HQEKV_E_ARG, "%s: nseg=%d out of range", who, nseg);
  if (nseg > 0 && !segs) return fail(HQEKV_E_ARG, "%s: null segment table", who);
  int64_t units = 0, max_units = 0;
  int m = 0;
  for (int k = 0; k < nseg; ++k) {
    const hqekv_seg &s = segs[k];
    if (s.n_tokens < 0) return fail(HQEKV_E_ARG, "%s: segment %d has negative n_tokens", who, k);
    if (s.n_tokens == 0) continue;
    if (!(s.bits == 16 || s.bits == 8 || s.bits == 4 || s.bits == 2 || s.bits == 1))
      return fail(HQEKV_E_ARG, "%s: segment %d bits=%d (must be 16, 8, 4, 2 or 1)", who, k, s.bits);
    if (!s.data) return fail(HQEKV_E_ARG, "%s: segment %d has null data", who, k);
    if (s.bits != 16) {
      if (!s.scale || !s.zero) return fail(HQEKV_E_ARG, "%s: segment %d lacks scale/zero", who, k);
      // K is grouped along the tokens (32 per scale); V along the channels, so a V class holds any count
      if (is_k && s.n_tokens % 32 != 0)
        return fail(HQEKV_E_ARG, "%s: segment %d n_tokens=%lld not a multiple of 32", who, k, (long long)s.n_tokens);
    }
    if (!s.idx && (s.pos_base < 0 || s.pos_base + s.n_tokens > Tall))
      return fail(HQEKV_E_ARG, "%s: segment %d positions [%lld,%lld) outside [0,%lld)", who, k,
                  (long long)s.pos_base, (long long)(s.pos_base + s.n_tokens), (long long)Tall);
    if ((uintptr_t)s.data & 3) return fail(HQEKV_E_ALIGN, "%s: segment %d data not 4-byte aligned", who, k);
    if (!is_k && s.bits != 16 && ((((uintptr_t)s.scale) | ((uintptr_t)s.zero)) & 7))
      return fail(HQEKV_E_ALIGN, "%s: segment %d scale/zero rows must be 8-byte aligned", who, k);
    if (s.bits == 16 && ((uintptr_t)s.data & 15))
      return fail(HQEKV_E_ALIGN, "%s: segment %d fp16 data must be 16-byte aligned", who, k);
    if (s.n_tokens * D >= (1LL << 31))
      return fail(HQEKV_E_UNSUPPORTED, "%s: segment %d: n_tokens * D must stay below 2^31 per (b, head) slab", who, k);
    // (every V class is token-major; on the K side only the fp16 residual is)
    const bool token_major = is_k ? (s.bits == 16 && s.layout == HQEKV_LAYOUT_TOKEN_MAJOR) : true;
    if (s.slab_tokens != 0 && (s.slab_tokens < s.n_tokens || !token_major))
      return fail(HQEKV_E_ARG, "%s: segment %d: slab_tokens applies to token-major segments and must be >= n_tokens", who, k);
    SegDev &d = tb->seg[m++];
    d.data = s.data;
    d.scale = (const half_t *)s.scale;
    d.zero = (const half_t *)s.zero;
    d.idx = s.idx;
    d.pos_base = s.pos_base;
    d.n_tokens = s.n_tokens;
    d.bits = s.bits;
    d.layout = (is_k && s.bits == 16 && s.layout == HQEKV_LAYOUT_TOKEN_MAJOR) ? HQEKV_LAYOUT_TOKEN_MAJOR
               : (s.bits == 1 && s.layout == HQEKV_LAYOUT_NORMAL1)              ? HQEKV_LAYOUT_NORMAL1
                                                                                : 0;
    d.slab_tokens = s.slab_tokens > 0 ? s.slab_tokens : s.n_tokens;
    d.unit_begin = (int32_t)units;
    const int64_t per = (is_k && d.layout == HQEKV_LAYOUT_TOKEN_MAJOR) ? 64 : unit_tokens;
    const int64_t nu = (s.n_tokens + per - 1) / per;
    d.n_units = (int32_t)nu;
    if (nu > max_units) max_units = nu;
    units += nu;
    if (nu > 65535) return fail(HQEKV_E_ARG, "%s: segment %d needs %lld work units (limit 65535)", who, k, (long long)nu);
  }
  if (units > 65535) return fail(HQEKV_E_UNSUPPORTED, "%s: %lld work units in one launch (limit 65535)", who, (long long)units);
  tb->nseg = m;
  tb->total_units = (int32_t)units;
  tb->max_units = (int32_t)max_units;
  for (int k = 0; k < HQEKV_MAX_SEGS; ++k) tb->begin[k] = k < m ? tb->seg[k].unit_begin : 0x7fffffff;
  tb->pad_ = 0;
  (void)D;
  return HQEKV_OK;
}

static int check_heads(const char *who, int64_t B, int64_t Hq, int64_t Hkv, int64_t D) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
    return fail(HQEKV_E_ARG, "%s: need B>0 and Hq %% Hkv == 0 (B=%lld Hq=%lld Hkv=%lld)", who, (long long)B,
                (long long)Hq, (long long)Hkv);
  const int64_t nrep = Hq / Hkv;
  if (nrep > 64) return fail(HQEKV_E_UNSUPPORTED, "%s: Hq/Hkv=%lld (supported: up to 64)", who, (long long)nrep);
  if (Hq > 0xffff) return fail(HQEKV_E_UNSUPPORTED, "%s: Hq=%lld (supported: up to 65535)", who, (long long)Hq);
  if (B * Hkv > 0x7fffffffLL) return fail(HQEKV_E_ARG, "%s: B*Hkv too large", who);
  if (D <= 0 || D % 32 != 0) return fail(HQEKV_E_ARG, "%s: D=%lld must be a positive multiple of 32", who, (long long)D);
  return HQEKV_OK;
}

// q.K^T tilings (HQEKV_QK_TILING_*): 1 = 8 waves per 512-token tile, 2 = 4 waves per tile (both split head_dim
// over the waves of a workgroup), 3 = one wave per 512-token tile, 4 = one wave per 256-token tile.
static int qk_tiling_of(int flags) { return (flags >> 4) & 0xf; }
static int64_t qk_tile_of(int tiling) { return tiling == 4 ? qw_tile(4) : QK_TILE; }   // qw_tile(8) == QK_TILE

// The one-wave tilings read head_dim 128 with 16-byte row accesses: every channel-major fp16 class must hold a
// multiple of 8 tokens.
static bool qk_wave_tiling_fits(const hqekv_seg *segs, int nseg, int64_t D) {
  if (D != 128) return false;
  for (int k = 0; k < nseg; ++k)
    if (segs[k].n_tokens > 0 && segs[k].bits == 16 && segs[k].layout != HQEKV_LAYOUT_TOKEN_MAJOR && segs[k].n_tokens % 8 != 0)
      return false;
  return true;
}

// tiling for a call: the forced one, or by launch size
static int resolve_qk_tiling(int forced, const hqekv_seg *segs, int nseg, int64_t BHkv, int64_t D, const char *who,
                             int *out) {
  if (forced < 0 || forced > 4) return fail(HQEKV_E_ARG, "%s: q.K^T tiling %d (known: 0 = by size, 1 .. 4)", who, forced);
  const bool fits = qk_wave_tiling_fits(segs, nseg, D);
  if (forced >= 3 && !fits)
    return fail(HQEKV_E_UNSUPPORTED, "%s: the one-wave q.K^T tilings need head_dim 128 and fp16 classes of a multiple of 8 tokens", who);
  if (forced) {
    *out = forced;
    return HQEKV_OK;
  }
  int64_t tiles512 = 0;
  for (int k = 0; k < nseg; ++k)
    if (segs[k].n_tokens > 0) tiles512 += (segs[k].n_tokens + QK_TILE - 1) / QK_TILE;
  const int64_t wgs = tiles512 * BHkv;
  // few tiles: 8 waves share a tile (shortest critical path); many: one wave per tile (least work per code)
  *out = wgs <= 1024 ? 1 : (fits ? 3 : 2);
  return HQEKV_OK;
}

static bool one_slice(int64_t nrep) { return nrep >= 1 && nrep <= 8; }

// Which form of the dot products a call uses: the matrix-core one exists for four query heads per KV head, and
// for a slice of four heads of a ratio above eight (12 = 8 + 4).
static bool dot_on_matrix_cores(int flags, int64_t nrep) {
  if ((nrep != 4 && one_slice(nrep)) || (flags & HQEKV_DOT_VALU)) return false;
  if (flags & HQEKV_DOT_MFMA) return true;
  return HQ_DEFAULT_DOT_MFMA;
}

// The kernels exist for 1 to 8 query heads per KV head; a larger ratio is cut into slices of at most eight
// (12 = 8 + 4, 13 = 8 + 5, ...), one launch per slice, each reading the K or V side again.
struct HeadSlices {
  int n, off[16], size[16];
};
static HeadSlices head_slices(int64_t nrep) {
  HeadSlices hs{};
  int off = 0;
  while (off < nrep && hs.n < 16) {
    const int c = nrep - off >= 8 ? 8 : (int)(nrep - off);
    hs.off[hs.n] = off;
    hs.size[hs.n++] = c;
    off += c;
  }
  return hs;
}
static int launch_qk_heads(const SegTable &tb, const void *q, void *scores, int64_t B, int64_t Hq, int64_t Hkv,
                           int64_t D, int64_t Tall, const FuseArgs &fz, hipStream_t st, int tiling, bool mf, int nrep,
                           int head_slice);

static int launch_qk(const SegTable &tb, const void *q, void *scores, int64_t B, int64_t Hq, int64_t Hkv,
                     int64_t D, int64_t Tall, const FuseArgs &fz, hipStream_t st, int tiling, bool mf) {
  if (tb.total_units == 0) return HQEKV_OK;
  const int64_t nrep = Hq / Hkv;
  if (one_slice(nrep)) return launch_qk_heads(tb, q, scores, B, Hq, Hkv, D, Tall, fz, st, tiling, mf, (int)nrep, (int)(nrep << 16));
  const HeadSlices hs = head_slices(nrep);
  for (int k = 0; k < hs.n; ++k) {
    const int rc = launch_qk_heads(tb, q, scores, B, Hq, Hkv, D, Tall, fz, st, tiling, mf, hs.size[k],
                                   (int)(nrep << 16) | hs.off[k]);
    if (rc) return rc;
  }
  return HQEKV_OK;
}

static int launch_qk_heads(const SegTable &tb, const void *q, void *scores, int64_t B, int64_t Hq, int64_t Hkv,
                           int64_t D, int64_t Tall, const FuseArgs &fz, hipStream_t st, int tiling, bool mf, int nrep,
                           int head_slice) {
  dim3 grid((unsigned)(B * Hkv), (unsigned)tb.total_units);
  if (tiling >= 3) {
#define LAUNCH(N_, TPL_, MF_)                                                                                        \
  hipLaunchKernelGGL((qk_wave_kernel<N_, TPL_, MF_>), grid, dim3(64), 0, st, tb, (const half_t *)q, (half_t *)scores, \
                     hq_with_slice((int)Hq, head_slice >> 16, head_slice & 0xffff), (int)Hkv, Tall, fz)
#define LAUNCH_DS(N_) \
  if (tiling == 3) LAUNCH(N_, 8, false); else LAUNCH(N_, 4, false)
    switch (nrep) {
      case 1: LAUNCH_DS(1); break;
      case 2: LAUNCH_DS(2); break;
      case 3: LAUNCH_DS(3); break;
      case 4:
        if (!mf) LAUNCH_DS(4);
        else if (tiling == 3) LAUNCH(4, 8, true);
        else LAUNCH(4, 4, true);
        break;
      case 5: LAUNCH_DS(5); break;
      case 6: LAUNCH_DS(6); break;
      case 7: LAUNCH_DS(7); break;
      default: LAUNCH_DS(8);
    }
#undef LAUNCH_DS
#undef LAUNCH
    return check_launch("qk_wave_kernel");
  }
  const int waves = tiling == 1 ? 8 : 4;
  const int tpw = 1;  // tiles per workgroup (2 and 4 measured no faster at B=8, 64k context)
  dim3 block((unsigned)waves * 64);
  const int rh = qk_reduce_heads(nrep, waves);  // QkReduce::RH
  const size_t shmem = (size_t)(nrep * D / 2 + waves * rh * QK_TILE) * sizeof(float);
#define LAUNCH(N_, W_, MF_)                                                                                        \
  hipLaunchKernelGGL((qk_hybrid_kernel<N_, W_, MF_>), grid, block, shmem, st, tb, (const half_t *)q, (half_t *)scores, \
                     hq_with_slice((int)Hq, head_slice >> 16, head_slice & 0xffff), (int)Hkv, (int)D, Tall, fz, tpw)
#define LAUNCH_W(N_) \
  if (waves == 8) LAUNCH(N_, 8, false); else LAUNCH(N_, 4, false)
  switch (nrep) {
    case 1: LAUNCH_W(1); break;
    case 2: LAUNCH_W(2); break;
    case 3: LAUNCH_W(3); break;
    case 4:
      if (!mf) LAUNCH_W(4);
      else if (waves == 8) LAUNCH(4, 8, true);
      else LAUNCH(4, 4, true);
      break;
    case 5: LAUNCH_W(5); break;
    case 6: LAUNCH_W(6); break;
    case 7: LAUNCH_W(7); break;
    default: LAUNCH_W(8);
  }
#undef LAUNCH_W
#undef LAUNCH
  return check_launch("qk_hybrid_kernel");
}

// chunk length for the p.V split-K: aim for a few workgroups per CU, never below 64 tokens
static int64_t pv_chunk_tokens(int64_t total_tokens, int64_t BHkv) {
  // Chunks hold equal token counts, so their byte counts differ by class (an fp16 row is eight 2-bit rows): a long
  // launch evens that out over two resident rounds of shorter chunks (B=8 at 64k context: 108 -> 101 us), a short
  // one keeps one round.
  const int64_t target_wgs = total_tokens * BHkv >= CB_FOLD_MIN_TOKEN_ROWS ? 256 * 8 : 256 * 4;
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

static int launch_pv(const SegTable &tb, int64_t chunk, void *p, void *out, float *partial, int64_t B,
                     int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall, const FuseArgs &fz, hipStream_t st,
                     bool mf, int stages = 3, const StepEpilogue *ep = nullptr) {
  const int64_t n_bhq = B * Hq;
  if (tb.total_units > 0 && (stages & 1)) {
    dim3 grid((unsigned)(B * Hkv), (unsigned)tb.total_units), block(PV_THREADS);
    const bool whole = one_slice(Hq / Hkv);
    HeadSlices hs = head_slices(Hq / Hkv);
    if (whole) hs = HeadSlices{1, {0}, {(int)(Hq / Hkv)}};
    for (int k = 0; k < hs.n; ++k) {
      const int head_slice = ((int)(Hq / Hkv) << 16) | (whole ? 0 : hs.off[k]);
#define LAUNCH(N_, D_, MF_)                                                                                   \
  hipLaunchKernelGGL((pv_hybrid_kernel<N_, D_, MF_>), grid, block, 0, st, tb, (half_t *)p, partial,          \
                     hq_with_slice((int)Hq, head_slice >> 16, head_slice & 0xffff), (int)Hkv, Tall, chunk, n_bhq, fz)
#define LAUNCH_D(N_) LAUNCH(N_, 128, false)
      switch (hs.size[k]) {
        case 1: LAUNCH_D(1); break;
        case 2: LAUNCH_D(2); break;
        case 3: LAUNCH_D(3); break;
        case 4:
          if (mf) LAUNCH(4, 128, true);
          else LAUNCH_D(4);
          break;
        case 5: LAUNCH_D(5); break;
        case 6: LAUNCH_D(6); break;
        case 7: LAUNCH_D(7); break;
        default: LAUNCH_D(8);
      }
#undef LAUNCH_D
#undef LAUNCH
      int rc = check_launch("pv_hybrid_kernel");
      if (rc) return rc;
    }
  }
  const bool combine = (stages & 2) && !fz.arrive;   // folded: the last p.V workgroups have written the output
  const bool epilogue = ep && (ep->ring_line || ep->app_rows > 0) && stages == 3;
  if (!combine && !epilogue) return HQEKV_OK;
  // The epilogue rides in the combine launch as extra workgroups (grid.z); one workgroup per RING_SPAN columns of
  // the ring row.  Without a combine (folded into p.V) the launch holds the epilogue alone.
  const dim3 base((unsigned)n_bhq, (unsigned)((D + CB_CH - 1) / CB_CH));
  unsigned z = combine ? 1u : 0u;
  if (epilogue) {
    const int64_t want = ep->ring_line ? (Tall + RING_SPAN - 1) / RING_SPAN : 1;
    z += (unsigned)((want + (int64_t)base.x * base.y - 1) / ((int64_t)base.x * base.y));
  }
  StepEpilogue none{};
  hipLaunchKernelGGL(pv_combine_kernel, dim3(base.x, base.y, z), dim3(CB_CH * CB_SLICES), 0, st, partial, (half_t *)out,
                     (int)tb.total_units, n_bhq, (int)D, epilogue ? *ep : none, combine ? 1 : 0);
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
  int tiling = 0;
  rc = resolve_qk_tiling(0, segs, nseg, B * Hkv, D, "qk_hybrid", &tiling);
  if (rc) return rc;
  SegTable tb{};
  rc = build_table(segs, nseg, true, D, qk_tile_of(tiling), Tall, &tb, "qk_hybrid");
  if (rc) return rc;
  return launch_qk(tb, q, scores, B, Hq, Hkv, D, Tall, FuseArgs{}, (hipStream_t)stream, tiling,
                   dot_on_matrix_cores(0, Hq / Hkv));
}

extern "C" int hqekv_scale_softmax(void *scores, const void *mask, int64_t mask_row_stride, int64_t n_rows,
                                   int64_t Tall, float inv_sqrt_d, void *stream) {
  if (n_rows < 0 || Tall <= 0 || n_rows > 0x7fffffffLL) return fail(HQEKV_E_ARG, "scale_softmax: bad shape");
  if (n_rows == 0) return HQEKV_OK;
  if (!scores) return fail(HQEKV_E_ARG, "scale_softmax: null scores");
  const dim3 grid((unsigned)n_rows), block(SM_THREADS);
  hipStream_t st = (hipStream_t)stream;
  half_t *sp = (half_t *)scores;
  const half_t *mp = (const half_t *)mask;
  const int64_t nv = (Tall + 7 + 8 * SM_THREADS - 1) / (8 * SM_THREADS);  // +7: worst-case alignment shift
  if (((uintptr_t)scores & 1) == 0 && nv <= 8) {
#define LAUNCH(N_) \
  hipLaunchKernelGGL(scale_softmax_reg_kernel<N_>, grid, block, 0, st, sp, mp, mask_row_stride, Tall, inv_sqrt_d)
    if (nv <= 1) LAUNCH(1); else if (nv <= 2) LAUNCH(2); else if (nv <= 4) LAUNCH(4); else LAUNCH(8);
#undef LAUNCH
  } else {
    hipLaunchKernelGGL(scale_softmax_kernel, grid, block, 0, st, sp, mp, mask_row_stride, Tall, inv_sqrt_d);
  }
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
  if (D != 128) return fail(HQEKV_E_UNSUPPORTED, "pv_hybrid: head_dim %lld (supported: 128)", (long long)D);
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
  return launch_pv(tb, chunk, const_cast<void *>(p), out, (float *)workspace, B, Hq, Hkv, D, Tall, FuseArgs{},
                   (hipStream_t)stream, dot_on_matrix_cores(0, Hq / Hkv));
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

struct DecodeLayout {  // carve-up of the caller's workspace
  int64_t chunk, partial_bytes, stats_off, stats_bytes, arrive_off, total;
  int64_t n_stat, chunks;
};

static int decode_layout(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v, int64_t B,
                         int64_t Hq, int64_t Hkv, int64_t D, DecodeLayout *L) {
  if (n_k < 0 || n_k > HQEKV_MAX_SEGS || n_v < 0 || n_v > HQEKV_MAX_SEGS || (n_k > 0 && !k_segs) ||
      (n_v > 0 && !v_segs) || B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0)
    return HQEKV_E_ARG;
  L->chunk = pv_chunk_tokens(seg_total_tokens(v_segs, n_v), B * Hkv);
  int64_t chunks = 0;
  for (int k = 0; k < n_v; ++k)
    if (v_segs[k].n_tokens > 0) chunks += (v_segs[k].n_tokens + L->chunk - 1) / L->chunk;
  if (chunks == 0) chunks = 1;
  int64_t tiles = 0;
  for (int k = 0; k < n_k; ++k)
    if (k_segs[k].n_tokens > 0) {
      // room for the statistics of the smallest tile any tiling uses (the token-major residual: 64 tokens)
      const int64_t per = (k_segs[k].bits == 16 && k_segs[k].layout == HQEKV_LAYOUT_TOKEN_MAJOR) ? 64 : qw_tile(4);   // 256
      tiles += (k_segs[k].n_tokens + per - 1) / per;
    }
  if (tiles == 0) tiles = 1;
  L->n_stat = tiles;
  L->partial_bytes = align_up(chunks * B * Hq * D * (int64_t)sizeof(float), 256);
  L->stats_off = L->partial_bytes;
  L->stats_bytes = align_up(B * Hq * tiles * (int64_t)sizeof(float2), 256);
  L->arrive_off = L->stats_off + L->stats_bytes;
  L->chunks = chunks;
  L->total = L->arrive_off + align_up(B * Hkv * (int64_t)sizeof(uint32_t), 256);
  return HQEKV_OK;
}

extern "C" int64_t hqekv_decode_workspace_bytes(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs,
                                                int n_v, int64_t B, int64_t Hq, int64_t Hkv, int64_t D) {
  DecodeLayout L;
  if (decode_layout(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D, &L)) return -1;
  return L.total;
}

static int fill_epilogue(const hqekv_step_extra *x, const void *attn_weights, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                         int64_t Tall, StepEpilogue *e) {
  *e = StepEpilogue{};
  if (!x) return HQEKV_OK;
  e->weights = (const half_t *)attn_weights;
  e->Tall = Tall;
  e->B = (int32_t)B;
  e->Hq = (int32_t)Hq;
  if (x->ring_line) {
    if (x->ring_order != 1 && x->ring_order != 2) return fail(HQEKV_E_ARG, "decode_step: ring_order must be 1 or 2");
    if ((uintptr_t)x->ring_line & 1) return fail(HQEKV_E_ALIGN, "decode_step: ring_line not 2-byte aligned");
    e->ring_line = (half_t *)x->ring_line;
    e->ring_by = x->ring_order;
  }
  if (x->append_rows < 0) return fail(HQEKV_E_ARG, "decode_step: negative append_rows");
  if (x->append_rows > 0) {
    if (!x->new_k || !x->new_v || !x->k_dst || !x->v_dst) return fail(HQEKV_E_ARG, "decode_step: append without source or destination");
    if (x->k_dst_slab_tokens < x->append_rows || x->v_dst_slab_tokens < x->append_rows)
      return fail(HQEKV_E_ARG, "decode_step: destination slabs shorter than the appended rows");
    if (((uintptr_t)x->new_k | (uintptr_t)x->new_v | (uintptr_t)x->k_dst | (uintptr_t)x->v_dst) & 15)
      return fail(HQEKV_E_ALIGN, "decode_step: appended rows and their destinations must be 16-byte aligned");
    e->app_rows = x->append_rows;
    e->app_row_elems = (int32_t)D;
    e->app_bh = (int32_t)(B * Hkv);
    e->app_src[0] = (const half_t *)x->new_k;
    e->app_src[1] = (const half_t *)x->new_v;
    e->app_dst[0] = (half_t *)x->k_dst;
    e->app_dst[1] = (half_t *)x->v_dst;
    e->app_src_slab[0] = e->app_src_slab[1] = (int64_t)x->append_rows * D;
    e->app_dst_slab[0] = x->k_dst_slab_tokens * D;
    e->app_dst_slab[1] = x->v_dst_slab_tokens * D;
  }
  return HQEKV_OK;
}

extern "C" int hqekv_ring_row(const void *attn_weights, int64_t B, int64_t Hq, int64_t Tall, void *line, int order,
                              void *stream) {
  if (!attn_weights || !line || B <= 0 || Hq <= 0 || Tall <= 0 || B > 0x7fffffffLL || Hq > 0x7fffffffLL)
    return fail(HQEKV_E_ARG, "ring_row: null pointer or empty shape");
  hqekv_step_extra x{};
  x.ring_line = line;
  x.ring_order = order;
  StepEpilogue e;
  const int rc = fill_epilogue(&x, attn_weights, B, Hq, 1, 32, Tall, &e);
  if (rc) return rc;
  const int64_t blocks = (Tall + RING_SPAN - 1) / RING_SPAN;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_UNSUPPORTED, "ring_row: Tall too large");
  hipLaunchKernelGGL(pv_combine_kernel, dim3((unsigned)blocks, 1, 1), dim3(CB_CH * CB_SLICES), 0, (hipStream_t)stream,
                     (const float *)nullptr, (half_t *)nullptr, 0, (int64_t)0, 0, e, 0);
  return check_launch("ring_row");
}

static int decode_impl(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                       const void *q, const void *mask, int64_t mask_row_stride, void *attn_weights,
                       void *attn_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall,
                       void *workspace, int64_t workspace_bytes, int flags, void *stream, const hqekv_step_extra *extra);

extern "C" int hqekv_decode_attn(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                                 const void *q, const void *mask, int64_t mask_row_stride, void *attn_weights,
                                 void *attn_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall,
                                 void *workspace, int64_t workspace_bytes, int flags, void *stream) {
  return decode_impl(k_segs, n_k, v_segs, n_v, q, mask, mask_row_stride, attn_weights, attn_out, B, Hq, Hkv, D, Tall,
                     workspace, workspace_bytes, flags, stream, nullptr);
}

extern "C" int hqekv_decode_step(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                                 const void *q, const void *mask, int64_t mask_row_stride, void *attn_weights,
                                 void *attn_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall,
                                 void *workspace, int64_t workspace_bytes, int flags, void *stream,
                                 const hqekv_step_extra *extra) {
  if (flags & (HQEKV_ONLY_QK | HQEKV_ONLY_PV | HQEKV_ONLY_COMBINE | HQEKV_ONLY_RAW_QK))
    return fail(HQEKV_E_ARG, "decode_step: the single-stage flags belong to hqekv_decode_attn");
  return decode_impl(k_segs, n_k, v_segs, n_v, q, mask, mask_row_stride, attn_weights, attn_out, B, Hq, Hkv, D, Tall,
                     workspace, workspace_bytes, flags, stream, extra);
}

static int decode_impl(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                       const void *q, const void *mask, int64_t mask_row_stride, void *attn_weights,
                       void *attn_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall,
                       void *workspace, int64_t workspace_bytes, int flags, void *stream, const hqekv_step_extra *extra) {
  int rc = check_heads("decode_attn", B, Hq, Hkv, D);
  if (rc) return rc;
  if (D != 128) return fail(HQEKV_E_UNSUPPORTED, "decode_attn: head_dim %lld (supported: 128)", (long long)D);
  if (!q || !attn_weights || !attn_out || Tall <= 0) return fail(HQEKV_E_ARG, "decode_attn: null pointer or Tall <= 0");
  DecodeLayout L;
  if (decode_layout(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D, &L)) return fail(HQEKV_E_ARG, "decode_attn: bad segment tables");
  if (!workspace || workspace_bytes < L.total)
    return fail(HQEKV_E_WORKSPACE, "decode_attn: workspace %lld bytes < %lld needed", (long long)workspace_bytes,
                (long long)L.total);
  if ((uintptr_t)workspace & 255) return fail(HQEKV_E_ALIGN, "decode_attn: workspace not 256-byte aligned");
  int tiling = 0;
  rc = resolve_qk_tiling(qk_tiling_of(flags), k_segs, n_k, B * Hkv, D, "decode_attn", &tiling);
  if (rc) return rc;
  SegTable kt{}, vt{};
  rc = build_table(k_segs, n_k, true, D, qk_tile_of(tiling), Tall, &kt, "decode_attn(K)");
  if (rc) return rc;
  rc = build_table(v_segs, n_v, false, D, L.chunk, Tall, &vt, "decode_attn(V)");
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  char *ws = (char *)workspace;
  // The softmax can ride inside the two GEMV launches when nothing is added to the logits and every
  // position is produced by exactly one K token and consumed by exactly one V token.
  const bool fuse = (flags & HQEKV_FUSE_SOFTMAX) && !mask && seg_total_tokens(k_segs, n_k) == Tall &&
                    seg_total_tokens(v_segs, n_v) == Tall && kt.total_units > 0 && vt.total_units > 0;
  FuseArgs fz{};
  if (fuse) {
    fz.stats = (float2 *)(ws + L.stats_off);
    fz.n_stat = (int32_t)kt.total_units;
    fz.inv_sqrt_d = 1.0f / (float)sqrt((double)D);
  }
  // Few chunks per (b, kv head) and a long p.V launch: the last p.V workgroup of each (b, kv head) adds the
  // partials up and the combine launch is dropped.  The write-through stores, the counter and the final loads
  // lengthen every workgroup's tail by 5-8 us, which only a launch of some 100 us absorbs (B=8 at 64k context:
  // step 204 -> 198 us; B=1 at 32k: p.V 14 -> 22 us against a 3 us combine, so short launches keep the combine).
  fz.two_step = (flags & HQEKV_TWO_STEP_DEQUANT) ? 1 : 0;
  const bool fold_pays = seg_total_tokens(v_segs, n_v) * B * Hkv >= CB_FOLD_MIN_TOKEN_ROWS;
  const bool fold_forced = (flags & HQEKV_FOLD_COMBINE) != 0;
  // (more than eight heads per KV head run as several p.V launches against the one counter: they keep the combine launch)
  if (kt.total_units > 0 && vt.total_units > 0 && vt.total_units <= CB_FOLD_MAX && !(flags & HQEKV_SEPARATE_COMBINE) &&
      (fold_pays || fold_forced) && one_slice(Hq / Hkv)) {
    fz.arrive = (uint32_t *)(ws + L.arrive_off);
    fz.out = (half_t *)attn_out;
  }
  if ((flags & HQEKV_DOT_MFMA) && (flags & HQEKV_DOT_VALU))
    return fail(HQEKV_E_ARG, "decode_attn: HQEKV_DOT_MFMA and HQEKV_DOT_VALU exclude each other");
  if ((flags & HQEKV_DOT_MFMA) && Hq / Hkv != 4 && one_slice(Hq / Hkv))
    return fail(HQEKV_E_UNSUPPORTED, "decode_attn: the matrix-core dot products need Hq/Hkv == 4, or a ratio above 8 (got %lld)", (long long)(Hq / Hkv));
  const bool mf = dot_on_matrix_cores(flags, Hq / Hkv);
  if (flags & HQEKV_ONLY_RAW_QK) {   // the q.K^T launch alone, raw fp16 scores: no scaling, no statistics, no softmax
    FuseArgs raw{};
    raw.two_step = fz.two_step;
    return launch_qk(kt, q, attn_weights, B, Hq, Hkv, D, Tall, raw, st, tiling, mf);
  }
  const int only = flags & (HQEKV_ONLY_QK | HQEKV_ONLY_PV | HQEKV_ONLY_COMBINE);
  const bool only_qk = only == HQEKV_ONLY_QK;
  if (only == 0 || only_qk) {
    rc = launch_qk(kt, q, attn_weights, B, Hq, Hkv, D, Tall, fz, st, tiling, mf);
    if (rc) return rc;
    if (!fuse) {
      rc = hqekv_scale_softmax(attn_weights, mask, mask_row_stride, B * Hq, Tall, 1.0f / (float)sqrt((double)D), stream);
      if (rc) return rc;
    }
  }
  if (only_qk) return HQEKV_OK;
  const int stages = only == HQEKV_ONLY_PV ? 1 : (only == HQEKV_ONLY_COMBINE ? 2 : 3);
  StepEpilogue ep;
  rc = fill_epilogue(extra, attn_weights, B, Hq, Hkv, D, Tall, &ep);
  if (rc) return rc;
  return launch_pv(vt, L.chunk, attn_weights, attn_out, (float *)ws, B, Hq, Hkv, D, Tall, fz, st, mf, stages, &ep);
}

// ------------------------------------------------------------------ per-class GEMV on the same kernels
// Both launches compute the same contraction; the p.V one reduces over many rows (tokens) with split-K and
// takes any row count, the q.K^T one wants the rows (channels) in multiples of 32.
static bool gemv_is_pv_shape(int64_t K, int64_t N) { return N == 128 && (K > N || K % 32 != 0); }

extern "C" int64_t hqekv_gemv_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N, int bits) {
  (void)bits;
  if (!gemv_is_pv_shape(K, N)) return 0;
  hqekv_seg s{};
  s.bits = 2;
  s.n_tokens = K;
  return hqekv_pv_workspace_bytes(&s, 1, B, Hq, Hkv, N);
}

static int gemv_group(const char *who, int layout, const void *fA, const void *code, const void *scale,
                      const void *zero, void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N, int bits,
                      void *workspace, int64_t workspace_bytes, void *stream) {
  if (K <= 0 || N <= 0 || N % 32 != 0) return fail(HQEKV_E_ARG, "%s: need N %% 32 == 0, K > 0", who);
  hqekv_seg s{};
  s.bits = bits;
  s.layout = layout;
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
  if (K % 32 != 0) return fail(HQEKV_E_UNSUPPORTED, "%s: K=%lld must be a multiple of 32", who, (long long)K);
  s.n_tokens = N;
  return hqekv_qk_hybrid(&s, 1, fA, out, B, Hq, Hkv, K, N, stream);
}

extern "C" int hqekv_gemv_uniform_group(const void *fA, const void *code, const void *scale, const void *zero,
                                        void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N,
                                        int bits, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!(bits == 1 || bits == 2 || bits == 4 || bits == 8)) return fail(HQEKV_E_ARG, "gemv_uniform_group: bits=%d", bits);
  return gemv_group("gemv_uniform_group", 0, fA, code, scale, zero, out, B, Hq, Hkv, K, N, bits, workspace,
                    workspace_bytes, stream);
}

extern "C" int hqekv_gemv_normal_group(const void *fA, const void *code, const void *stdv, const void *meanv,
                                       void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N,
                                       int bits, void *workspace, int64_t workspace_bytes, void *stream) {
  if (bits != 1)
    return fail(HQEKV_E_UNSUPPORTED, "gemv_normal_group: bits=%d (only the 1-bit normal-quantile class is built)", bits);
  return gemv_group("gemv_normal_group", HQEKV_LAYOUT_NORMAL1, fA, code, stdv, meanv, out, B, Hq, Hkv, K, N, 1,
                    workspace, workspace_bytes, stream);
}
