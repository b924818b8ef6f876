// Cache maintenance on the device: one launch rebuilds every precision class of one side (K or V) of a layer's
// cache from the old classes and the new fp16 tokens, following a block-level plan the host worked out.
//
// What the reference does per compression (quant/hqe_2.py:552-836) is a sequence of boolean-mask gathers,
// dequantise / re-quantise calls and torch.cat re-copies, one group of launches per (source, target) pair.  All of
// it moves whole blocks of 32 tokens, and every block ends in exactly one place, so the whole compression is a
// gather: destination block u of class c comes from block v of source s.  A unit of work is one quantisation
// group of one block -- K: (block, channel), the 32 tokens of a channel; V: (token, 32 channels) -- held by one
// lane as 32 fp16 values:
//   same width            copy of the packed words, scale and zero (a survivor keeps its bytes)
//   fp16 -> b bits        the quantiser of quant/pack_unpack.py:156-193 (or :218-253 for the 1-bit normal class)
//   a bits -> b < a bits  dequantise with the reference's two fp16 roundings (quant/pack_unpack.py:331-332), then
//                         quantise: what K_high_2_low / V_high_2_low do (quant/hqe_2.py:88-170)
//   fp16 -> fp16          copy (new K arrives token-major and is stored channel-major)
// Evicted blocks are simply in nobody's plan.  The arithmetic is the one of the stand-alone kernels (quant_math.h),
// so the bytes equal those of the step-by-step path.
#include "common.h"
#include "quant_math.h"

#pragma clang fp contract(off)

namespace hq {

struct MigClass {
  void *data;
  half_t *scale;
  half_t *zero;
  int64_t *idx;
  int64_t n_tokens;
  int64_t slab_tokens;  // tokens between (b, h) slabs of a token-major fp16 source (>= n_tokens)
  int32_t bits;
  int32_t layout;
};

struct MigArgs {
  MigClass src[HQEKV_MAX_SEGS];
  MigClass dst[HQEKV_MAX_SEGS];
  int32_t dst_begin[HQEKV_MAX_SEGS + 1];  // first plan entry of every destination class; [n_dst] = total
  int32_t n_dst;
  int32_t n_src;
  const int32_t *plan_src;  // (source slot << 24) | source block, per destination block
  const int32_t *plan_pos;  // new position of the block's first token / 32
  int32_t *status;          // optional: set to non-zero when a plan entry is refused
};

// The plan lives in device memory and is read by the kernel only, so the kernel is what checks it: an entry must name
// a populated source class, a block inside it and a position inside the new sequence.  An entry that does not is
// skipped (its destination block keeps whatever the buffer held) and flagged; nothing is read or written out of range.
__device__ __forceinline__ bool plan_entry_ok(const MigArgs &a, int32_t code, int32_t pos, int total) {
  const uint32_t slot = (uint32_t)code >> 24, blk = (uint32_t)code & 0xffffffu;
  if (slot >= (uint32_t)a.n_src) return false;
  const int64_t n = a.src[slot].n_tokens;
  return n > 0 && a.src[slot].data != nullptr && (int64_t)blk < (n >> 5) && pos >= 0 && pos < total;
}
__device__ __forceinline__ void plan_refused(const MigArgs &a) {
  if (a.status) atomicOr(a.status, 1);
}

// where one lane's group lives: fp16 values (with the element stride) or packed words + scale + zero
struct GroupRef {
  half_t *f16;
  int64_t stride;
  uint32_t *words;
  half_t *s, *z;
};

template <bool IS_K>
__device__ __forceinline__ GroupRef group_ref(const MigClass &c, int64_t bh, int64_t block, int lane, int D) {
  GroupRef r{};
  const int64_t n = c.n_tokens;
  if (IS_K) {
    const int d = lane;  // channel
    if (c.bits == 16) {
      if (c.layout == HQEKV_LAYOUT_TOKEN_MAJOR) {  // (B,H,T,D)
        r.f16 = (half_t *)c.data + ((bh * c.slab_tokens + block * 32) * D + d);
        r.stride = D;
      } else {  // (B,H,D,T)
        r.f16 = (half_t *)c.data + ((bh * D + d) * n + block * 32);
        r.stride = 1;
      }
    } else {
      const int64_t g = (bh * D + d) * (n >> 5) + block;
      r.words = (uint32_t *)c.data + g * c.bits;  // 32 codes of b bits = b words
      r.s = c.scale + g;
      r.z = c.zero + g;
    }
  } else {
    const int ng = D >> 5;
    const int k = lane / ng, cg = lane % ng;  // token of the block, channel group
    if (c.bits == 16) {
      const int64_t t = bh * c.slab_tokens + block * 32 + k;
      r.f16 = (half_t *)c.data + (t * D + cg * 32);
      r.stride = 1;
    } else {
      const int64_t g = (bh * n + block * 32 + k) * ng + cg;
      r.words = (uint32_t *)c.data + g * c.bits;
      r.s = c.scale + g;
      r.z = c.zero + g;
    }
  }
  return r;
}

// 32 fp16 values as 16 registers: xp[j] = (x[2j], x[2j+1])
__device__ __forceinline__ void load_f16(const GroupRef &r, uint32_t (&xp)[16]) {
  if (r.stride == 1) {
    const uint4 *p = reinterpret_cast<const uint4 *>(r.f16);  // block starts are 64-byte aligned
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint4 v = p[i];
      xp[4 * i] = v.x;
      xp[4 * i + 1] = v.y;
      xp[4 * i + 2] = v.z;
      xp[4 * i + 3] = v.w;
    }
  } else {
    const unsigned short *p = reinterpret_cast<const unsigned short *>(r.f16);
#pragma unroll
    for (int j = 0; j < 16; ++j)
      xp[j] = (uint32_t)p[(2 * j) * r.stride] | ((uint32_t)p[(2 * j + 1) * r.stride] << 16);
  }
}
__device__ __forceinline__ void store_f16(const GroupRef &r, const uint32_t (&xp)[16]) {
  uint4 *p = reinterpret_cast<uint4 *>(r.f16);  // fp16 classes are stored with unit stride
#pragma unroll
  for (int i = 0; i < 4; ++i) p[i] = make_uint4(xp[4 * i], xp[4 * i + 1], xp[4 * i + 2], xp[4 * i + 3]);
}

// out = rnd16(rnd16(c * scale) + zero); NORMAL: rnd16(rnd16(+-k * std) + mean)
template <int BITS, bool NORMAL>
__device__ __forceinline__ void dequant_group(const GroupRef &r, uint32_t (&xp)[16]) {
  constexpr int PF = 32 / BITS;
  uint32_t w[BITS];
#pragma unroll
  for (int i = 0; i < BITS; ++i) w[i] = r.words[i];
  const half_t s = *r.s, z = *r.z;
  // fp16 multiply and add, each one rounding of the exact result (through fp32 the compiler's mixed-precision fma
  // with a +0 addend would lose the sign of a -0 product)
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    half2_t v;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int k = 2 * j + e;
      const uint32_t ci = code_at<BITS>(w[k / PF], k % PF);
      const half_t m = NORMAL ? (ci != 0u ? (half_t)0.67431640625f : (half_t)-0.67431640625f) * s : (half_t)(float)ci * s;
      v[e] = m + z;
    }
    xp[j] = h2_bits(v);
  }
}

template <int BITS>
__device__ __forceinline__ void quant_group(const GroupRef &r, const uint32_t (&xp)[16]) {
  constexpr int PF = 32 / BITS;
  constexpr int HALF = PF / 2;
  constexpr float INV_QMAX = 1.0f / (float)((1 << BITS) - 1);
  half2_t lo2 = bits_h2(xp[0]), hi2 = lo2;
#pragma unroll
  for (int j = 1; j < 16; ++j) {
    lo2 = __builtin_elementwise_min(lo2, bits_h2(xp[j]));
    hi2 = __builtin_elementwise_max(hi2, bits_h2(xp[j]));
  }
  half_t mn_h = (half_t)__builtin_fminf((float)lo2[0], (float)lo2[1]);
  float mn = (float)mn_h, mx = __builtin_fmaxf((float)hi2[0], (float)hi2[1]);
  // a zero extreme takes the sign of the group's first zero (torch's tie rule); rare, so the wave branches around it
  if (__builtin_amdgcn_ballot_w64(mn == 0.0f || mx == 0.0f) != 0 && (mn == 0.0f || mx == 0.0f)) {
    half_t v[32];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const half2_t h = bits_h2(xp[j]);
      v[2 * j] = h[0];
      v[2 * j + 1] = h[1];
    }
    const half_t z = __builtin_bit_cast(half_t, (unsigned short)first_zero_bits(v));
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
  float u[32];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const half2_t c = bits_h2(xp[j]) - mn2;
    u[2 * j] = (float)c[0];
    u[2 * j + 1] = (float)c[1];
  }
#pragma unroll
  for (int wj = 0; wj < BITS; ++wj) {
    uint32_t zz[HALF];
#pragma unroll
    for (int i = 0; i < HALF; ++i) zz[i] = code_pair_biased<BITS>(u[wj * PF + i], rcp, u[wj * PF + i + HALF], rcp);
    r.words[wj] = horner_pack<BITS, HALF>(zz);
  }
  *r.s = sc;
  *r.z = mn_h;
}

// the 1-bit normal-quantile quantiser: statistics in the order of torch's GPU reduction, code = [x > mean]
__device__ __forceinline__ void quant_group_normal1(const GroupRef &r, const uint32_t (&xp)[16]) {
  float xf[32];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const half2_t v = bits_h2(xp[j]);
    xf[2 * j] = (float)v[0];
    xf[2 * j + 1] = (float)v[1];
  }
  const Normal1Stats st = normal1_finish(welford_tree<32>(xf));
  uint32_t w = 0;
#pragma unroll
  for (int k = 0; k < 32; ++k) w |= normal1_code((half_t)(xf[k] - (float)st.mean_h), st.thr) << k;
  r.words[0] = w;
  *r.s = st.std_h;
  *r.z = st.mean_h;
}

// One quantisation group: lane = channel (K) or (token, channel group) (V) of source block sb -> destination block db.
template <bool IS_K>
__device__ __forceinline__ void migrate_group(const MigClass &sc, const MigClass &dc, int64_t bh, int64_t sb, int64_t db,
                                              int lane, int D) {
  const GroupRef sr = group_ref<IS_K>(sc, bh, sb, lane, D);
  const GroupRef dr = group_ref<IS_K>(dc, bh, db, lane, D);
  if (sc.bits != 16 && sc.bits == dc.bits) {  // a survivor of a quantised class keeps its bytes
    for (int i = 0; i < sc.bits; ++i) dr.words[i] = sr.words[i];
    *dr.s = *sr.s;
    *dr.z = *sr.z;
    return;
  }
  uint32_t xp[16];
  const bool sn = sc.layout == HQEKV_LAYOUT_NORMAL1;
  switch (sc.bits) {
    case 16: load_f16(sr, xp); break;
    case 8: dequant_group<8, false>(sr, xp); break;
    case 4: dequant_group<4, false>(sr, xp); break;
    case 2: dequant_group<2, false>(sr, xp); break;
    default:
      if (sn) dequant_group<1, true>(sr, xp);
      else dequant_group<1, false>(sr, xp);
  }
  switch (dc.bits) {
    case 16: store_f16(dr, xp); break;
    case 8: quant_group<8>(dr, xp); break;
    case 4: quant_group<4>(dr, xp); break;
    case 2: quant_group<2>(dr, xp); break;
    default:
      if (dc.layout == HQEKV_LAYOUT_NORMAL1) quant_group_normal1(dr, xp);
      else quant_group<1>(dr, xp);
  }
}

__device__ __forceinline__ int dst_class_of(const MigArgs &a, int u) {
  int ci = 0;
#pragma unroll
  for (int k = 1; k < HQEKV_MAX_SEGS; ++k) ci += (k < a.n_dst && u >= a.dst_begin[k]) ? 1 : 0;
  return ci;
}

constexpr int MIG_THREADS = 128;
constexpr int MIG_KB = 16;  // K side: destination blocks per workgroup

// V side: a workgroup per destination block; its 32 tokens x D/32 groups are one contiguous stretch of every plane.
// K side: a group is 32 tokens of ONE channel row -- b words of the row -- and a block's groups lie a whole row
// apart, so a workgroup takes 16 consecutive destination blocks and lets neighbouring lanes take neighbouring
// blocks of a row: 16 b-word pieces side by side (64 bytes at 1 bit ... 512 at 8), and as long as the blocks come
// from consecutive places of one source class (survivors of a class stay in order) the reads line up the same
// way.  (A lane per channel, as on the V side, touched a separate cache line per lane: the K launch took four to
// six times as long as the V launch for the same bytes.)  Blocks of new tokens arrive token-major, where the
// channels of a token are what is contiguous: a workgroup that holds any of those walks its blocks one by one
// with a lane per channel.
template <bool IS_K>
__global__ __launch_bounds__(MIG_THREADS) void cache_migrate_kernel(MigArgs a, int D) {
  const int64_t bh = blockIdx.y;
  const int total = a.dst_begin[HQEKV_MAX_SEGS];
  if constexpr (!IS_K) {
    const int u = blockIdx.x;
    const MigClass dc = a.dst[dst_class_of(a, u)];
    const int64_t db = u - a.dst_begin[dst_class_of(a, u)];
    const int32_t code = a.plan_src[u];
    if (!plan_entry_ok(a, code, a.plan_pos[u], total)) {   // uniform: the whole workgroup serves this entry
      if (threadIdx.x == 0) plan_refused(a);
      return;
    }
    if (bh == 0 && threadIdx.x < 32 && dc.idx) dc.idx[db * 32 + threadIdx.x] = (int64_t)a.plan_pos[u] * 32 + threadIdx.x;
    for (int lane = threadIdx.x; lane < D; lane += MIG_THREADS)
      migrate_group<false>(a.src[code >> 24], dc, bh, code & 0xffffff, db, lane, D);
  } else {
    const int u0 = blockIdx.x * MIG_KB;
    const int u = u0 + (int)(threadIdx.x % MIG_KB);
    const int uc = u < total ? u : u0;   // (u0 < total by the grid size)
    const int ci = dst_class_of(a, uc);
    const int64_t db = uc - a.dst_begin[ci];
    const int32_t code = a.plan_src[uc];
    const bool entry_ok = plan_entry_ok(a, code, a.plan_pos[uc], total);
    const bool live = u < total && entry_ok;
    if (u < total && !entry_ok && threadIdx.x < MIG_KB) plan_refused(a);
    const int si = entry_ok ? (int)((uint32_t)code >> 24) : 0;
    const bool token_major = entry_ok && a.src[si].bits == 16 && a.src[si].layout == HQEKV_LAYOUT_TOKEN_MAJOR;
    if (bh == 0) {  // positions of the blocks' tokens
      for (int e = threadIdx.x; e < MIG_KB * 32; e += MIG_THREADS) {
        const int ue = u0 + e / 32;
        if (ue < total && plan_entry_ok(a, a.plan_src[ue], a.plan_pos[ue], total)) {
          const int ce = dst_class_of(a, ue);
          int64_t *idx = a.dst[ce].idx;
          if (idx) idx[(int64_t)(ue - a.dst_begin[ce]) * 32 + e % 32] = (int64_t)a.plan_pos[ue] * 32 + e % 32;
        }
      }
    }
    if (__syncthreads_or(live && token_major)) {
      for (int j = 0; j < MIG_KB && u0 + j < total; ++j) {
        const int cj = dst_class_of(a, u0 + j);
        const int32_t code_j = a.plan_src[u0 + j];
        if (!plan_entry_ok(a, code_j, a.plan_pos[u0 + j], total)) continue;   // uniform
        for (int lane = threadIdx.x; lane < D; lane += MIG_THREADS)
          migrate_group<true>(a.src[code_j >> 24], a.dst[cj], bh, code_j & 0xffffff, u0 + j - a.dst_begin[cj], lane, D);
      }
    } else if (live) {
      const MigClass sc = a.src[si], dc = a.dst[ci];
      for (int d = threadIdx.x / MIG_KB; d < D; d += MIG_THREADS / MIG_KB)
        migrate_group<true>(sc, dc, bh, code & 0xffffff, db, d, D);
    }
  }
}

static int check_class(const hqekv_cache_class &c, bool is_src, int k, int64_t D) {
  const char *side = is_src ? "source" : "destination";
  if (c.n_tokens < 0 || c.n_tokens % 32 != 0)
    return fail(HQEKV_E_ARG, "cache_migrate: %s %d holds %lld tokens (whole blocks of 32 only)", side, k, (long long)c.n_tokens);
  if (c.n_tokens == 0) return HQEKV_OK;
  if (!(c.bits == 16 || c.bits == 8 || c.bits == 4 || c.bits == 2 || c.bits == 1))
    return fail(HQEKV_E_ARG, "cache_migrate: %s %d bits=%d", side, k, c.bits);
  if (!c.data || (c.bits != 16 && (!c.scale || !c.zero)))
    return fail(HQEKV_E_ARG, "cache_migrate: %s %d lacks data / scale / zero", side, k);
  if ((uintptr_t)c.data & (c.bits == 16 ? 15 : 3)) return fail(HQEKV_E_ALIGN, "cache_migrate: %s %d data misaligned", side, k);
  if (c.n_tokens * D >= (1LL << 40)) return fail(HQEKV_E_UNSUPPORTED, "cache_migrate: %s %d too large", side, k);
  return HQEKV_OK;
}

}  // namespace hq

using namespace hq;

extern "C" int hqekv_cache_migrate(int is_k, const hqekv_cache_class *src, int n_src, const hqekv_cache_class *dst,
                                   int n_dst, const int32_t *plan, int64_t BH, int64_t D, int32_t *status, void *stream) {
  if (n_src < 0 || n_src > HQEKV_MAX_SEGS || n_dst < 0 || n_dst > HQEKV_MAX_SEGS || (n_src && !src) || (n_dst && !dst))
    return fail(HQEKV_E_ARG, "cache_migrate: bad class tables");
  if (BH <= 0 || BH > 65535 || D <= 0 || D % 32 != 0 || D > 1024)
    return fail(HQEKV_E_ARG, "cache_migrate: need 0 < B*H <= 65535 and head_dim a multiple of 32 up to 1024");
  MigArgs a{};
  int64_t total = 0;
  for (int k = 0; k < n_src; ++k) {
    const int rc = check_class(src[k], true, k, D);
    if (rc) return rc;
    // fp16 sources are read 32 values at a time: channel-major rows and token-major rows start 16-byte aligned
    const int64_t slab = src[k].slab_tokens > 0 ? src[k].slab_tokens : src[k].n_tokens;
    if (slab < src[k].n_tokens || (slab != src[k].n_tokens && !(src[k].bits == 16 && (!is_k || src[k].layout == HQEKV_LAYOUT_TOKEN_MAJOR))))
      return fail(HQEKV_E_ARG, "cache_migrate: source %d: slab_tokens applies to token-major fp16 sources and must be >= n_tokens", k);
    a.src[k] = MigClass{src[k].data, (half_t *)src[k].scale, (half_t *)src[k].zero, nullptr, src[k].n_tokens, slab, src[k].bits, src[k].layout};
  }
  for (int k = 0; k < n_dst; ++k) {
    const int rc = check_class(dst[k], false, k, D);
    if (rc) return rc;
    if (dst[k].bits == 16 && dst[k].layout == HQEKV_LAYOUT_TOKEN_MAJOR && is_k)
      return fail(HQEKV_E_UNSUPPORTED, "cache_migrate: the fp16 K class is stored channel-major");
    if (dst[k].slab_tokens != 0 && dst[k].slab_tokens != dst[k].n_tokens)
      return fail(HQEKV_E_ARG, "cache_migrate: destination %d must be stored densely", k);
    a.dst[k] = MigClass{dst[k].data, (half_t *)dst[k].scale, (half_t *)dst[k].zero, dst[k].idx, dst[k].n_tokens, dst[k].n_tokens, dst[k].bits, dst[k].layout};
    a.dst_begin[k] = (int32_t)total;
    total += dst[k].n_tokens / 32;
  }
  for (int k = n_dst; k <= HQEKV_MAX_SEGS; ++k) a.dst_begin[k] = (int32_t)total;
  if (total == 0) return HQEKV_OK;
  if (total >= (1 << 24)) return fail(HQEKV_E_UNSUPPORTED, "cache_migrate: %lld blocks (limit 2^24)", (long long)total);
  if (!plan) return fail(HQEKV_E_ARG, "cache_migrate: null plan");
  a.n_dst = n_dst;
  a.n_src = n_src;
  a.status = status;
  a.plan_src = plan;
  a.plan_pos = plan + total;
  const dim3 block(MIG_THREADS);
  if (is_k)
    hipLaunchKernelGGL(cache_migrate_kernel<true>, dim3((unsigned)((total + MIG_KB - 1) / MIG_KB), (unsigned)BH), block, 0,
                       (hipStream_t)stream, a, (int)D);
  else
    hipLaunchKernelGGL(cache_migrate_kernel<false>, dim3((unsigned)total, (unsigned)BH), block, 0, (hipStream_t)stream, a,
                       (int)D);
  return check_launch("cache_migrate_kernel");
}
