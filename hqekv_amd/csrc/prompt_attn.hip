// The prompt side of the attention layer (model/llama_hqe.py:141-188): causal attention over the whole prompt, and the
// probabilities of its last rows, which seed the importance ring.  The reference calls flash-attention for the first
// and a dense matmul + softmax over the last 20 query rows for the second; here both are matrix-core kernels for
// head_dim 128 in fp16 with fp32 accumulation, reading K and V once per query head through the caches (the query
// heads of one KV head are neighbours in the grid), without `repeat_kv` copies.
//
// Both kernels compute S^T = K . Q^T -- keys along M, queries along N of v_mfma_f32_32x32x16_f16 -- so that a lane
// owns ONE query (column lane % 32): the running maximum, the sum and the rescaling of the output are per-lane
// scalars, and the exponentials a lane holds (keys 8 g + 4 (lane / 32) + j of a 32-key tile, g = 0..3, j = 0..3) are
// already laid out as the B operand of the second product, O^T = V^T . P^T.  That product needs, per lane, eight
// KEYS of one channel (4 h + j and 8 + 4 h + j of a 16-key step, for lane half h): V stays row-major in LDS and the
// operand comes out of two transposing reads (ds_read_b64_tr_b16: a group of 16 lanes names four key rows x 32 bytes,
// every lane receives four consecutive keys of one channel).
#include "common.h"

namespace hq {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef __fp16 h4raw_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef __attribute__((address_space(3))) h4raw_t lds_h4_t;

constexpr int PA_D = 128;
constexpr int PA_WAVES = 4;
constexpr int PA_THREADS = 64 * PA_WAVES;
constexpr int PA_BR = 32 * PA_WAVES;   // query rows per workgroup
#ifndef HQ_PA_BC
#define HQ_PA_BC 32
#endif
constexpr int PA_BC = HQ_PA_BC;        // keys per tile: 32 (164 registers, 32 KB of LDS: three workgroups per CU) or 64 (two)
constexpr int PA_NS = PA_BC / 32;      // 32-key score tiles per key tile
constexpr int PA_WGS = PA_BC == 64 ? 2 : 3;

struct PromptArgs {
  const half_t *q, *k, *v;
  half_t *out;
  int64_t q_b, q_h, q_t;   // strides in elements; the channel stride is 1
  int64_t k_b, k_h, k_t;
  int64_t v_b, v_h, v_t;
  int64_t o_b, o_h, o_t;
  int32_t Hq, Hkv, T;
  float scale;
};


// A tile of keys goes from memory to LDS without passing through registers (`buffer_load_dwordx4 ... lds`: lane l's
// 16 bytes land at M0 + 16 l, so one wave instruction fills four 256-byte rows).  K and V are both row-major in LDS,
// [key][128 channels], unpadded; banks are spread by a swizzle of the 16-byte pieces inside a row, applied on the
// memory side: the lane that fills piece slot c of a row fetches piece c ^ (row % 16) of K, c ^ 4 (row % 4) of V.
// These loads are inline asm (the compiler makes every LDS access after the builtin form wait for all of them), so the
// wait -- vmcnt(0), once per tile, right before the barrier -- is explicit.
typedef int desc_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ desc_t make_desc(const void *base, uint32_t bytes) {   // `base` and `bytes` wave-uniform
  const uint64_t a = (uint64_t)(uintptr_t)base;
  desc_t d;
  d.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  d.y = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu));
  d.z = __builtin_amdgcn_readfirstlane((int)bytes);
  d.w = 0x00020000;
  return d;
}
__device__ __forceinline__ uint32_t lds_offset_of(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
__device__ __forceinline__ void dma_1k(uint32_t lds, desc_t d, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(lds), "v"(voff), "s"(d), "s"(soff) : "memory");
}
__device__ __forceinline__ void wait_all_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
struct PaSource {
  desc_t k, v;
  uint32_t k_lane, v_lane;   // this thread's byte offsets inside a tile (row tid / 16, swizzled piece)
  uint32_t k_row, v_row;     // bytes between two keys
};
// rows tid / 16 + 16 i of the tile; wave w's instruction i fills rows 16 i + 4 w .. + 3
__device__ __forceinline__ void pa_tile_dma(const PaSource &src, int k0, const half_t *ks, const half_t *vs, int w) {
  const uint32_t kb = lds_offset_of(ks) + (uint32_t)w * 1024u, vb = lds_offset_of(vs) + (uint32_t)w * 1024u;
#pragma unroll
  for (int i = 0; i < PA_BC / 16; ++i) {
    dma_1k(kb + 4096u * i, src.k, src.k_lane, (uint32_t)(k0 + 16 * i) * src.k_row);
    dma_1k(vb + 4096u * i, src.v, src.v_lane, (uint32_t)(k0 + 16 * i) * src.v_row);
  }
}

// S^T of one key tile for the wave's 32 queries: PA_NS score tiles of 32 keys, 16 fp32 values per lane each
__device__ __forceinline__ void pa_scores(const half_t *ks, const h8_t (&qreg)[8], int n, int h, f16_t (&sc)[PA_NS]) {
#pragma unroll
  for (int mt = 0; mt < PA_NS; ++mt) sc[mt] = (f16_t)(0.f);
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int piece = ((2 * s + h) ^ (n & 15)) * 8;   // (rows n and 32 + n share the swizzle)
#pragma unroll
    for (int mt = 0; mt < PA_NS; ++mt) {
      const h8_t kk = *reinterpret_cast<const h8_t *>(ks + (32 * mt + n) * PA_D + piece);
      sc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kk, qreg[s], sc[mt], 0, 0, 0);
    }
  }
}
template <bool CAUSAL>
__global__ __launch_bounds__(PA_THREADS, PA_WGS) void prompt_attn_kernel(PromptArgs a) {
  __shared__ __align__(16) half_t ks_all[2][PA_BC * PA_D];
  __shared__ __align__(16) half_t vs_all[2][PA_BC * PA_D];
  const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int qb = (int)gridDim.x - 1 - (int)blockIdx.x;   // the longest rows first
  const int q0 = qb * PA_BR;
  const int b = (int)blockIdx.y / a.Hq, hq = (int)blockIdx.y % a.Hq, hkv = hq / (a.Hq / a.Hkv);
  const int T = a.T;
  const half_t *qp = a.q + b * a.q_b + hq * a.q_h;
  const half_t *kp = a.k + b * a.k_b + hkv * a.k_h;
  const half_t *vp = a.v + b * a.v_b + hkv * a.v_h;
  const int my_q = q0 + 32 * w + n;
  // the lane's query row: 8 steps of 16 channels, of which it supplies 8 (by lane half)
  h8_t qreg[8];
  {
    const half_t *qr = qp + (int64_t)min(my_q, T - 1) * a.q_t + 8 * h;
#pragma unroll
    for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const h8_t *>(qr + 16 * s);
  }
  f16_t o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = (f16_t)(0.f);
  float m = -INFINITY, lsum = 0.f;
  const float sl2 = a.scale * 1.4426950408889634f;
  const int kend = CAUSAL ? min(T, q0 + PA_BR) : T;
  const int n_tiles = (kend + PA_BC - 1) / PA_BC;
  PaSource src;
  src.k = make_desc(kp, (uint32_t)((int64_t)T * a.k_t * 2));   // (below 4 GiB: checked by the host)
  src.v = make_desc(vp, (uint32_t)((int64_t)T * a.v_t * 2));
  src.k_row = (uint32_t)a.k_t * 2u;
  src.v_row = (uint32_t)a.v_t * 2u;
  {
    const uint32_t row = threadIdx.x >> 4, slot = threadIdx.x & 15;
    src.k_lane = row * src.k_row + ((slot ^ (row & 15)) * 16u);
    src.v_lane = row * src.v_row + ((slot ^ (4 * (row & 3))) * 16u);
  }
  // Two tiles in LDS, one barrier per tile: iteration j waits for its own requests of tile j (made an iteration ago),
  // passes the barrier -- now every wave's part of tile j is there and every wave has finished tile j - 1 -- requests
  // tile j + 1 into the buffer that tile j - 1 was read from, and works on tile j.
  // where this lane points the transposing reads of V: lane r of a group of 16 names key row 4h + r / 4 of a step and
  // the 8 bytes of channels 32 dt + 16 (n / 16) + 4 (r % 4) ..; the row's pieces are swizzled by 4 (row % 4) = 4 (r / 4)
  int v_off[4];
  {
    const int r = lane & 15, key = 4 * h + (r >> 2);
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const int piece = 4 * dt + 2 * (n >> 4) + ((r & 3) >> 1);
      v_off[dt] = key * PA_D + ((piece ^ (4 * (r >> 2))) * 8) + 4 * (r & 1);
    }
  }
  // (rows past the end of the prompt are outside the buffer descriptors: whatever such a row holds in LDS -- zeros from
  // this fill or an older tile's finite values -- meets an exponential that is exactly zero)
#pragma unroll
  for (int i = 0; i < PA_BC / 8; ++i) *reinterpret_cast<uint4 *>(&vs_all[0][0] + (threadIdx.x + PA_THREADS * i) * 8) = make_uint4(0, 0, 0, 0);
  __syncthreads();
  pa_tile_dma(src, 0, ks_all[0], vs_all[0], w);   // (a tile past the last one is fetched and never used)
  auto step = [&](int tile, const half_t *ks, const half_t *vs, half_t *ks_nxt, half_t *vs_nxt) {
    const int k0 = tile * PA_BC;
    wait_all_loads();   // this wave's part of tile j, requested an iteration ago
    __syncthreads();
    pa_tile_dma(src, k0 + PA_BC, ks_nxt, vs_nxt, w);   // in flight across the products
    // (a tile that lies after every query of this wave is worked through like any other: all its elements are masked,
    // the maximum stays and the exponentials are zeros; skipping it would cost a copy of the accumulators per tile)
    f16_t s[PA_NS];
    pa_scores(ks, qreg, n, h, s);
    const bool edge = (k0 + PA_BC > T) || (CAUSAL && k0 + PA_BC - 1 > q0 + 32 * w);   // some element of the tile is masked
    // the running maximum is kept in units of the scaled logit (base-2 exponent); a raw score enters as s * sl2
    if (edge) {   // (uniform per wave; one branch around all 32 selects)
      const int last_key = (CAUSAL ? min(my_q, T - 1) : T - 1) - k0 - 4 * h;   // the last visible key, relative to element r's base
#pragma unroll
      for (int mt = 0; mt < PA_NS; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (32 * mt + 8 * (r >> 2) + (r & 3) > last_key) s[mt][r] = -INFINITY;
    }
    float raw = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < PA_NS; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) raw = fmaxf(raw, s[mt][r]);
    float mx = fmaxf(m, raw * sl2);   // (sl2 > 0)
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // (the first tile always holds key 0, which no query masks: mx is finite from then on)
    // Per lane on purpose: a divergent branch keeps the accumulators where they are (inactive lanes must keep their
    // values, so the products are in place under the execution mask, skipped when no lane needs them); a wave-uniform
    // branch made the compiler copy all 64 accumulators per tile, and without a branch the 64 products are a quarter
    // of the tile's vector instructions.
    if (mx != m) {   // this query's maximum moved: rescale what it has added up so far
      const float alpha = __builtin_amdgcn_exp2f(m - mx);   // (the bare instruction: results below 2^-126 may flush to zero)
      lsum *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) o[dt] *= alpha;
      m = mx;
    }
    float part = 0.f;
    h8_t p[2 * PA_NS];
#pragma unroll
    for (int mt = 0; mt < PA_NS; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][r], sl2, -mx));
        part += e;
        p[2 * mt + (r >> 3)][r & 7] = (half_t)e;
      }
    lsum += part;
#pragma unroll
    for (int t = 0; t < 2 * PA_NS; ++t)
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        // V^T operand through the transposing LDS read: a group of 16 lanes names four key rows x 32 bytes and each
        // lane receives four consecutive keys of one channel; two reads (keys 4h + j, 8 + 4h + j) make the operand
        const half_t *src_lo = vs + v_off[dt] + 16 * t * PA_D;
        const h4raw_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_h4_t *)(src_lo));
        const h4raw_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_h4_t *)(src_lo + 8 * PA_D));
        h8_t av;
        __builtin_memcpy(&av, &lo, 8);
        __builtin_memcpy(reinterpret_cast<char *>(&av) + 8, &hi, 8);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, p[t], o[dt], 0, 0, 0);
      }
  };
  // two tiles per round, so that each half works on fixed buffers; an odd count runs one tile more, all of it masked
  for (int tile = 0; tile < n_tiles; tile += 2) {
    step(tile, ks_all[0], vs_all[0], ks_all[1], vs_all[1]);
    step(tile + 1, ks_all[1], vs_all[1], ks_all[0], vs_all[0]);
  }
  wait_all_loads();   // the last request (a tile nobody reads) must have landed before this workgroup's LDS can go to another
  lsum += __shfl_xor(lsum, 32, 64);
  if (my_q < T) {
    const float inv = 1.0f / lsum;
    half_t *orow = a.out + b * a.o_b + hq * a.o_h + (int64_t)my_q * a.o_t;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        h4_t y;
#pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = (half_t)(o[dt][4 * g + j] * inv);
        *reinterpret_cast<h4_t *>(orow + 32 * dt + 8 * g + 4 * h) = y;
      }
  }
}

// ---- probabilities of the last R <= 32 query rows, with the reference's roundings (model/llama_hqe.py:156-168):
// the product rounded to fp16, times the scale rounded to fp16, plus the mask rounded to fp16, floored at the most
// negative fp16, softmax in fp32, rounded to fp16.  One workgroup per (b, query head); its four waves deal the
// 32-key tiles round-robin and walk them twice: maximum and sum, then the probabilities.
struct LastRowsArgs {
  const half_t *q, *k;
  const half_t *mask;   // additive, (B, 1, R, T) with strides, or nullptr: causal
  half_t *probs;        // (B, Hq, R, T) contiguous
  int64_t q_b, q_h, q_t;
  int64_t k_b, k_h, k_t;
  int64_t m_b, m_r;
  int32_t Hq, Hkv, T, R;
  float scale;
  float2 *partial;      // (B * Hq, slices, 32) (maximum, sum) of a slice of the keys, or nullptr: one workgroup per head does it all
  int32_t slices;
};

// PHASE 0: one workgroup per (b, query head) walks all keys twice.  With the keys cut into slices (grid.y) for short
// prompts and small batches: PHASE 1 leaves each slice's (maximum, sum) per row in `partial`, PHASE 2 merges them and
// writes the slice's probabilities.
template <int PHASE>
__global__ __launch_bounds__(PA_THREADS, 2) void prompt_last_rows_kernel(LastRowsArgs a) {
  __shared__ float sh_m[PA_WAVES][32], sh_l[PA_WAVES][32];
  const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int b = (int)blockIdx.x / a.Hq, hq = (int)blockIdx.x % a.Hq, hkv = hq / (a.Hq / a.Hkv);
  const int T = a.T, R = a.R;
  const half_t *kp = a.k + b * a.k_b + hkv * a.k_h;
  const int row = min(n, R - 1);         // lanes past the last row repeat it and store nothing
  const int my_q = T - R + row;
  h8_t qreg[8];
  {
    const half_t *qr = a.q + b * a.q_b + hq * a.q_h + (int64_t)my_q * a.q_t + 8 * h;
#pragma unroll
    for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const h8_t *>(qr + 16 * s);
  }
  const half_t *mrow = a.mask ? a.mask + b * a.m_b + (int64_t)row * a.m_r : nullptr;
  const int all_tiles = (T + 31) / 32;
  const int per_slice = PHASE == 0 ? all_tiles : (all_tiles + a.slices - 1) / a.slices;
  const int tile0 = PHASE == 0 ? 0 : (int)blockIdx.y * per_slice, n_tiles = min(all_tiles, tile0 + per_slice);
  // the 16 scores of this lane for 32-key tile `tile`, as the reference's fp16 chain leaves them (in fp32)
  auto tile_scores = [&](int tile, float (&x)[16]) {
    const int key_row = min(32 * tile + n, T - 1);
    const half_t *kr = kp + (int64_t)key_row * a.k_t + 8 * h;
    f16_t s = (f16_t)(0.f);
#pragma unroll
    for (int st = 0; st < 8; ++st)
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const h8_t *>(kr + 16 * st), qreg[st], s, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 32 * tile + 8 * (r >> 2) + 4 * h + (r & 3);
      half_t v = (half_t)((float)(half_t)s[r] * a.scale);
      if (mrow) {
        v = (half_t)((float)v + (float)mrow[min(key, T - 1)]);
        v = (half_t)fmaxf((float)v, -65504.f);
        x[r] = key < T ? (float)v : -INFINITY;
      } else {
        x[r] = (key < T && key <= my_q) ? (float)v : -INFINITY;
      }
    }
  };
  float m = -INFINITY, l = 0.f;
  if (PHASE != 2) {
    for (int tile = tile0 + w; tile < n_tiles; tile += PA_WAVES) {
      float x[16];
      tile_scores(tile, x);
      float mx = m;
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, x[r]);
      if (mx == -INFINITY) continue;   // nothing but masked keys so far
      float part = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) part += __expf(x[r] - mx);
      l = l * __expf(m - mx) + part;
      m = mx;
    }
    // the two halves of the wave, then the four waves
    const float mo = __shfl_xor(m, 32, 64), lo = __shfl_xor(l, 32, 64);
    const float mx = fmaxf(m, mo);
    l = (m == -INFINITY ? 0.f : l * __expf(m - mx)) + (mo == -INFINITY ? 0.f : lo * __expf(mo - mx));
    m = mx;
    if (h == 0) {
      sh_m[w][n] = m;
      sh_l[w][n] = l;
    }
    __syncthreads();
    float mx2 = -INFINITY;
#pragma unroll
    for (int k = 0; k < PA_WAVES; ++k) mx2 = fmaxf(mx2, sh_m[k][n]);
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < PA_WAVES; ++k) tot += sh_m[k][n] == -INFINITY ? 0.f : sh_l[k][n] * __expf(sh_m[k][n] - mx2);
    m = mx2;
    l = tot;
    if (PHASE == 1) {
      if (threadIdx.x < 32) a.partial[((int64_t)blockIdx.x * a.slices + blockIdx.y) * 32 + n] = make_float2(m, l);
      return;
    }
  } else {   // merge the slices' statistics, in slice order
    const float2 *ps = a.partial + (int64_t)blockIdx.x * a.slices * 32 + n;
    for (int sl = 0; sl < a.slices; ++sl) m = fmaxf(m, ps[sl * 32].x);
    for (int sl = 0; sl < a.slices; ++sl) {
      const float2 v = ps[sl * 32];
      l += v.x == -INFINITY ? 0.f : v.y * __expf(v.x - m);
    }
  }
  const float inv = 1.0f / l;
  half_t *prow = a.probs + (((int64_t)b * a.Hq + hq) * R + row) * (int64_t)T;
  for (int tile = tile0 + w; tile < n_tiles; tile += PA_WAVES) {
    float x[16];
    tile_scores(tile, x);
    if (n >= R) continue;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int key = 32 * tile + 8 * g + 4 * h;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (key + j < T) prow[key + j] = (half_t)(__expf(x[4 * g + j] - m) * inv);
    }
  }
}

}  // namespace hq

using namespace hq;

static bool rows_16_byte_aligned(const void *p, int64_t s0, int64_t s1, int64_t s2) {
  return ((uintptr_t)p & 15) == 0 && s0 % 8 == 0 && s1 % 8 == 0 && s2 % 8 == 0;
}

extern "C" int hqekv_prompt_attn(const void *q, const int64_t *q_strides, const void *k, const int64_t *k_strides,
                                 const void *v, const int64_t *v_strides, void *out, const int64_t *out_strides, int64_t B,
                                 int64_t Hq, int64_t Hkv, int64_t T, int64_t D, float scale, int causal, void *stream) {
  if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !out_strides)
    return fail(HQEKV_E_ARG, "prompt_attn: null pointer");
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || T <= 0 || Hq % Hkv) return fail(HQEKV_E_ARG, "prompt_attn: need B, T > 0 and Hq %% Hkv == 0");
  if (!(scale > 0.f)) return fail(HQEKV_E_ARG, "prompt_attn: the scale must be positive");
  if (D != PA_D) return fail(HQEKV_E_UNSUPPORTED, "prompt_attn: head_dim %lld (supported: 128)", (long long)D);
  if (T > 0x7fffff00LL || B * Hq > 65535) return fail(HQEKV_E_UNSUPPORTED, "prompt_attn: T or B * Hq too large");
  if (!rows_16_byte_aligned(q, q_strides[0], q_strides[1], q_strides[2]) || !rows_16_byte_aligned(k, k_strides[0], k_strides[1], k_strides[2]) ||
      !rows_16_byte_aligned(v, v_strides[0], v_strides[1], v_strides[2]) || ((uintptr_t)out & 7) || out_strides[0] % 4 || out_strides[1] % 4 || out_strides[2] % 4)
    return fail(HQEKV_E_ALIGN, "prompt_attn: rows of q, k, v must be 16-byte aligned (of out: 8-byte)");
  // (the tiles of K and V are fetched through 32-bit buffer offsets from each head's first row)
  if (T * k_strides[2] * 2 >= (1LL << 32) || T * v_strides[2] * 2 >= (1LL << 32) || k_strides[2] <= 0 || v_strides[2] <= 0)
    return fail(HQEKV_E_UNSUPPORTED, "prompt_attn: a head's K or V rows must span less than 4 GiB (T * token stride * 2 bytes)");
  PromptArgs a;
  a.q = (const half_t *)q; a.k = (const half_t *)k; a.v = (const half_t *)v; a.out = (half_t *)out;
  a.q_b = q_strides[0]; a.q_h = q_strides[1]; a.q_t = q_strides[2];
  a.k_b = k_strides[0]; a.k_h = k_strides[1]; a.k_t = k_strides[2];
  a.v_b = v_strides[0]; a.v_h = v_strides[1]; a.v_t = v_strides[2];
  a.o_b = out_strides[0]; a.o_h = out_strides[1]; a.o_t = out_strides[2];
  a.Hq = (int32_t)Hq; a.Hkv = (int32_t)Hkv; a.T = (int32_t)T; a.scale = scale;
  const dim3 grid((unsigned)((T + PA_BR - 1) / PA_BR), (unsigned)(B * Hq));
  if (causal) hipLaunchKernelGGL(prompt_attn_kernel<true>, grid, dim3(PA_THREADS), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(prompt_attn_kernel<false>, grid, dim3(PA_THREADS), 0, (hipStream_t)stream, a);
  return check_launch("prompt_attn");
}

static int last_rows_slices(int64_t B, int64_t Hq, int64_t T) {
  // enough workgroups for the chip when there are few heads; a slice keeps at least 2048 keys
  int64_t s = (512 + B * Hq - 1) / (B * Hq);
  const int64_t most = (T + 2047) / 2048;
  if (s > most) s = most;
  if (s > 64) s = 64;
  return s < 1 ? 1 : (int)s;
}

extern "C" int64_t hqekv_prompt_last_rows_workspace_bytes(int64_t B, int64_t Hq, int64_t T) {
  if (B <= 0 || Hq <= 0 || T <= 0) return -1;
  const int sl = last_rows_slices(B, Hq, T);
  return sl > 1 ? B * Hq * sl * 32 * (int64_t)sizeof(float2) : 0;
}

extern "C" int hqekv_prompt_last_rows(const void *q, const int64_t *q_strides, const void *k, const int64_t *k_strides,
                                      const void *mask, const int64_t *mask_strides, void *probs, int64_t B, int64_t Hq,
                                      int64_t Hkv, int64_t T, int64_t D, int64_t R, float scale, void *workspace,
                                      int64_t workspace_bytes, void *stream) {
  if (!q || !k || !probs || !q_strides || !k_strides || (mask && !mask_strides)) return fail(HQEKV_E_ARG, "prompt_last_rows: null pointer");
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || T <= 0 || Hq % Hkv || R <= 0 || R > 32 || R > T)
    return fail(HQEKV_E_ARG, "prompt_last_rows: need B > 0, Hq %% Hkv == 0 and 0 < R <= min(32, T)");
  if (D != PA_D) return fail(HQEKV_E_UNSUPPORTED, "prompt_last_rows: head_dim %lld (supported: 128)", (long long)D);
  if (T > 0x7fffff00LL || B * Hq > 0x7fffffffLL) return fail(HQEKV_E_UNSUPPORTED, "prompt_last_rows: T or B * Hq too large");
  if (!rows_16_byte_aligned(q, q_strides[0], q_strides[1], q_strides[2]) || !rows_16_byte_aligned(k, k_strides[0], k_strides[1], k_strides[2]))
    return fail(HQEKV_E_ALIGN, "prompt_last_rows: rows of q and k must be 16-byte aligned");
  LastRowsArgs a;
  a.q = (const half_t *)q; a.k = (const half_t *)k; a.mask = (const half_t *)mask; a.probs = (half_t *)probs;
  a.q_b = q_strides[0]; a.q_h = q_strides[1]; a.q_t = q_strides[2];
  a.k_b = k_strides[0]; a.k_h = k_strides[1]; a.k_t = k_strides[2];
  a.m_b = mask ? mask_strides[0] : 0; a.m_r = mask ? mask_strides[1] : 0;
  a.Hq = (int32_t)Hq; a.Hkv = (int32_t)Hkv; a.T = (int32_t)T; a.R = (int32_t)R; a.scale = scale;
  // the keys in slices when the caller brought room for the slices' statistics; else one workgroup per head
  const int sl = last_rows_slices(B, Hq, T);
  const int64_t need = hqekv_prompt_last_rows_workspace_bytes(B, Hq, T);
  if (sl > 1 && workspace && workspace_bytes >= need) {
    if ((uintptr_t)workspace & 7) return fail(HQEKV_E_ALIGN, "prompt_last_rows: workspace not 8-byte aligned");
    a.partial = (float2 *)workspace;
    a.slices = sl;
    const dim3 grid((unsigned)(B * Hq), (unsigned)sl);
    hipLaunchKernelGGL(prompt_last_rows_kernel<1>, grid, dim3(PA_THREADS), 0, (hipStream_t)stream, a);
    hipLaunchKernelGGL(prompt_last_rows_kernel<2>, grid, dim3(PA_THREADS), 0, (hipStream_t)stream, a);
  } else {
    a.partial = nullptr;
    a.slices = 1;
    hipLaunchKernelGGL(prompt_last_rows_kernel<0>, dim3((unsigned)(B * Hq)), dim3(PA_THREADS), 0, (hipStream_t)stream, a);
  }
  return check_launch("prompt_last_rows");
}
