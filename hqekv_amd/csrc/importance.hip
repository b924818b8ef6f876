// What the cache policy ranks blocks by, on the device: a token's importance from the ring of recent attention rows,
// the mean importance of every 32-token block (K ranking), the same weighted with the V token ranges (V ranking), and
// the ranges of new V tokens -- the reference's short chains of torch reductions (model/public_func.py:58-106,217-221;
// quant/hqe_2.py:510-518), one launch each.  The results decide rankings, so every fp16 rounding and every order of
// additions is torch's own on the GPU, measured with order-sensitive inputs and checked against torch on the device:
//   * a sum over the ROWS of a matrix (the 20 ring rows, the batch, the KV heads) is taken by one thread per column
//     with four interleaved fp32 accumulators -- row k goes to accumulator k mod 4 -- added as ((a0 + a1) + a2) + a3;
//   * a sum over 32 CONTIGUOUS values is a balanced tree over adjacent pairs in fp32;
//   * every intermediate tensor is fp16: each step rounds to nearest even; a division by 32 is a multiplication by
//     its (exact) reciprocal; tensor / tensor is the correctly rounded fp32 quotient.
#include "common.h"

#pragma clang fp contract(off)

namespace hq {

constexpr int IMP_THREADS = 256;

template <typename Load>
__device__ __forceinline__ float sum_rows_like_torch(int n_rows, Load &&load) {
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  int r = 0;
  for (; r + 3 < n_rows; r += 4) {
    a0 += load(r);
    a1 += load(r + 1);
    a2 += load(r + 2);
    a3 += load(r + 3);
  }
  if (r < n_rows) a0 += load(r);
  if (r + 1 < n_rows) a1 += load(r + 1);
  if (r + 2 < n_rows) a2 += load(r + 2);
  return ((a0 + a1) + a2) + a3;
}

// lane 0 of every group of 32 lanes ends up with the adjacent-pairs tree sum of the group's values
__device__ __forceinline__ float tree_sum_32(float v) {
#pragma unroll
  for (int off = 1; off < 32; off <<= 1) v += __shfl_down(v, off, 32);
  return v;
}

// importance[c] = rnd16(rnd16(sum of ring column c) / min(rows, n - c)), divided by 32 in place as the ranking helper
// does (model/public_func.py:94-96); block score = sum of the block's 32 divided values.
__global__ __launch_bounds__(IMP_THREADS) void importance_scores_kernel(const half_t *__restrict__ ring, int rows,
                                                                       int64_t max_len, int64_t n, int64_t total,
                                                                       half_t *__restrict__ imp_out,
                                                                       half_t *__restrict__ scores) {
  const int64_t c = (int64_t)blockIdx.x * IMP_THREADS + threadIdx.x;
  float v = 0.f;
  if (c < total) {
    const half_t *col = ring + c;
    const half_t s = (half_t)sum_rows_like_torch(rows, [&](int r) { return (float)col[(int64_t)r * max_len]; });
    const int64_t seen_i = n - c < (int64_t)rows ? n - c : (int64_t)rows;
    const half_t seen = (half_t)(float)seen_i;
    const half_t imp = (half_t)((float)s / (float)seen);
    const half_t d = (half_t)((float)imp * 0.03125f);
    imp_out[c] = d;
    v = (float)d;
  }
  v = tree_sum_32(v);
  if ((threadIdx.x & 31) == 0 && c < total) scores[c >> 5] = (half_t)v;
}

// block scores of x[c] (* w[c]) / 32
__global__ __launch_bounds__(IMP_THREADS) void weighted_scores_kernel(const half_t *__restrict__ x,
                                                                     const half_t *__restrict__ w, int64_t total,
                                                                     half_t *__restrict__ scores) {
  const int64_t c = (int64_t)blockIdx.x * IMP_THREADS + threadIdx.x;
  float v = 0.f;
  if (c < total) {
    half_t t = x[c];
    if (w) t = (half_t)((float)t * (float)w[c]);
    v = (float)(half_t)((float)t * 0.03125f);
  }
  v = tree_sum_32(v);
  if ((threadIdx.x & 31) == 0 && c < total) scores[c >> 5] = (half_t)v;
}

// out[t] = sum over heads of rnd16(sum over batch of rnd16(max_d - min_d)), one workgroup per token
constexpr int RANGE_MAX_ROWS = 1024;
__global__ __launch_bounds__(IMP_THREADS) void token_range_kernel(const half_t *__restrict__ v, int B, int H, int64_t T,
                                                                 int D, int64_t slab_tokens, half_t *__restrict__ out) {
  __shared__ half_t r[RANGE_MAX_ROWS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int row = wave; row < B * H; row += IMP_THREADS / 64) {
    const half_t *p = v + ((int64_t)row * slab_tokens + t) * D;
    float mx = -INFINITY, mn = INFINITY;
    for (int d = lane; d < D; d += 64) {
      const float x = (float)p[d];
      mx = fmaxf(mx, x);
      mn = fminf(mn, x);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      mx = fmaxf(mx, xor_f(mx, m));
      mn = fminf(mn, xor_f(mn, m));
    }
    if (lane == 0) r[row] = (half_t)(mx - mn);   // both are fp16 numbers: the fp32 difference rounded once
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const float s = sum_rows_like_torch(H, [&](int h) {
      if (B == 1) return (float)r[h];
      return (float)(half_t)sum_rows_like_torch(B, [&](int b) { return (float)r[b * H + h]; });
    });
    out[t] = (half_t)s;
  }
}

}  // namespace hq

using namespace hq;

extern "C" int hqekv_importance_scores(const void *ring, int32_t rows, int64_t max_len, int64_t n, int64_t total,
                                       void *importance_out, void *scores_out, void *stream) {
  if (!ring || !importance_out || !scores_out) return fail(HQEKV_E_ARG, "importance_scores: null pointer");
  if (rows <= 0 || total <= 0 || total > n || n > max_len || total % 32)
    return fail(HQEKV_E_ARG, "importance_scores: need 0 < total <= n <= max_len, total a multiple of 32, rows > 0");
  const int64_t blocks = (total + IMP_THREADS - 1) / IMP_THREADS;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_UNSUPPORTED, "importance_scores: too many columns");
  hipLaunchKernelGGL(importance_scores_kernel, dim3((unsigned)blocks), dim3(IMP_THREADS), 0, (hipStream_t)stream,
                     (const half_t *)ring, (int)rows, max_len, n, total, (half_t *)importance_out, (half_t *)scores_out);
  return check_launch("importance_scores");
}

extern "C" int hqekv_weighted_block_scores(const void *x, const void *weights, int64_t total, void *scores_out,
                                           void *stream) {
  if (!x || !scores_out) return fail(HQEKV_E_ARG, "weighted_block_scores: null pointer");
  if (total <= 0 || total % 32) return fail(HQEKV_E_ARG, "weighted_block_scores: total must be a positive multiple of 32");
  const int64_t blocks = (total + IMP_THREADS - 1) / IMP_THREADS;
  if (blocks > 0x7fffffffLL) return fail(HQEKV_E_UNSUPPORTED, "weighted_block_scores: too many columns");
  hipLaunchKernelGGL(weighted_scores_kernel, dim3((unsigned)blocks), dim3(IMP_THREADS), 0, (hipStream_t)stream,
                     (const half_t *)x, (const half_t *)weights, total, (half_t *)scores_out);
  return check_launch("weighted_block_scores");
}

extern "C" int hqekv_token_range(const void *v, int64_t B, int64_t H, int64_t T, int64_t D, int64_t slab_tokens,
                                 void *out, void *stream) {
  if (!v || !out) return fail(HQEKV_E_ARG, "token_range: null pointer");
  if (B <= 0 || H <= 0 || T <= 0 || D <= 0 || slab_tokens < T)
    return fail(HQEKV_E_ARG, "token_range: empty shape or slab_tokens < T");
  if (B * H > RANGE_MAX_ROWS) return fail(HQEKV_E_UNSUPPORTED, "token_range: B * H = %lld > %d", (long long)(B * H), RANGE_MAX_ROWS);
  if (T > 0x7fffffffLL || D > 0x7fffffffLL) return fail(HQEKV_E_UNSUPPORTED, "token_range: T or D too large");
  hipLaunchKernelGGL(token_range_kernel, dim3((unsigned)T), dim3(IMP_THREADS), 0, (hipStream_t)stream, (const half_t *)v,
                     (int)B, (int)H, T, (int)D, slab_tokens, (half_t *)out);
  return check_launch("token_range");
}
