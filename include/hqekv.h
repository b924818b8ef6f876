/*
 * libhqekv -- C ABI of the MI355X (gfx950) quantized-KV decode-attention path.
 *
 * Plain pointers and sizes only: every pointer is a DEVICE pointer unless stated otherwise,
 * `stream` is a hipStream_t passed as void* (NULL = the null stream).  The library never
 * allocates or frees device memory, never synchronises, never switches device and keeps no
 * pointer after a call returns.  Outputs and workspaces are owned by the caller.
 *
 * Return value of every int function: 0 = ok, < 0 = invalid argument (HQEKV_E_*),
 * > 0 = a hipError_t raised by the launch.  hqekv_last_error() returns a thread-local
 * description of the last non-zero return.
 *
 * Storage layouts are the reference's cache layouts, consumed as stored (no transposes):
 *   K class, b bits : code (B,Hkv,D,T/pf) int32, scale/zero (B,Hkv,D,T/32) fp16, pf = 32/b
 *   V class, b bits : code (B,Hkv,T,D/pf) int32, scale/zero (B,Hkv,T,D/32) fp16
 *   fp16 K class    : (B,Hkv,D,T) fp16 (channel-major);  fp16 V class: (B,Hkv,T,D)
 *   residual new_K / new_V : (B,Hkv,T,D) fp16 (token-major)
 * Codes are packed LSB first: word j holds elements j*pf .. j*pf+pf-1 of the last axis.
 * b is 8, 4, 2 or 1: the 1-bit class is the uniform one of the reference's 'uniform_group' strategy
 * (quant/hqe_matmul.py:375-377, quant/hqe_2.py:482-484; 32 codes per word, qmax 1), which the decode
 * layer's count repair feeds even with a zero 1-bit share (model/public_func.py:259-268, start_idx 4).
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference checkout).
 */
#ifndef HQEKV_H
#define HQEKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HQEKV_OK 0
#define HQEKV_E_ARG (-1)      /* bad size / bits / null pointer            */
#define HQEKV_E_ALIGN (-2)    /* pointer or stride not aligned as required */
#define HQEKV_E_WORKSPACE (-3)/* workspace too small                       */
#define HQEKV_E_UNSUPPORTED (-4)

#define HQEKV_MAX_SEGS 8
#define HQEKV_GROUP 32

int hqekv_version(void);
const char *hqekv_last_error(void);

/* ------------------------------------------------------------------ quantise / pack
 * Replaces uniform_group_quantize_pack_last_dim (quant/pack_unpack.py:156-193: the
 * min/max/scale/sub/div/clamp/round torch chain plus the Triton _pack_along_last_dim
 * kernel at :16-51) with one pass.
 *
 * x is (n_outer, n_rows, L) fp16 with a contiguous last axis; groups of 32 along L.
 * Strides are in ELEMENTS of the respective array (fp16 for x/scale/zero, int32 words for
 * code), so the outputs may be windows of larger, capacity-sized cache buffers (append).
 * Requires L % 32 == 0, x 16-byte aligned rows (x strides % 8 == 0), bits in {1, 2, 4, 8}.
 */
int hqekv_quant_pack_rows(const void *x, int64_t x_outer_stride, int64_t x_row_stride,
                          void *code, int64_t code_outer_stride, int64_t code_row_stride,
                          void *scale, void *zero, int64_t sz_outer_stride, int64_t sz_row_stride,
                          int64_t n_outer, int64_t n_rows, int64_t L, int bits, void *stream);

/* Same quantiser for K handed over token-major: x is (n_outer, T, D) fp16 (what the model
 * produces), groups are 32 consecutive TOKENS of one channel, outputs are channel-major:
 * code (n_outer, D, T/pf), scale/zero (n_outer, D, T/32).  Replaces the
 * `.transpose(2, 3)` + reshape copy + quantiser of quant_new_K (quant/hqe_2.py:31-35).
 * Requires T % 32 == 0, D % 2 == 0.
 */
int hqekv_quant_pack_k_tokenmajor(const void *x, int64_t x_outer_stride, int64_t x_token_stride,
                                  void *code, int64_t code_outer_stride, int64_t code_row_stride,
                                  void *scale, void *zero, int64_t sz_outer_stride, int64_t sz_row_stride,
                                  int64_t n_outer, int64_t T, int64_t D, int bits, void *stream);

/* Replaces uniform_group_dequantize_unpack_last_dim (quant/pack_unpack.py:316-333):
 * out = rnd16(rnd16(fp16(code) * scale) + zero), (n_outer, n_rows, L) fp16.
 * scale == NULL: plain unpack_along_last_dim (quant/pack_unpack.py:255-295), codes as fp16.
 */
int hqekv_dequant_unpack_rows(const void *code, int64_t code_outer_stride, int64_t code_row_stride,
                              const void *scale, const void *zero, int64_t sz_outer_stride,
                              int64_t sz_row_stride, void *out, int64_t out_outer_stride,
                              int64_t out_row_stride, int64_t n_outer, int64_t n_rows, int64_t L,
                              int bits, void *stream);

/* The 1-bit normal-quantile class of the 'high_uniform_group_low_normal_group' strategy: replaces
 * normal_group_quantize_pack_last_dim / normal_group_dequantize_unpack_last_dim with bit == 1
 * (quant/pack_unpack.py:218-253, 356-376; 2-entry tables of :6-14: bounds [0, inf], centres -+0.6745).
 * Same shapes, strides and alignment rules as the uniform entry points above, 32 codes per word;
 * `stdv` / `meanv` take the places of scale / zero (unbiased std and mean of each group, fp16).
 * code = [rnd16(rnd16(x - mean) / std) > 0]; dequantised x = rnd16(rnd16(+-fp16(0.6745) * std) + mean).
 */
int hqekv_normal1_quant_pack_rows(const void *x, int64_t x_outer_stride, int64_t x_row_stride,
                                  void *code, int64_t code_outer_stride, int64_t code_row_stride,
                                  void *stdv, void *meanv, int64_t sz_outer_stride, int64_t sz_row_stride,
                                  int64_t n_outer, int64_t n_rows, int64_t L, void *stream);
int hqekv_normal1_quant_pack_k_tokenmajor(const void *x, int64_t x_outer_stride, int64_t x_token_stride,
                                          void *code, int64_t code_outer_stride, int64_t code_row_stride,
                                          void *stdv, void *meanv, int64_t sz_outer_stride,
                                          int64_t sz_row_stride, int64_t n_outer, int64_t T, int64_t D,
                                          void *stream);
int hqekv_normal1_dequant_unpack_rows(const void *code, int64_t code_outer_stride, int64_t code_row_stride,
                                      const void *stdv, const void *meanv, int64_t sz_outer_stride,
                                      int64_t sz_row_stride, void *out, int64_t out_outer_stride,
                                      int64_t out_row_stride, int64_t n_outer, int64_t n_rows, int64_t L,
                                      void *stream);

/* No counterpart in the reference: a device-side proof obligation of the quantiser above.  The kernels
 * evaluate the reference's v = u / scale (quant/pack_unpack.py:173, fp16 operands, fp32 divide, fp16
 * result) as u * (1/scale); this call compares the two over all 2^32 pairs of fp16 bit patterns.
 * counts: 4 x uint64 on the device, zeroed by the caller.  [0] pairs whose 8-bit code
 * rne(clamp(v, 0, 255)) differs (the 4- and 2-bit codes are min(code8, qmax)), [1] the same with both sign
 * bits clear (the quantiser's domain), [2] pairs whose fp16 quotient differs at all, [3] the largest |v|
 * (fp16 bit pattern) among those: below 0x0400, i.e. only ties among fp16 denormals, which all round to
 * code 0.
 */
int hqekv_selftest_quant_division(void *counts, void *stream);

/* No counterpart in the reference: checks the wave-wide reductions the attention kernels are built on
 * (DPP steps inside a row of 16 lanes, lane-row swaps across rows) on caller-supplied data.
 * in: (n_waves, 64) fp32; out: (n_waves, 4) fp32 = sum, max, and the same two through plain shuffles.
 */
int hqekv_selftest_wave_reduce(const void *in, void *out, int64_t n_waves, void *stream);

/* No counterpart in the reference: the measurement yardstick.  One launch of `n_workgroups` workgroups that only reads
 * `bytes` bytes at `src` (16-byte loads, eight in flight per lane) and XORs them into `sum` (n_workgroups uint32,
 * device, so the reads cannot be elided).  Its duration, launch included, is the floor for any kernel that must read
 * the same bytes once; the benchmark prints it beside the decode kernels' figures.  src 16-byte aligned, bytes a
 * multiple of 16, n_workgroups in [1, 65535].
 */
int hqekv_selftest_stream_read(const void *src, int64_t bytes, void *sum, int64_t n_workgroups, void *stream);

/* Replaces pack_along_last_dim (quant/pack_unpack.py:16-70): q is (n_rows, L) int32 codes,
 * code is (n_rows, L/pf) int32, both contiguous. */
int hqekv_pack_i32(const void *q, void *code, int64_t n_rows, int64_t L, int bits, void *stream);

/* ------------------------------------------------------------------ per-class GEMV
 * Replaces gemv_forward_cuda_uniform_group (quant/csrc/gemv_cuda.h:46-54, launched from
 * cuda_bmm_fA_qB_uniform_group, quant/matmul.py:263-299) and
 * gemv_forward_cuda_wv_uniform_group (gemv_cuda.h:235-243), WITHOUT the three
 * transpose().contiguous() copies of matmul.py:293-295:
 *
 *   out[b,hq,n] = sum_k fA[b,hq,k] * (scale[b,hkv,k,n/32] * code[b,hkv,k,n] + zero[b,hkv,k,n/32])
 *
 * fA (B,Hq,K) fp16, code (B,Hkv,K,N/pf) int32, scale/zero (B,Hkv,K,N/32) fp16, out (B,Hq,N)
 * fp16; hkv = hq / (Hq/Hkv).  fp32 accumulation, one rounding to fp16.
 * q.K^T is K = head_dim, N = tokens;  p.V is K = tokens, N = head_dim.
 * `workspace` is needed only when hqekv_gemv_workspace_bytes() > 0 (split-K partials).
 */
int64_t hqekv_gemv_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N, int bits);
int hqekv_gemv_uniform_group(const void *fA, const void *code, const void *scale, const void *zero,
                             void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N,
                             int bits, void *workspace, int64_t workspace_bytes, void *stream);

/* The same GEMV over a class in normal-quantile coding.  Replaces gemv_forward_cuda_normalize_group and
 * gemv_forward_cuda_wv_normalize_group (quant/csrc/gemv_cuda.h; launched from cuda_bmm_fA_qB_normal_group,
 * quant/matmul.py:72-95, and cuda_bmm_fA_qB_wv_normal_group, :147-170), which the attention glue calls for the
 * 1-bit class under 'high_uniform_group_low_normal_group' (quant/hqe_matmul.py:372,424):
 *
 *   out[b,hq,n] = sum_k fA[b,hq,k] * rnd16(rnd16(centre[code[b,hkv,k,n]] * std[b,hkv,k,n/32]) + mean[b,hkv,k,n/32])
 *
 * with the 2-entry table centre = -+fp16(0.6745) (quant/pack_unpack.py:6-14).  Shapes, dtypes and workspace
 * as above (hqekv_gemv_workspace_bytes with the same sizes); `bits` must be 1, the only width the path uses.
 */
int hqekv_gemv_normal_group(const void *fA, const void *code, const void *stdv, const void *meanv,
                            void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t K, int64_t N,
                            int bits, void *workspace, int64_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------ hybrid (all classes, one launch)
 * One segment = one precision class of one layer's cache.  `idx` maps element j of the class
 * to its position in the compacted sequence (int64, shared by all batch rows and heads,
 * quant/csrc/gemv_cuda_uniform.cu:945); idx == NULL means position = pos_base + j (used for
 * the fp16 residual at the tail).  Evicted tokens are simply absent from every segment.
 */
#define HQEKV_LAYOUT_TOKEN_MAJOR 1 /* K segment with bits == 16 stored (B,Hkv,T,D): the residual new_K   */
#define HQEKV_LAYOUT_NORMAL1 2     /* bits == 1 only: normal-quantile coding, scale = std, zero = mean:  */
                                   /* x = rnd16(rnd16(+-0.6745 * std) + mean), the 1-bit class of the   */
                                   /* 'high_uniform_group_low_normal_group' strategy                    */
                                   /* (quant/pack_unpack.py:356-376, quant/hqe_matmul.py:371-374)       */
typedef struct hqekv_seg {
  int32_t bits;          /* 16, 8, 4, 2 or 1                                           */
  int32_t layout;        /* HQEKV_LAYOUT_*: 0 = as listed at the top of this file       */
  int64_t n_tokens;      /* K side: multiple of 32 unless bits == 16; V side: any       */
  int64_t pos_base;      /* used when idx == NULL                                      */
  const void *data;      /* codes (int32) or fp16 values                               */
  const void *scale;     /* NULL when bits == 16                                       */
  const void *zero;
  const int64_t *idx;    /* (n_tokens) or NULL                                         */
  int64_t slab_tokens;   /* token-major segments only (the fp16 residual of either side, every V class -- codes, scale
                            and zero alike): token rows between two (b, kv head) slabs in memory when the segment is a
                            window of a longer, capacity-sized buffer; 0 = n_tokens (dense)        */
} hqekv_seg;

/* Replaces gemv_forward_cuda_qk_group_hq (quant/csrc/gemv_cuda.h:78-109; kernel
 * quant/csrc/gemv_cuda_uniform.cu:941-1228), i.e. cuda_bmm_forward_qk_group_hq
 * (quant/matmul.py:351-434): raw scores q.K^T scattered through idx.
 * q (B,Hq,D) fp16 -> scores (B,Hq,Tall) fp16 (row stride Tall).  `segs` is a HOST pointer.
 */
int hqekv_qk_hybrid(const hqekv_seg *segs, int nseg, const void *q, void *scores, int64_t B,
                    int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall, void *stream);

/* Replaces the torch epilogue of qkv_matmul (quant/quant_matmul_hq.py:100-103):
 * w = rnd16(w * (1/sqrt(D))) ; w += mask ; w = max(w, -65504) ; softmax in fp32 ; round to fp16.
 * In place on scores (B*Hq rows of Tall).  mask may be NULL; otherwise fp16 with
 * mask_row_stride elements between (b,hq) rows (0 = one row broadcast to all).
 */
int hqekv_scale_softmax(void *scores, const void *mask, int64_t mask_row_stride, int64_t n_rows,
                        int64_t Tall, float inv_sqrt_d, void *stream);

/* Replaces gemv_forward_cuda_wv_group_hq (quant/csrc/gemv_cuda.h:139-170; kernel
 * quant/csrc/gemv_cuda_wv_uniform.cu:347-745), i.e. cuda_bmm_forward_wv_group_hq
 * (quant/matmul.py:507-579): out[b,hq,:] = sum over segments of p[b,hq,idx[j]] * V[j,:].
 * p (B,Hq,Tall) fp16, out (B,Hq,D) fp16.  Split-K over tokens with a deterministic,
 * fixed-order combine (no float atomics).  `segs` is a HOST pointer.
 */
int64_t hqekv_pv_workspace_bytes(const hqekv_seg *segs, int nseg, int64_t B, int64_t Hq,
                                 int64_t Hkv, int64_t D);
int hqekv_pv_hybrid(const hqekv_seg *segs, int nseg, const void *p, void *out, int64_t B,
                    int64_t Hq, int64_t Hkv, int64_t D, int64_t Tall, void *workspace,
                    int64_t workspace_bytes, void *stream);

/* The whole decode-attention layer-step on one stream.  Replaces qkv_matmul / qkv_matmul_hq
 * (quant/quant_matmul_hq.py:23-174) and qkv_matmul_hqe_2 (quant/hqe_matmul.py:354-451).
 * attn_weights (B,Hq,Tall) fp16 receives the probabilities (the caller's importance tracker needs
 * them, model/llama_hqe.py:200); attn_out is (B,Hq,D) fp16.
 *
 * flags = 0: three launches plus the combine (qk_hybrid -> scale_softmax -> pv_hybrid), valid for any
 *   idx arrays and any mask.
 * flags & HQEKV_FUSE_SOFTMAX: no softmax launch.  The q.K^T launch stores scaled logits and per-tile softmax
 *   statistics, the p.V launch normalises while it gathers; the fixed-order combine stays a third,
 *   small launch.  REQUIRES that the idx arrays of the K segments, and those of the V segments, each cover
 *   every position in [0, Tall) exactly once (true for every cache the reference's cache policy builds);
 *   taken only when mask == NULL and both segment lists hold exactly Tall tokens, otherwise the call
 *   silently runs the flags = 0 path.
 * The workspace must hold hqekv_decode_workspace_bytes() bytes, 256-byte aligned; its contents need
 * not be initialised and are not preserved.  Calls that share a workspace must not overlap in time.
 * HQEKV_ONLY_QK / HQEKV_ONLY_PV / HQEKV_ONLY_COMBINE run one part of the call (q.K^T [+ softmax] / the p.V
 * kernel / the combine) so that each can be timed on its own; the later parts expect the earlier ones to
 * have run on the same buffers.
 * HQEKV_QK_TILING(n): which q.K^T tiling the call uses, n = 0 (default) chooses by launch size; any other
 * value forces one of the tilings listed below, whatever the size -- results agree to the stated tolerance
 * (the summation order over head_dim differs), so tests and measurements can name a tiling per call.
 */
#define HQEKV_FUSE_SOFTMAX 1
#define HQEKV_SEPARATE_COMBINE 2 /* always sum the split-K partials with a launch of their own                       */
#define HQEKV_FOLD_COMBINE 4     /* let the last p.V workgroup of each (b, kv head) sum them whenever there are at
                                    most 64 chunks; by default that is done only for long launches (>= 2^21 V token
                                    rows), where it saves more than it costs.  Both ways add in the same order and
                                    give the same bits                                                            */
#define HQEKV_TWO_STEP_DEQUANT 8  /* The kernels read a code c out of a packed word as the fp16 number bias + c.  The
                                    one-wave q.K^T tilings turn a tile whose scales are all below 32 in magnitude into
                                    c * s with one fused multiply-add, (bias + c) * s - bias * s (bias * s is exact
                                    there, so the product is rounded once, like the reference's), and any other tile
                                    with a subtraction and a multiplication.  This flag takes the second route for
                                    every tile; the bits are the same, and tests compare the two                  */
#define HQEKV_QK_TILING(n) (((n) & 0xf) << 4)
#define HQEKV_QK_TILING_8WAVES 1 /* 512-token tile, head_dim split over 8 waves (launches of <= 1024 tiles) */
#define HQEKV_QK_TILING_4WAVES 2 /* 512-token tile, head_dim split over 4 waves                              */
#define HQEKV_QK_TILING_WAVE512 3 /* one wave per 512-token tile, no split of head_dim (launches of > 1024 tiles;
                                     needs head_dim 128 and fp16 classes of a multiple of 8 tokens)          */
#define HQEKV_QK_TILING_WAVE256 4 /* one wave per 256-token tile: twice the waves per SIMD (same requirements)  */
#define HQEKV_ONLY_QK 0x100
#define HQEKV_ONLY_PV 0x200
#define HQEKV_ONLY_COMBINE 0x400
/* Form of the inner products of both GEMV launches.  With four query heads per KV head (Hq/Hkv == 4) the products of
 * the dequantised values with the query (or with the probabilities) can run on the matrix cores: one 4x4x4 fp16 matrix
 * instruction per four elements of the reduction axis and lane, in place of eight two-element dot products on the
 * vector ALU.  The dequantised values are the same bits either way, products are exact and accumulation is fp32 in
 * both; only the order of the additions differs.  Neither flag: the library's default for the shape.
 * Head ratios (Hq up to 65535): the kernels exist for 1 to 8 query heads per KV head; a larger ratio, up to 64, is served in slices of
 * at most eight heads (12 = 8 + 4, 13 = 8 + 5, ...), one launch per slice and GEMV (each reads the cache again), a
 * slice of four in the form the flags name.  HQEKV_DOT_MFMA with a ratio of 1-3 or 5-8 returns HQEKV_E_UNSUPPORTED. */
#define HQEKV_DOT_MFMA 0x800
#define HQEKV_DOT_VALU 0x1000
/* Run the q.K^T launch alone and leave the RAW fp16 scores in attn_weights (no scaling, no softmax), with the tiling
 * and the form of the dot products the other flags name: what gemv_forward_cuda_qk_group_hq returns
 * (quant/csrc/gemv_cuda.h:78-109), for callers and tests that want the scores of one particular tiling. */
#define HQEKV_ONLY_RAW_QK 0x2000
int64_t hqekv_decode_workspace_bytes(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                                     int64_t B, int64_t Hq, int64_t Hkv, int64_t D);
int hqekv_decode_attn(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                      const void *q, const void *mask, int64_t mask_row_stride,
                      void *attn_weights, void *attn_out, int64_t B, int64_t Hq, int64_t Hkv,
                      int64_t D, int64_t Tall, void *workspace, int64_t workspace_bytes, int flags,
                      void *stream);

/* The decode step of the reference's attention layer as ONE call: hqekv_decode_attn plus what the layer does around it
 * on every generated token (model/llama_hqe.py:131-136, 200) --
 *   new_K = cat(residual, k), new_V = cat(residual, v)     two rows copied behind the residual, which the caller keeps
 *                                                          in capacity-sized buffers (see hqekv_seg.slab_tokens)
 *   last_weights.update(attn_weights)                      one row of the importance ring:
 *                                                          attn_weights.sum(0).sum(0), model/public_func.py:243-257
 * -- folded into the call's last launch (extra workgroups of the split-K combine, or a launch of their own when the
 * combine runs inside p.V).  The ring row follows the order in which torch's GPU reduction adds the rows (fp32
 * accumulation, one rounding to fp16 per reduction): ring_order is the number of threads that reduction deals the
 * head rows to for the shape at hand -- 2 when Tall is a multiple of 4, at least 256, and attn_weights is 8-byte
 * aligned; else 1 -- pinned against torch.sum on the device for 32 heads and batch sizes 1..8.
 * The appended rows are not read by this call's attention: the caller names this step's key and value as segments of
 * their own.  `extra` may be NULL (then the call is hqekv_decode_attn); single-stage flags are refused.
 */
typedef struct hqekv_step_extra {
  void *ring_line;             /* (Tall) fp16, any 2-byte alignment; NULL = no ring row                    */
  int32_t ring_order;          /* 1 or 2, see above                                                        */
  int32_t append_rows;         /* token rows of new_k / new_v per (b, kv head); 0 = nothing to append      */
  const void *new_k, *new_v;   /* (B,Hkv,append_rows,D) fp16, dense, 16-byte aligned                       */
  void *k_dst, *v_dst;         /* where slab 0's first appended row goes (16-byte aligned)                 */
  int64_t k_dst_slab_tokens;   /* token rows between two (b, kv head) slabs of the destination buffers     */
  int64_t v_dst_slab_tokens;
} hqekv_step_extra;
int hqekv_decode_step(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                      const void *q, const void *mask, int64_t mask_row_stride,
                      void *attn_weights, void *attn_out, int64_t B, int64_t Hq, int64_t Hkv,
                      int64_t D, int64_t Tall, void *workspace, int64_t workspace_bytes, int flags,
                      void *stream, const hqekv_step_extra *extra);
/* The ring row alone: line[t] = rnd16(sum_h rnd16(sum_b attn_weights[b,h,t])) in torch's order (`order` as
 * ring_order above).  Replaces last_attn_weights.update for one decode row (model/public_func.py:250-254). */
int hqekv_ring_row(const void *attn_weights, int64_t B, int64_t Hq, int64_t Tall, void *line, int order,
                   void *stream);

/* What the cache policy ranks blocks by (model/public_func.py:217-221 calculate_token_importance, :85-106
 * get_block_importance / get_block_token_idx with its in-place divide, quant/hqe_2.py:510-518 the V ranking's
 * importance * range, model/public_func.py:58-73 calculate_token_range), one launch each instead of a chain of torch
 * reductions.  All tensors fp16; every rounding and every order of additions is the one torch's GPU kernels use for
 * these shapes (rows of a matrix: one walker per column, four interleaved fp32 accumulators; 32 contiguous values: a
 * balanced tree over adjacent pairs), pinned against torch on the device.
 *   hqekv_importance_scores   ring (rows x max_len, row stride max_len): importance_out[c] = (sum of column c /
 *                             min(rows, n - c)) / 32 for c < total -- the values the ranking helper leaves behind in
 *                             its argument -- and scores_out[b] = sum of block b's 32 values (total = 32 * blocks <= n)
 *   hqekv_weighted_block_scores  scores_out[b] = sum over block b of (x[c] * weights[c]) / 32; weights NULL: x[c] / 32
 *   hqekv_token_range         v (B, H, T, D) fp16 token-major, slabs slab_tokens * D elements apart:
 *                             out[t] = sum_h sum_b (max_d v - min_d v), each sum rounded to fp16
 */
int hqekv_importance_scores(const void *ring, int32_t rows, int64_t max_len, int64_t n, int64_t total,
                            void *importance_out, void *scores_out, void *stream);
int hqekv_weighted_block_scores(const void *x, const void *weights, int64_t total, void *scores_out, void *stream);
int hqekv_token_range(const void *v, int64_t B, int64_t H, int64_t T, int64_t D, int64_t slab_tokens, void *out,
                      void *stream);

/* ------------------------------------------------------------------ the prompt side of the attention layer
 * Replaces, for head_dim 128 in fp16, what model/llama_hqe.py:141-188 does over a prompt: flash_attention_forward
 * (:147-155) and, for the importance ring, the dense matmul + mask + softmax over the last 20 query rows with
 * repeat_kv copies of K (:157-168).  Tensors are (B, H, T, 128) fp16 given by their strides in ELEMENTS for the
 * batch, head and token axes (channel stride 1, rows 16-byte aligned), so slices of a fused QKV projection are read
 * where they lie; K and V have Hkv heads, query head h reads KV head h / (Hq / Hkv).
 *   hqekv_prompt_attn       out (B, Hq, T, 128, strides as given) = softmax(q k^T * scale [causal]) v, fp32
 *                           accumulation and running softmax, probabilities rounded to fp16 before the second product
 *                           (scale > 0; B * Hq <= 65535)
 *   hqekv_prompt_last_rows  probs (B, Hq, R, T) contiguous: the probabilities of the last R <= 32 query rows with the
 *                           reference's roundings -- product to fp16, times scale to fp16, plus mask to fp16, floored
 *                           at -65504, softmax in fp32, to fp16.  mask: additive fp16 (B, 1, R, T) given by its batch
 *                           and row strides (key stride 1), or NULL for the causal rule (row r sees keys <= T - R + r).
 *                           workspace (hqekv_prompt_last_rows_workspace_bytes, may be 0): room for per-slice statistics,
 *                           with which few heads are spread over the chip in two launches; NULL: one workgroup per head.
 */
int hqekv_prompt_attn(const void *q, const int64_t *q_strides, const void *k, const int64_t *k_strides, const void *v,
                      const int64_t *v_strides, void *out, const int64_t *out_strides, int64_t B, int64_t Hq, int64_t Hkv,
                      int64_t T, int64_t D, float scale, int causal, void *stream);
int64_t hqekv_prompt_last_rows_workspace_bytes(int64_t B, int64_t Hq, int64_t T);
int hqekv_prompt_last_rows(const void *q, const int64_t *q_strides, const void *k, const int64_t *k_strides,
                           const void *mask, const int64_t *mask_strides, void *probs, int64_t B, int64_t Hq, int64_t Hkv,
                           int64_t T, int64_t D, int64_t R, float scale, void *workspace, int64_t workspace_bytes,
                           void *stream);

/* ------------------------------------------------------------------ cache maintenance (one launch per side)
 * Replaces the per-(source, target) gathers, dequantise / re-quantise calls and torch.cat re-copies of one
 * compression -- V_high_2_eviction / K_high_2_eviction (quant/hqe_2.py:44-86), quant_new_K (:16-42), K_high_2_low
 * (:88-130), V_high_2_low (:132-170) and their call sequence in KV_cache_hqe_2 (:552-836; KV_cache_compress,
 * quant/hybrid_quant.py:318-612, is the same without eviction) -- by ONE gather over whole 32-token blocks.
 *
 * `src` lists the old classes of one side plus the new fp16 tokens, `dst` the classes after the compression (all
 * freshly allocated by the caller, exact size).  Layouts as listed at the top of this file; a K source with bits == 16
 * and layout HQEKV_LAYOUT_TOKEN_MAJOR is (B,H,T,D) (the new tokens), HQEKV_LAYOUT_NORMAL1 marks 1-bit classes in
 * normal-quantile coding.  `plan` (device, int32) holds, for every destination block in the order of `dst`,
 * first (source slot << 24) | source block, then -- after all of those -- the block's new first position / 32;
 * the kernel also writes the destination classes' idx arrays from it (idx may be NULL).  A block that is in no
 * destination is dropped (evicted).  Same width: the packed bytes are copied; fp16 -> b bits: quantised; a -> b < a
 * bits: dequantised with the two fp16 roundings, then quantised; never the other way round.
 * is_k != 0: classes are (B,H,D,*) with groups of 32 tokens per channel; else (B,H,T,*) with groups of 32 channels.
 * The plan is device memory the host never sees, so the kernel checks every entry it reads: a source slot that is
 * not populated, a source block past the end of its class or a position outside the new sequence makes the kernel
 * skip that destination block (nothing out of range is touched) and, when `status` (device, one int32 the caller has
 * zeroed; may be NULL) is given, set it to a non-zero value.
 */
typedef struct hqekv_cache_class {
  int32_t bits;      /* 16, 8, 4, 2 or 1                       */
  int32_t layout;    /* HQEKV_LAYOUT_*                         */
  int64_t n_tokens;  /* multiple of 32; 0 = empty slot         */
  int64_t slab_tokens; /* tokens between two (b, h) slabs in memory when the class is a window of a longer
                          token-major tensor (the new tokens without the residual behind them); 0 = n_tokens */
  void *data;
  void *scale;       /* NULL when bits == 16                   */
  void *zero;
  int64_t *idx;      /* destination only: (n_tokens) or NULL   */
} hqekv_cache_class;
int hqekv_cache_migrate(int is_k, const hqekv_cache_class *src, int n_src, const hqekv_cache_class *dst,
                        int n_dst, const int32_t *plan, int64_t BH, int64_t D, int32_t *status, void *stream);

/* The plan for hqekv_cache_migrate, worked out on the HOST (every pointer here is a host pointer; nothing is launched).
 * Replaces the class-by-class selection of one compression (quant/hqe_2.py:552-659 for K, :672-836 for V: torch.isin
 * masks per (source, target) pair) and the re-ranking of the positions after an eviction (:661-670) by their outcome.
 *   old_blocks[c], old_counts[c]  c = 0..4 (fp16, 8, 4, 2, 1 bit): block numbers (first position / 32) of class c's
 *                                 blocks in stored order; together they are 0 .. hist_blocks-1
 *   n_new_blocks                  blocks of new fp16 tokens; they are numbered hist_blocks ..
 *   order                         all hist_blocks + n_new_blocks block numbers, most important first
 *   target_tokens[n_targets]      tokens the ranking is cut into: fp16, 8, 4, 2, 1 bit [, evicted]; multiples of 32
 * A block moves only to a lower precision (ranked higher, it stays); inside a new class: the members that stay, the
 * new tokens, then what comes down from fp16, 8, 4, 2 bit, each in source order.
 *   counts_out[5]                 blocks of every new class
 *   plan_out[2 * total]           room for every block; filled: per new block (n_alive of them, classes back to
 *                                 back) (source slot << 24) | block inside the source (slot 5 = the new tokens), then
 *                                 -- from plan_out[n_alive] on -- its new block number (its rank among the survivors):
 *                                 the 2 * n_alive words hqekv_cache_migrate reads
 *   alive_out[total], n_alive_out the surviving blocks' old numbers, ascending
 */
int hqekv_plan_side(const int32_t *const *old_blocks, const int32_t *old_counts, int32_t hist_blocks,
                    int32_t n_new_blocks, const int64_t *order, const int64_t *target_tokens, int32_t n_targets,
                    int32_t *counts_out, int32_t *plan_out, int32_t *alive_out, int32_t *n_alive_out);

/* No counterpart in the reference: hqekv_decode_attn for callers that cannot allocate (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  Same arguments minus the workspace: the split-K
 * partials and softmax statistics go to a fixed buffer of HQEKV_STATIC_SCRATCH_BYTES inside the library's device
 * image, one copy per GPU, held until the process ends; its address is looked up on the first call on a device
 * (hipGetSymbolAddress, which may make the runtime load the library's device image): make that first call on every
 * device BEFORE a stream capture begins -- a call with the real shapes or any small one -- since a runtime that loads
 * code inside a capture may refuse the capture.  Later calls only launch kernels.
 * The call allocates and frees nothing.  A call whose hqekv_decode_workspace_bytes() exceeds the buffer returns
 * HQEKV_E_WORKSPACE (use hqekv_decode_attn then).  All calls on one GPU share the buffer: calls that overlap in
 * time on one GPU (two streams, two threads) race; calls ordered on one stream are fine.
 */
#define HQEKV_STATIC_SCRATCH_BYTES (8u << 20)
int hqekv_decode_attn_static(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                             const void *q, const void *mask, int64_t mask_row_stride,
                             void *attn_weights, void *attn_out, int64_t B, int64_t Hq, int64_t Hkv,
                             int64_t D, int64_t Tall, int flags, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HQEKV_H */
