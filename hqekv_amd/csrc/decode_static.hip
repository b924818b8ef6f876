// hqekv_decode_attn without a caller workspace: the split-K partials and the per-tile softmax statistics live in
// a fixed array inside the library's device image (one copy per GPU, held until the process ends), so the call
// allocates nothing -- for callers under stream capture or in loops that must not touch the allocator.
//
// Host code never uses the array's name as an address (in host code the name is a stand-in, not a device
// pointer): the device address is looked up once per device, with that device current, and kept.
#include <mutex>

#include "common.h"

// The kernels receive the array through the same workspace argument the caller-workspace entry point passes.
static __device__ __align__(256) unsigned char scratch[HQEKV_STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
void *g_scratch_of[MAX_DEVICES];  // device address of `scratch` on each GPU, nullptr until looked up
std::mutex g_scratch_mu;

int scratch_address(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hq::fail((int)e, "decode_attn_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= MAX_DEVICES) return hq::fail(HQEKV_E_UNSUPPORTED, "decode_attn_static: device ordinal %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_of[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hq::fail((int)e, "decode_attn_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    if (!p) return hq::fail(HQEKV_E_UNSUPPORTED, "decode_attn_static: the scratch array has no address on device %d", dev);
    g_scratch_of[dev] = p;
  }
  *out = g_scratch_of[dev];
  return HQEKV_OK;
}

}  // namespace

extern "C" int hqekv_decode_attn_static(const hqekv_seg *k_segs, int n_k, const hqekv_seg *v_segs, int n_v,
                                        const void *q, const void *mask, int64_t mask_row_stride,
                                        void *attn_weights, void *attn_out, int64_t B, int64_t Hq, int64_t Hkv,
                                        int64_t D, int64_t Tall, int flags, void *stream) {
  const int64_t need = hqekv_decode_workspace_bytes(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D);
  if (need < 0) return hq::fail(HQEKV_E_ARG, "decode_attn_static: bad segment tables");
  if (need > (int64_t)HQEKV_STATIC_SCRATCH_BYTES)
    return hq::fail(HQEKV_E_WORKSPACE,
                    "decode_attn_static: this call needs %lld bytes of scratch, the built-in buffer holds %lld; "
                    "use hqekv_decode_attn with a caller workspace",
                    (long long)need, (long long)HQEKV_STATIC_SCRATCH_BYTES);
  void *ws = nullptr;
  const int rc = scratch_address(&ws);
  if (rc) return rc;
  // every part of the workspace is written before it is read within one call, so nothing has to be cleared
  return hqekv_decode_attn(k_segs, n_k, v_segs, n_v, q, mask, mask_row_stride, attn_weights, attn_out, B, Hq, Hkv, D,
                           Tall, ws, (int64_t)HQEKV_STATIC_SCRATCH_BYTES, flags, stream);
}
