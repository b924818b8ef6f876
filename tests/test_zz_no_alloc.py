"""hqekv_decode_attn_static -- the decode-attention call that allocates nothing (its scratch is a fixed array in
the library's device image) -- against hqekv_decode_attn with a caller workspace: same kernels, same order of
summation, so probabilities and outputs must be bit-identical.  Two calls in a row on the shared buffer, the
second on a smaller cache (what the first call left behind must not leak into it), then a call that does not fit."""
import ctypes as C

import pytest
import torch

from hqekv_amd import synth
from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu


def _tables(q, pkv, dev):
    from hqekv_amd import _lib
    from hqekv_amd import attention as A
    keep = []
    Tall = A.value_length(pkv)
    k_items, hk, _ = A.key_segments(pkv, dev, Tall, keep)
    v_items, hv, _ = A.value_segments(pkv, dev, Tall, keep)
    return _lib.make_segs(k_items), len(k_items), _lib.make_segs(v_items), len(v_items), hk, Tall, keep


def _both(q, pkv, dev, flags):
    """-> ((weights, out) through the caller-workspace entry, (weights, out) through the static one)"""
    from hqekv_amd import _lib
    from hqekv_amd import attention as A
    lib = _lib.load()
    B, Hq, _, D = q.shape
    k_segs, n_k, v_segs, n_v, Hkv, Tall, keep = _tables(q, pkv, dev)
    res = []
    for static in (False, True):
        w = torch.zeros(B, Hq, 1, Tall, dtype=torch.float16, device=dev)
        o = torch.zeros(B, Hq, 1, D, dtype=torch.float16, device=dev)
        st = _lib.stream_ptr(dev)
        if static:
            rc = lib.hqekv_decode_attn_static(k_segs, n_k, v_segs, n_v, q.data_ptr(), None, 0, w.data_ptr(),
                                              o.data_ptr(), B, Hq, Hkv, D, Tall, flags, st)
        else:
            ws = A.decode_workspace(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D, dev)
            rc = lib.hqekv_decode_attn(k_segs, n_k, v_segs, n_v, q.data_ptr(), None, 0, w.data_ptr(), o.data_ptr(),
                                       B, Hq, Hkv, D, Tall, ws.data_ptr(), ws.numel() * 4, flags, st)
        _lib.check(rc, "decode_attn_static" if static else "decode_attn")
        torch.cuda.synchronize()
        res.append((w, o))
    return res


def _cache(B, Hq, Hkv, T, residual, seed, dev):
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, 128, seed)
    classes = synth.split_blocks(T - residual, (0.05, 0.15, 0.30, 0.30, 0.20), seed)
    cache = synth.build_cache(K, V, classes, residual, O.uniform_group_quantize_pack_last_dim)
    return q, cache, q.to(dev), synth.cache_to(cache, dev)


@pytest.mark.parametrize("flags", [1, 0, 1 | 4], ids=["fused", "general", "fused_folded_combine"])
def test_static_scratch_entry_matches_workspace_entry(dev, flags):
    """The third case forces the folded combine (HQEKV_FOLD_COMBINE), whose arrival counters live in the shared
    buffer too: they must be back at zero for the second call."""
    big = _cache(2, 8, 2, 4096 + 21, 21, 31, dev)
    small = _cache(1, 8, 2, 640 + 3, 3, 32, dev)
    for q, cache, qd, cd in (big, small):   # the second call is the smaller one, on the buffer the first one used
        (w0, o0), (w1, o1) = _both(qd, cd, dev, flags)
        assert torch.equal(w0, w1) and torch.equal(o0, o1)
        w_ref, o_ref = O.qkv_matmul(q, cache, None, 128, use_mask=False, round_per_class=False)
        torch.testing.assert_close(w1.float().cpu(), w_ref.float(), rtol=1e-3, atol=2e-3)
        torch.testing.assert_close(o1.float().cpu(), o_ref.float(), rtol=1e-3, atol=2e-3)


def test_static_scratch_entry_leaves_device_memory_alone(dev):
    """Free device memory, as the driver reports it, is the same before and after calls of the static entry (the first
    call on the device, which looks up the buffer's address, has been made before the measurement starts)."""
    from hqekv_amd import _lib
    lib = _lib.load()
    q, cache, qd, cd = _cache(2, 8, 2, 2048 + 5, 5, 33, dev)
    B, Hq, _, D = qd.shape
    k_segs, n_k, v_segs, n_v, Hkv, Tall, keep = _tables(qd, cd, dev)
    w = torch.zeros(B, Hq, 1, Tall, dtype=torch.float16, device=dev)
    o = torch.zeros(B, Hq, 1, D, dtype=torch.float16, device=dev)
    st = _lib.stream_ptr(dev)

    def call(flags):
        _lib.check(lib.hqekv_decode_attn_static(k_segs, n_k, v_segs, n_v, qd.data_ptr(), None, 0, w.data_ptr(),
                                                o.data_ptr(), B, Hq, Hkv, D, Tall, flags, st), "decode_attn_static")
    call(1)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    reserved_before = torch.cuda.memory_reserved(dev)
    for flags in (1, 0, 1 | 4, 1):
        call(flags)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before and torch.cuda.memory_reserved(dev) == reserved_before


def test_static_scratch_entry_rejects_what_does_not_fit(dev):
    """A batch whose split-K partials exceed the built-in buffer is refused with a clear error and nothing runs."""
    from hqekv_amd import _lib
    lib = _lib.load()
    B, Hq, Hkv, D, T = 640, 32, 8, 128, 64
    segs = _lib.make_segs([dict(bits=16, n_tokens=T, data=None, idx=None, pos_base=0)])
    segs[0].data = 256   # never dereferenced: the size check comes first
    need = lib.hqekv_decode_workspace_bytes(segs, 1, segs, 1, B, Hq, Hkv, D)
    assert need > _lib.STATIC_SCRATCH_BYTES
    rc = lib.hqekv_decode_attn_static(segs, 1, segs, 1, 256, None, 0, 256, 256, B, Hq, Hkv, D, T, 1, None)
    assert rc == -3 and b"built-in buffer" in lib.hqekv_last_error()
