"""The matrix-core form of the inner products (HQEKV_DOT_MFMA, four query heads per KV head) against the CPU oracle
and against the vector-ALU form (HQEKV_DOT_VALU) of the same call.  Both forms feed the same dequantised values into
exact products with fp32 accumulation; only the order of the additions differs, so both are held to the oracle with
the tolerance of the path: 1e-3 relative + 2e-3 absolute."""
import pytest
import torch

from hqekv_amd import synth
from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 2e-3


def _close(a, b, what=""):
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=RTOL, atol=ATOL, msg=lambda m: f"{what}: {m}")


def _shuffled(classes, n_tokens, seed):
    pos, kept = synth.survivor_positions(classes, n_tokens)
    perm = torch.randperm(kept, generator=torch.Generator().manual_seed(seed))
    out, start = {}, 0
    for b, p in pos.items():
        out[b] = perm[start:start + p.numel()]
        start += p.numel()
    return out


def _quant(low_normal):
    def f(x, g, bits):
        if bits == 1 and low_normal:
            return O.normal_group_quantize_pack_last_dim(x, 32, 1)
        return O.uniform_group_quantize_pack_last_dim(x, 32, bits)
    return f


def _flags(fused, tiling, extra=0):
    from hqekv_amd import _lib
    return (_lib.FUSE_SOFTMAX if fused else 0) | _lib.qk_tiling(tiling) | extra


@pytest.mark.parametrize("tiling", ["auto", "8waves", "4waves", "wave512", "wave256"])
@pytest.mark.parametrize("low_normal", [False, True], ids=["uniform1", "normal1"])
@pytest.mark.parametrize("residual", [0, 1, 37, 130])
def test_matrix_core_form_all_classes(dev, tiling, low_normal, residual):
    """All six classes (either 1-bit coding), a last tile / chunk that is not full in every class, shuffled
    positions, residuals of even and odd length, every q.K^T tiling, the fused and the general path."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    B, Hkv, Hq, D = 2, 2, 8, 128
    T = 75 * 32 + residual
    seed = 1300 + residual
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, seed)
    classes = synth.split_blocks(T - residual, (0.08, 0.12, 0.2, 0.25, 0.25, 0.1), seed)
    cache = synth.build_cache(K, V, classes, residual, _quant(low_normal), _shuffled(classes, T - residual, seed))
    Tall = cache[41]
    strategy = "high_uniform_group_low_normal_group" if low_normal else "uniform_group"
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, strategy, use_mask=False, round_per_class=False)
    n = _lib.QK_TILINGS.get(tiling, 0)
    dcache = synth.cache_to(cache, dev)
    for fused in (True, False):
        w, o = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True, flags=_flags(fused, n, _lib.DOT_MFMA),
                                low_uniform=not low_normal)
        wv, ov = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True, flags=_flags(fused, n, _lib.DOT_VALU),
                                  low_uniform=not low_normal)
        _close(w, w_ref, f"attn_weights fused={fused}")
        _close(o, o_ref, f"attn_output fused={fused}")
        _close(w, wv, f"matrix cores vs vector ALU, attn_weights fused={fused}")
        _close(o, ov, f"matrix cores vs vector ALU, attn_output fused={fused}")
        torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(B, Hq, 1), rtol=0, atol=5e-3)


def test_matrix_core_form_exact_integer_case(dev):
    """Known answer that needs no oracle: 8-bit codes with scale 1 and zero 0 hold small integers, the query holds
    small integers, so every raw score is an integer below 2048 and exact in fp16 whatever the order of the
    additions; V likewise with one-hot probabilities (a huge logit on one token).  Any wrong operand placement in
    the matrix instruction (head <-> lane, element order inside the 4-element step) shows up as a wrong integer."""
    from hqekv_amd import _lib
    B, Hq, Hkv, D, T = 1, 8, 2, 128, 512
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, 4, (B, Hkv, D, T), generator=g, dtype=torch.int32)
    kc = O.pack_along_last_dim(codes, 8)
    ks = torch.ones(B, Hkv, D, T // 32, dtype=torch.float16)
    kz = torch.zeros_like(ks)
    q = torch.randint(-2, 3, (B, Hq, 1, D), generator=g).half()
    ref = torch.matmul(q.float(), O.repeat_kv(codes.float().transpose(2, 3), 4).transpose(2, 3))   # (B,Hq,1,T)
    assert float(ref.abs().max()) < 2048
    lib = _lib.load()
    keep = [kc.to(dev), ks.to(dev), kz.to(dev)]
    segs = _lib.make_segs([dict(bits=8, n_tokens=T, data=keep[0], scale=keep[1], zero=keep[2], idx=None, pos_base=0)])
    vcodes = torch.randint(0, 200, (B, Hkv, T, D), generator=g, dtype=torch.int32)
    vc = O.pack_along_last_dim(vcodes, 8).to(dev)
    vs = torch.ones(B, Hkv, T, D // 32, dtype=torch.float16, device=dev)
    vz = torch.zeros_like(vs)
    vsegs = _lib.make_segs([dict(bits=8, n_tokens=T, data=vc, scale=vs, zero=vz, idx=None, pos_base=0)])
    need = lib.hqekv_decode_workspace_bytes(segs, 1, vsegs, 1, B, Hq, Hkv, D)
    ws = torch.empty(need // 4 + 64, dtype=torch.float32, device=dev)
    qd = q.to(dev).contiguous()
    # the fused q.K^T stage alone leaves the scaled logits: rnd16(rnd16(score) * (1 / sqrt(128))) with the fp32 reciprocal
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(128.0, dtype=torch.float32).sqrt()
    expect = (ref.half().float() * inv).half()
    for tiling in (1, 2, 3, 4):
        for dot in (_lib.DOT_MFMA, _lib.DOT_VALU):
            w = torch.zeros(B, Hq, 1, T, dtype=torch.float16, device=dev)
            out = torch.zeros(B, Hq, 1, D, dtype=torch.float16, device=dev)
            rc = lib.hqekv_decode_attn(segs, 1, vsegs, 1, qd.data_ptr(), None, 0, w.data_ptr(), out.data_ptr(), B, Hq, Hkv,
                                       D, T, ws.data_ptr(), ws.numel() * 4,
                                       _lib.FUSE_SOFTMAX | _lib.ONLY_QK | _lib.qk_tiling(tiling) | dot, _lib.stream_ptr(dev))
            _lib.check(rc, "decode_attn")
            torch.cuda.synchronize()
            assert torch.equal(w.cpu(), expect), (tiling, dot)
    # p.V: probabilities that are exactly one-hot per head after the softmax -> the output is one V row per head
    hot = torch.randint(0, T, (Hq,), generator=g)
    big = torch.zeros(B, Hq, 1, T, dtype=torch.float16)
    for h in range(Hq):
        big[0, h, 0, hot[h]] = 1.0
    for dot in (_lib.DOT_MFMA, _lib.DOT_VALU):
        p = big.to(dev).clone()
        out = torch.zeros(B, Hq, 1, D, dtype=torch.float16, device=dev)
        rc = lib.hqekv_decode_attn(segs, 1, vsegs, 1, qd.data_ptr(), None, 0, p.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, T,
                                   ws.data_ptr(), ws.numel() * 4, _lib.ONLY_PV | dot, _lib.stream_ptr(dev))
        _lib.check(rc, "decode_attn p.V")
        rc = lib.hqekv_decode_attn(segs, 1, vsegs, 1, qd.data_ptr(), None, 0, p.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, T,
                                   ws.data_ptr(), ws.numel() * 4, _lib.ONLY_COMBINE | dot, _lib.stream_ptr(dev))
        _lib.check(rc, "decode_attn combine")
        torch.cuda.synchronize()
        for h in range(Hq):
            assert torch.equal(out[0, h, 0].cpu().float(), vcodes[0, h // 4, hot[h]].float()), (h, dot)


def test_matrix_core_form_needs_four_heads_per_kv_head(dev):
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    q, K, V = synth.make_qkv(1, 4, 2, 64, 128, 3)
    cache = O.empty_cache(K, V, 64)
    with pytest.raises(ValueError, match="Hq/Hkv == 4"):
        decode_attention(q.to(dev), synth.cache_to(cache, dev), None, 64, zero_init=True, flags=_lib.DOT_MFMA)
    with pytest.raises(ValueError, match="exclude"):
        decode_attention(q.to(dev), synth.cache_to(cache, dev), None, 64, zero_init=True,
                         flags=_lib.DOT_MFMA | _lib.DOT_VALU)


@pytest.mark.parametrize("tiling", ["wave512", "wave256"])
def test_matrix_core_form_fused_bias_removal_gives_the_same_bits(dev, tiling):
    """Large K scales force the two-step dequantisation for some tiles of a launch; the flag that forces it
    everywhere must not change a bit on the matrix-core form either."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    B, Hq, Hkv, D, residual = 2, 8, 2, 128, 11
    T = 96 * 32 + residual
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, 77)
    g = torch.Generator().manual_seed(78)
    for j in torch.randperm((T - residual) // 32, generator=g)[:24].tolist():
        K[:, :, j * 32:(j + 1) * 32, 8:16] *= 3000.0
    q[..., 8:16] = 0
    classes = synth.split_blocks(T - residual, (0.1, 0.2, 0.3, 0.3, 0.1, 0.0), 77)
    cache = synth.build_cache(K, V, classes, residual, O.uniform_group_quantize_pack_last_dim)
    Tall = cache[41]
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, use_mask=False, round_per_class=False)
    n = _lib.QK_TILINGS[tiling]
    dcache = synth.cache_to(cache, dev)
    for fused in (True, False):
        w1, o1 = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True, flags=_flags(fused, n, _lib.DOT_MFMA))
        w2, o2 = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True,
                                  flags=_flags(fused, n, _lib.DOT_MFMA | _lib.TWO_STEP_DEQUANT))
        assert torch.equal(w1, w2) and torch.equal(o1, o2)
        _close(w1, w_ref, "attn_weights")
        _close(o1, o_ref, "attn_output")


@pytest.mark.parametrize("permute", [False, True], ids=["blockidx", "randperm"])
def test_matrix_core_form_config4_mix_batch8(dev, permute):
    """Configuration 4's class mix at B=8, 32 query heads over 8 KV heads, 16384 tokens (a launch of more than 1024
    tiles), every batch row against the oracle; fold and separate combine give the same bits."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    from tests.test_scale_gpu import _c4_mix_case
    q, cache, w_ref, o_ref = _c4_mix_case(permute)
    Tall = cache[41]
    dcache = synth.cache_to(cache, dev)
    outs = []
    for extra in (_lib.SEPARATE_COMBINE, _lib.FOLD_COMBINE):
        w, o = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True,
                                flags=_lib.FUSE_SOFTMAX | _lib.DOT_MFMA | extra)
        _close(w, w_ref, "attn_weights")
        _close(o, o_ref, "attn_output")
        outs.append((w.clone(), o.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
