"""The benchmark configurations at their stated sizes, and every q.K^T tiling forced per call.

Small and medium cases are compared with the CPU oracle on every batch row.  At the full sizes of configurations
4 and 5 (B=8 at 65536 tokens, B=4 at 131072) the oracle runs on the first and the last batch row, and all rows are
held to size-independent properties: the probabilities of a row sum to one, and with q = 0 the output is the mean
of the dequantised V rows.  Tolerance everywhere: 1e-3 relative + 2e-3 absolute, fp32 accumulation."""
import functools

import pytest
import torch

from hqekv_amd import synth
from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 2e-3
C4_MIX = (0.10, 0.0, 0.20, 0.50, 0.20)   # fp16 / 8 / 4 / 2 bit / evicted shares of configuration 4


def _close(a, b, what=""):
    torch.testing.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, msg=lambda m: f"{what}: {m}")


def _tilings():
    from hqekv_amd import _lib
    return sorted(_lib.QK_TILINGS.items(), key=lambda kv: kv[1])


def _flags(fused: bool, tiling: int) -> int:
    from hqekv_amd import _lib
    return (_lib.FUSE_SOFTMAX if fused else 0) | _lib.qk_tiling(tiling)


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


@functools.lru_cache(maxsize=2)
def _c4_mix_case(permute: bool):
    """The CPU side of the B=8 case (inputs, oracle cache, oracle result), shared by its parametrisations."""
    B, Hq, Hkv, T, D, residual = 8, 32, 8, 16384 + 19, 128, 19
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, 404)
    classes = synth.split_blocks(T - residual, C4_MIX, 404)
    override = _shuffled(classes, T - residual, 404) if permute else None
    cache = synth.build_cache(K, V, classes, residual, O.uniform_group_quantize_pack_last_dim, override)
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, use_mask=False, round_per_class=False)
    return q, cache, w_ref, o_ref


@pytest.mark.parametrize("permute", [False, True], ids=["blockidx", "randperm"])
@pytest.mark.parametrize("tiling", ["8waves", "4waves", "wave512", "wave256", "auto"])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "general"])
def test_config4_mix_batch8_every_row(dev, tiling, permute, fused):
    """Configuration 4's class mix at B=8, 32 query heads over 8 KV heads, 16384 tokens: a launch of more than
    1024 tiles (what selects the large-launch tiling by itself), with each tiling forced in turn."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    B, Hq = 8, 32
    q, cache, w_ref, o_ref = _c4_mix_case(permute)
    Tall = cache[41]
    n = dict(_tilings()).get(tiling, 0)
    w, o = decode_attention(q.to(dev), synth.cache_to(cache, dev), None, Tall, zero_init=True, flags=_flags(fused, n))
    assert w.shape == (B, Hq, 1, Tall)
    _close(w, w_ref, f"attn_weights ({tiling})")
    _close(o, o_ref, f"attn_output ({tiling})")
    torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(B, Hq, 1), rtol=0, atol=5e-3)


@pytest.mark.parametrize("tiling", ["8waves", "4waves", "wave512", "wave256"])
@pytest.mark.parametrize("n_rep", [1, 2, 4, 8])
@pytest.mark.parametrize("low_normal", [False, True], ids=["uniform1", "normal1"])
def test_every_tiling_every_gqa_ratio(dev, tiling, n_rep, low_normal):
    """Each tiling with 1, 2, 4 and 8 query heads per KV head, all six classes (either 1-bit coding), a last tile
    that is not full in every class, shuffled positions and a residual, on the fused and the general path."""
    from hqekv_amd.attention import decode_attention
    B, Hkv, D, residual = 2, 2, 128, 37
    T = 75 * 32 + residual
    Hq = Hkv * n_rep
    seed = 900 + n_rep
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, seed)
    classes = synth.split_blocks(T - residual, (0.08, 0.12, 0.2, 0.25, 0.25, 0.1), seed)
    cache = synth.build_cache(K, V, classes, residual, _quant(low_normal), _shuffled(classes, T - residual, seed))
    Tall = cache[41]
    strategy = "high_uniform_group_low_normal_group" if low_normal else "uniform_group"
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, strategy, use_mask=False, round_per_class=False)
    n = dict(_tilings())[tiling]
    for fused in (True, False):
        w, o = decode_attention(q.to(dev), synth.cache_to(cache, dev), None, Tall, zero_init=True,
                                flags=_flags(fused, n), low_uniform=not low_normal)
        _close(w, w_ref, f"attn_weights fused={fused}")
        _close(o, o_ref, f"attn_output fused={fused}")


@pytest.mark.parametrize("tiling", ["wave512", "wave256"])
@pytest.mark.parametrize("outliers", [False, True], ids=["small_scales", "large_scales"])
def test_fused_bias_removal_gives_the_same_bits(dev, tiling, outliers):
    """The one-wave tilings dequantise a tile whose scales are all below 32 with one fused multiply-add per pair of
    codes, and any other tile with the subtraction and the multiplication apart; the flag that forces the second
    route everywhere must not change a bit of the probabilities.  With outliers, some 32-token blocks of K are
    scaled up until their 2-, 4- and 8-bit scales pass 32 (both routes inside one launch), and the oracle still
    agrees; the query is zero in the outlier channels' share so that the logits stay in range."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    B, Hq, Hkv, D, residual = 2, 8, 2, 128, 11
    T = 96 * 32 + residual
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, 77)
    if outliers:
        g = torch.Generator().manual_seed(78)
        blocks = torch.randperm((T - residual) // 32, generator=g)[:24]
        for j in blocks.tolist():
            K[:, :, j * 32:(j + 1) * 32, 8:16] *= 3000.0   # 8-bit scale ~ 6 * 3000 / 255 = 70
        assert bool(torch.isfinite(K).all())
        q[..., 8:16] = 0
    classes = synth.split_blocks(T - residual, (0.1, 0.2, 0.3, 0.3, 0.1, 0.0), 77)
    cache = synth.build_cache(K, V, classes, residual, O.uniform_group_quantize_pack_last_dim)
    if outliers:
        assert max(float(cache[s].abs().max()) for s in (6, 14, 22) if cache[s] is not None) >= 32.0  # K scales
    Tall = cache[41]
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, use_mask=False, round_per_class=False)
    n = dict(_tilings())[tiling]
    dcache = synth.cache_to(cache, dev)
    for fused in (True, False):
        w1, o1 = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True, flags=_flags(fused, n))
        w2, o2 = decode_attention(q.to(dev), dcache, None, Tall, zero_init=True,
                                  flags=_flags(fused, n) | _lib.TWO_STEP_DEQUANT)
        assert torch.equal(w1, w2) and torch.equal(o1, o2)
        _close(w1, w_ref, "attn_weights")
        _close(o1, o_ref, "attn_output")


def test_unknown_tiling_is_an_error(dev):
    from hqekv_amd import _lib
    from hqekv_amd.attention import decode_attention
    q, K, V = synth.make_qkv(1, 4, 2, 64, 128, 3)
    cache = O.empty_cache(K, V, 64)
    with pytest.raises(ValueError, match="tiling"):
        decode_attention(q.to(dev), synth.cache_to(cache, dev), None, 64, zero_init=True, flags=_lib.qk_tiling(15))


def _device_layer(name, dev, layer=0):
    """One layer's cache of a named configuration, generated and quantised on the device."""
    from hqekv_amd.pack_unpack import uniform_group_quantize_pack_last_dim as hip_quant
    cfg = synth.CONFIGS[name]
    g = torch.Generator(device=dev).manual_seed(cfg["seed"] + 1000 * layer)
    K = torch.randn(cfg["B"], cfg["Hkv"], cfg["T"], cfg["D"], generator=g, device=dev, dtype=torch.float16)
    for c in synth.OUTLIER_CHANNELS:
        K[..., c] *= 10.0
    V = torch.randn(cfg["B"], cfg["Hkv"], cfg["T"], cfg["D"], generator=g, device=dev, dtype=torch.float16)
    q = torch.randn(cfg["B"], cfg["Hq"], 1, cfg["D"], generator=g, device=dev, dtype=torch.float16)
    classes = synth.split_blocks(cfg["T"] - cfg["residual"], cfg["fractions"], cfg["seed"])
    cache = synth.build_cache(K, V, classes, cfg["residual"], hip_quant)
    return cfg, q, cache


def _row(cache, b):
    """Batch row b of a cache tuple, on the CPU."""
    return tuple((x[b:b + 1].cpu() if x.dim() == 4 else x.cpu()) if torch.is_tensor(x) else x for x in cache)


@pytest.mark.parametrize("name,counts", [
    ("c4", {16: 6560, 4: 13120, 2: 32768, 0: 13088}),
    ("c5", None),
])
def test_config_full_size(dev, name, counts):
    """Configurations 4 (B=8, 65536 tokens) and 5's layer shape (B=4, 131072 tokens) at full size: the oracle on
    batch rows 0 and B-1, row sums on every row, each q.K^T tiling, and the q = 0 mean-of-V property on all rows."""
    from hqekv_amd import _lib
    from hqekv_amd import pack_unpack as P
    from hqekv_amd.attention import decode_attention
    cfg, q, cache = _device_layer(name, dev)
    B, Hq, Hkv, D = cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["D"]
    if counts is not None:
        classes = synth.split_blocks(cfg["T"], cfg["fractions"], cfg["seed"])
        assert {b: classes[b].numel() for b in counts} == counts
    Tall = cache[41]
    # The probabilities are held to the oracle's.  The output is held to the oracle's p.V of the SAME probabilities:
    # with 50 000+ tokens and K outliers a raw score now and then sits on an fp16 rounding boundary, another
    # summation order over head_dim rounds it the other way, and a peaked row moves by a fraction of a percent --
    # inside the tolerance for the probabilities, but the output would inherit it on top of its own rounding.
    refs = {}
    for b in (0, B - 1):
        row = _row(cache, b)
        w_ref, _ = O.qkv_matmul(q[b:b + 1].cpu(), row, None, D, use_mask=False, round_per_class=False)
        refs[b] = (w_ref, O.repeat_kv(O.reconstruct_cache(row, "uniform_group")[1], Hq // Hkv).float())
    first = None
    for tiling, n in [("auto", 0)] + _tilings():
        w, o = decode_attention(q, cache, None, Tall, zero_init=False, flags=_flags(True, n))
        for b, (w_ref, v_dense) in refs.items():
            _close(w[b:b + 1], w_ref, f"{name} attn_weights row {b} ({tiling})")
            _close(o[b:b + 1], torch.matmul(w[b:b + 1].float().cpu(), v_dense), f"{name} attn_output row {b} ({tiling})")
        torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(B, Hq, 1), rtol=0, atol=5e-3)
        if first is None:
            first = (w.clone(), o.clone())
        else:   # the tilings agree on every row, also where the oracle was not run
            torch.testing.assert_close(w.float(), first[0].float(), rtol=RTOL, atol=ATOL)
            torch.testing.assert_close(o.float(), first[1].float(), rtol=RTOL, atol=ATOL)
    # the general path (separate softmax launch) on the same cache
    w, o = decode_attention(q, cache, None, Tall, zero_init=True, flags=0)
    torch.testing.assert_close(w.float(), first[0].float(), rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(o.float(), first[1].float(), rtol=RTOL, atol=ATOL)
    # q = 0: every probability is 1/Tall, the output is the mean of the dequantised V rows -- every batch row
    w, o = decode_attention(torch.zeros_like(q), cache, None, Tall, zero_init=False, flags=_flags(True, 0))
    # (1 / Tall is an fp16 denormal at these lengths: half a denormal step of rounding)
    assert torch.allclose(w.float(), torch.full_like(w, 1.0 / Tall, dtype=torch.float32), rtol=1e-3, atol=3.1e-8)
    total = torch.zeros(B, Hkv, D, dtype=torch.float32, device=dev)
    if cache[2] is not None:
        total += cache[2].float().sum(2)
    for bits, base in ((8, 8), (4, 16), (2, 24)):
        if cache[base] is not None:
            total += P.uniform_group_dequantize_unpack_last_dim(cache[base], cache[base + 2], cache[base + 3], 32, bits).float().sum(2)
    expect = (total * w[0, 0, 0, 0].float())[:, :, None, None, :].expand(B, Hkv, Hq // Hkv, 1, D).reshape(B, Hq, 1, D)
    torch.testing.assert_close(o.float(), expect, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("bit", [2, 4, 8])
def test_config3_full_size_append(dev, bit):
    """Configuration 3 at its stated size: K (handed over as the transposed view of token-major memory) and V of
    8 heads x 8192 new tokens x 128 channels quantised into the window that starts at token 24576 of buffers with
    room for 32768 tokens.  Codes, scales and zeros are bit-identical to the oracle's, and nothing outside the
    window changes."""
    from hqekv_amd import pack_unpack as P
    B, H, D, new, old, cap = 1, 8, 128, 8192, 24576, 32768
    pf = 32 // bit
    _, K, V = synth.make_qkv(B, 32, H, new, D, 1237)
    sent_i, sent_h = -1234567, -3.0
    kc = torch.full((B, H, D, cap // pf), sent_i, dtype=torch.int32, device=dev)
    ks = torch.full((B, H, D, cap // 32), sent_h, dtype=torch.float16, device=dev)
    kz = torch.full_like(ks, sent_h)
    vc = torch.full((B, H, cap, D // pf), sent_i, dtype=torch.int32, device=dev)
    vs = torch.full((B, H, cap, D // 32), sent_h, dtype=torch.float16, device=dev)
    vz = torch.full_like(vs, sent_h)
    P.quantize_pack_into(K.to(dev).transpose(2, 3), bit, kc[..., old // pf:], ks[..., old // 32:], kz[..., old // 32:])
    P.quantize_pack_into(V.to(dev), bit, vc[:, :, old:], vs[:, :, old:], vz[:, :, old:])
    okc, oks, okz = O.uniform_group_quantize_pack_last_dim(K.transpose(2, 3).contiguous(), 32, bit)
    ovc, ovs, ovz = O.uniform_group_quantize_pack_last_dim(V, 32, bit)
    assert torch.equal(kc[..., old // pf:].cpu(), okc)
    assert torch.equal(ks[..., old // 32:].cpu(), oks) and torch.equal(kz[..., old // 32:].cpu(), okz)
    assert torch.equal(vc[:, :, old:].cpu(), ovc)
    assert torch.equal(vs[:, :, old:].cpu(), ovs) and torch.equal(vz[:, :, old:].cpu(), ovz)
    assert bool((kc[..., :old // pf] == sent_i).all()) and bool((vc[:, :, :old] == sent_i).all())
    for t in (ks[..., :old // 32], kz[..., :old // 32], vs[:, :, :old], vz[:, :, :old]):
        assert bool((t == sent_h).all())
