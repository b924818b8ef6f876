"""Pins for the CPU oracle: known answers, closed forms, invariants and brute force chosen so that a
dropped term, a wrong shift or a transposed operand fails at least one of them.  No GPU needed."""
import json
from pathlib import Path

import pytest
import torch

from oracle import hqe_oracle as O

GOLDEN = Path(__file__).parent / "golden"


# ------------------------------------------------------------------ pack / unpack
def test_pack_known_answer_lsb_first():
    q = torch.tensor([0, 1, 2, 3] * 4, dtype=torch.int32).reshape(1, 1, 1, 16)
    w = O.pack_along_last_dim(q, 2)
    assert w.item() == -454761244 and (w.item() & 0xFFFFFFFF) == 0xE4E4E4E4
    # one code in slot i sets exactly bits [i*b, i*b+b)
    for bit in (1, 2, 4, 8):
        pf = 32 // bit
        for i in range(pf):
            q = torch.zeros(1, 1, 1, pf, dtype=torch.int32)
            q[..., i] = 2 ** bit - 1
            assert (O.pack_along_last_dim(q, bit).item() & 0xFFFFFFFF) == ((2 ** bit - 1) << (i * bit))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_pack_unpack_round_trip_every_value_in_every_slot(bit):
    pf = 32 // bit
    vals = torch.arange(2 ** bit, dtype=torch.int32)
    q = torch.stack([vals.roll(s) for s in range(pf)], dim=-1).reshape(1, 1, -1, pf)  # every value in every slot
    code = O.pack_along_last_dim(q, bit)
    assert code.shape == (1, 1, 2 ** bit, 1) and code.dtype == torch.int32
    assert torch.equal(O.unpack_codes(code, bit), q)
    assert torch.equal(O.unpack_along_last_dim(code, bit), q.to(torch.float16))


def test_golden_pack_vectors():
    g = json.loads((GOLDEN / "pack_vectors.json").read_text())
    for case in g["cases"]:
        q = torch.tensor(case["codes"], dtype=torch.int32).reshape(1, 1, 1, -1)
        w = O.pack_along_last_dim(q, case["bit"]).flatten().tolist()
        assert [x & 0xFFFFFFFF for x in w] == case["words_u32"], case["name"]


# ------------------------------------------------------------------ quantise
def test_quantise_known_answer_arange():
    """The reference's own smoke input (quant/pack_unpack.py:382): arange(128), groups of 32, 2 bit.
    mn = 32g, mx - mn = 31, scale = fp16(31/3) = 10.3359375; codes by hand: k/10.3359375 rounded half-even."""
    x = torch.arange(0, 128, dtype=torch.float16).reshape(1, 1, 1, -1)
    for mode in ("recip", "true"):
        code, scale, mn = O.uniform_group_quantize_pack_last_dim(x, 32, 2, mode)
        assert scale.flatten().tolist() == [10.3359375] * 4
        assert mn.flatten().tolist() == [0.0, 32.0, 64.0, 96.0]
        expect = [0] * 6 + [1] * 10 + [2] * 10 + [3] * 6
        assert O.unpack_codes(code, 2).flatten().tolist() == expect * 4
    g = json.loads((GOLDEN / "quant_arange128.json").read_text())
    assert [w & 0xFFFFFFFF for w in code.flatten().tolist()] == g["words_u32_2bit"]
    # 1 bit (the uniform 1-bit class): scale = mx - mn = 31, code = [k >= 16]
    code1, scale1, mn1 = O.uniform_group_quantize_pack_last_dim(x, 32, 1)
    assert scale1.flatten().tolist() == [g["scale_1bit"]] * 4 and mn1.flatten().tolist() == [0.0, 32.0, 64.0, 96.0]
    assert [w & 0xFFFFFFFF for w in code1.flatten().tolist()] == g["words_u32_1bit"] == [0xFFFF0000] * 4
    # half of the range is a tie and goes to the even code 0
    tie = torch.tensor([0.0, 1.0, 2.0] + [0.0] * 29, dtype=torch.float16).reshape(1, 1, 1, 32)
    assert O.unpack_codes(O.uniform_group_quantize_pack_last_dim(tie, 32, 1)[0], 1).flatten().tolist()[:3] == [0, 0, 1]


def test_quantise_8bit_identity_on_integers():
    g = torch.Generator().manual_seed(0)
    x = torch.randint(0, 256, (1, 2, 3, 64), generator=g).to(torch.float16)
    x[..., 0], x[..., 31], x[..., 32], x[..., 63] = 0, 255, 0, 255  # every group spans exactly 0..255
    code, scale, mn = O.uniform_group_quantize_pack_last_dim(x, 32, 8)
    assert (scale == 1).all() and (mn == 0).all()
    assert torch.equal(O.unpack_codes(code, 8), x.to(torch.int32))
    assert torch.equal(O.uniform_group_dequantize_unpack_last_dim(code, scale, mn, 32, 8), x)


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_quantise_invariants(bit):
    g = torch.Generator().manual_seed(bit)
    x = (torch.randn(2, 2, 16, 128, generator=g) * 3).half()
    before = x.clone()
    code, scale, mn = O.uniform_group_quantize_pack_last_dim(x, 32, bit)
    assert torch.equal(x, before), "the oracle must not mutate its input"
    c = O.unpack_codes(code, bit).reshape(2, 2, 16, 4, 32)
    xg = x.reshape(2, 2, 16, 4, 32)
    qmax = 2 ** bit - 1
    assert c.min() >= 0 and c.max() <= qmax
    assert torch.equal(mn, xg.min(-1)[0])                       # zero point is the group minimum
    assert (c.gather(-1, xg.argmin(-1, keepdim=True)) == 0).all()   # the minimum maps to code 0
    assert (c.gather(-1, xg.argmax(-1, keepdim=True)) == qmax).all()  # the maximum maps to the top code
    dq = O.uniform_group_dequantize_unpack_last_dim(code, scale, mn, 32, bit).reshape(2, 2, 16, 4, 32)
    err = (dq.float() - xg.float()).abs()
    bound = scale.float().unsqueeze(-1) / 2 + 3 * 2.0 ** -11 * xg.float().abs().amax(-1, keepdim=True) + 1e-3
    assert (err <= bound).all()
    # monotone: a larger input never gets a smaller code within a group
    order = xg.argsort(-1)
    assert (c.gather(-1, order).diff(dim=-1) >= 0).all()


def test_quantise_constant_group_and_scalar_division_modes():
    x = torch.full((1, 1, 1, 32), 1.5, dtype=torch.float16)
    code, scale, mn = O.uniform_group_quantize_pack_last_dim(x, 32, 4)
    assert code.abs().sum() == 0 and scale.item() == 0 and mn.item() == 1.5
    assert torch.equal(O.uniform_group_dequantize_unpack_last_dim(code, scale, mn, 32, 4), x)
    # the two scalar-division rules differ by at most one fp16 ulp of the scale
    g = torch.Generator().manual_seed(5)
    y = torch.randn(1, 4, 64, 256, generator=g).half()
    for bit in (1, 2, 4, 8):
        a = O.uniform_group_quantize_pack_last_dim(y, 32, bit, "recip")[1].float()
        b = O.uniform_group_quantize_pack_last_dim(y, 32, bit, "true")[1].float()
        assert ((a - b).abs() <= b.abs() * 2.0 ** -10).all()


def test_dequantise_two_roundings_by_hand():
    # code 3, scale 0.3333 (fp16 0.33325195), zero 100: fp16(3*0.33325195)=0.99951172, fp16(100.99951172)=101.0
    code = O.pack_along_last_dim(torch.tensor([3] + [0] * 31, dtype=torch.int32).reshape(1, 1, 1, 32), 2)
    s = torch.tensor(0.3333, dtype=torch.float16).reshape(1, 1, 1, 1)
    z = torch.tensor(100.0, dtype=torch.float16).reshape(1, 1, 1, 1)
    dq = O.uniform_group_dequantize_unpack_last_dim(code, s, z, 32, 2)
    assert dq[0, 0, 0, 0].item() == 101.0 and dq[0, 0, 0, 1].item() == 100.0
    # a case a single fused rounding gets wrong: 10 * fp16(0.1) = 0.999755859375 is a tie that rounds to
    # 1.0; 2050 + 1.0 = 2051 is a tie (ulp 2) that rounds to the even 2052.  One rounding of the exact
    # 2050.99976 would give 2050.
    s2 = torch.tensor(0.0999755859375, dtype=torch.float16).reshape(1, 1, 1, 1)
    z2 = torch.tensor(2050.0, dtype=torch.float16).reshape(1, 1, 1, 1)
    code2 = O.pack_along_last_dim(torch.tensor([10] + [0] * 31, dtype=torch.int32).reshape(1, 1, 1, 32), 4)
    dq2 = O.uniform_group_dequantize_unpack_last_dim(code2, s2, z2, 32, 4)
    assert dq2[0, 0, 0, 0].item() == 2052.0


# ------------------------------------------------------------------ GEMV
def test_gemv_collapses_to_integer_matvec():
    g = torch.Generator().manual_seed(1)
    c = torch.randint(0, 8, (1, 2, 16, 64), generator=g, dtype=torch.int32)
    q = torch.randint(-2, 3, (1, 4, 1, 16), generator=g).half()
    code = O.pack_along_last_dim(c, 4)
    s = torch.ones(1, 2, 16, 2, dtype=torch.float16)
    z = torch.zeros_like(s)
    out = O.gemv_uniform_group(32, q, code, s, z, 4)
    exact = torch.matmul(q.long(), O.repeat_kv(c.long(), 2))
    assert torch.equal(out.long(), exact)
    # all codes zero: out = sum_k q_k * zero_k for every column of the group
    z2 = torch.randn(1, 2, 16, 2, generator=g).half()
    out0 = O.gemv_uniform_group(32, q, torch.zeros_like(code), s, z2, 4)
    ref0 = torch.matmul(q.float(), O.repeat_kv(z2, 2).float()).half()
    assert torch.equal(out0[..., 0:1], ref0[..., 0:1]) and torch.equal(out0[..., 63:64], ref0[..., 1:2])


def test_repeat_kv_maps_query_head_to_kv_head():
    x = torch.arange(3).reshape(1, 3, 1, 1).float()
    assert O.repeat_kv(x, 2).flatten().tolist() == [0, 0, 1, 1, 2, 2]  # hq // n_rep


# ------------------------------------------------------------------ hybrid attention
def test_hybrid_all_fp16_equals_dense_attention_under_permutation():
    g = torch.Generator().manual_seed(3)
    B, Hq, Hkv, T, D = 1, 4, 2, 96, 32
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    K = torch.randn(B, Hkv, T, D, generator=g).half()
    V = torch.randn(B, Hkv, T, D, generator=g).half()
    perm = torch.randperm(64, generator=g)
    t = [None] * 42
    t[0], t[1] = K[:, :, :64].transpose(2, 3).contiguous(), perm
    t[2], t[3] = V[:, :, :64].contiguous(), perm.clone()
    t[39], t[40], t[41] = K[:, :, 64:], V[:, :, 64:], T
    w, o = O.qkv_matmul(q, tuple(t), None, D, use_mask=False, round_per_class=False)
    Kp, Vp = K.clone(), V.clone()
    Kp[:, :, perm], Vp[:, :, perm] = K[:, :, :64], V[:, :, :64]
    s = torch.matmul(q.float(), O.repeat_kv(Kp, 2).transpose(2, 3).float()).half()
    s = (s.float() * (torch.tensor(1.0) / torch.tensor(D ** 0.5))).half()
    p = torch.softmax(s.float(), -1).half()
    assert torch.equal(w, p)
    torch.testing.assert_close(o.float(), torch.matmul(p.float(), O.repeat_kv(Vp, 2).float()), rtol=1e-3, atol=1e-3)
    assert abs(float(w.float().sum(-1).mean()) - 1.0) < 2e-3


def test_hybrid_single_class_equals_per_class_gemv():
    g = torch.Generator().manual_seed(4)
    B, Hq, Hkv, T, D = 1, 4, 1, 64, 32
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    K = torch.randn(B, Hkv, T, D, generator=g).half()
    V = torch.randn(B, Hkv, T, D, generator=g).half()
    kc, ks, kz = O.uniform_group_quantize_pack_last_dim(K.transpose(2, 3).contiguous(), 32, 4)
    vc, vs, vz = O.uniform_group_quantize_pack_last_dim(V, 32, 4)
    idx = torch.arange(T)
    t = [None] * 42
    t[12], t[13], t[14], t[15] = kc, idx, ks, kz
    t[16], t[17], t[18], t[19] = vc, idx.clone(), vs, vz
    t[41] = T
    w, o = O.qkv_matmul(q, tuple(t), None, D, use_mask=False)
    s = O.gemv_uniform_group(32, q, kc, ks, kz, 4)
    p = O._scale_clamp_softmax(s, D, None, "recip")
    assert torch.equal(w, p)
    assert torch.equal(o, O.gemv_uniform_group(32, p, vc, vs, vz, 4))


def test_mask_and_errors():
    q = torch.zeros(1, 2, 1, 32, dtype=torch.float16)
    with pytest.raises(ValueError, match="invalid past_key_value"):
        O.qkv_matmul(q, O.empty_cache(), None, 32)
    with pytest.raises(ValueError, match="invalid quant_strategy"):
        O.qkv_matmul(q, O.empty_cache(), None, 32, "bogus")
    K = torch.randn(1, 1, 8, 32).half()
    mask = torch.zeros(1, 1, 1, 8, dtype=torch.float16)
    mask[..., :4] = torch.finfo(torch.float16).min
    w, _ = O.qkv_matmul(q, O.empty_cache(K, K, 8), mask, 32)
    assert (w[..., :4] == 0).all() and torch.allclose(w[..., 4:].float(), torch.full((1, 2, 1, 4), 0.25))


# ------------------------------------------------------------------ policy helpers
def test_make_sum_equal_closed_form():
    a = torch.tensor([2, 0, 10, 10, 10, 5])
    assert O.make_sum_equal(a, 35).tolist() == [2, 0, 10, 10, 8, 5]      # surplus 2 taken from index 4
    assert O.make_sum_equal(a, 40).tolist() == [2, 0, 10, 10, 13, 5]     # deficit added to index 4
    assert O.make_sum_equal(a, 25).tolist() == [2, 0, 10, 8, 0, 5]       # walks down when index 4 runs out
    assert a.tolist() == [2, 0, 10, 10, 10, 5]


def test_block_ranking_and_rerank_brute_force():
    g = torch.Generator().manual_seed(9)
    imp = torch.rand(8 * 32, generator=g)
    idx = O.get_block_token_idx(32, 8, imp)
    means = imp.reshape(8, 32).mean(-1)
    assert idx.reshape(8, 32)[:, 0].div(32, rounding_mode="floor").tolist() == means.argsort(descending=True).tolist()
    assert sorted(idx.tolist()) == list(range(256))
    # survivors' ranks, brute force with Python sets
    classes = [idx[:64], None, idx[64:160], idx[160:224]]   # idx[224:] evicted
    out = O.rerank_after_eviction(classes)
    alive = sorted(set(range(256)) - set(idx[224:].tolist()))
    for c, o in zip(classes, out):
        if c is None:
            assert o is None
        else:
            assert o.tolist() == [alive.index(int(v)) for v in c.tolist()]
    flat = sorted(v for o in out if o is not None for v in o.tolist())
    assert flat == list(range(224))


def test_token_range_closed_form():
    v = torch.tensor([[[[1.0, -2.0, 3.0], [0.0, 0.5, 0.25]]]]).half()  # (1,1,2,3)
    r = O.calculate_token_range(v, None)
    assert r.tolist() == [5.0, 0.5]
    assert O.calculate_token_range(v, r).tolist() == [5.0, 0.5, 5.0, 0.5]
    assert O.calculate_token_range(None, r) is None


def test_class_sizes_worked_by_hand():
    """model/llama_hqe.py:216-224 and :235-239 worked with pencil arithmetic (exact fractions, no case sits on a
    rounding tie), asserted on the oracle AND on the product's formulas.

    416 tokens = 13 blocks, shipped shares 4/2/1 bit = 0.25 each, evicted 0.25: fp16 share 64/416 = 2/13, the
    rest 11/13 * 0.25 = 11/52 each; 13 * (2/13, 0, 11/52 x 4) = (2, 0, 2.75 x 4) -> rounded (2, 0, 3, 3, 3, 3) = 14,
    one too many, taken from the 1-bit entry -> (2, 0, 3, 3, 2, 3) blocks = (64, 0, 96, 96, 64, 96) tokens.
    1056 tokens = 33 blocks, shares 0.2 / 0.3 / 0.4, evicted 0.1: 31/33 of them -> 33 * share = (2, 0, 6.2, 9.3, 12.4,
    3.1) -> (2, 0, 6, 9, 12, 3) = 32, one short, added to the 1-bit entry -> (2, 0, 6, 9, 13, 3) blocks.
    96 tokens = 3 blocks, shares 0.7 / 0.7 / 0 / 0: 3 * (2/3, 0, 0.7/3, 0.7/3, 0, 0) = (2, 0, 0.7, 0.7, 0, 0) -> (2, 0, 1, 1,
    0, 0) = 4, one too many; the 1-bit entry is empty, so the 2-bit entry gives it up -> (2, 0, 1, 0, 0, 0)."""
    from hqekv_amd.decode_layer import class_token_counts, ratios_for_next_increment
    t = lambda *v: torch.tensor(v, dtype=torch.float32)
    cases = [
        (416, t(0.25, 0.25, 0.25), t(0.25), [64, 0, 96, 96, 64, 96], [2 / 13, 0, 11 / 52, 11 / 52, 11 / 52, 11 / 52]),
        (1056, t(0.2, 0.3, 0.4), t(0.1), [64, 0, 192, 288, 416, 96], [2 / 33, 0, 6.2 / 33, 9.3 / 33, 12.4 / 33, 3.1 / 33]),
        (96, t(0.7, 0.7, 0.0), t(0.0), [64, 0, 32, 0, 0, 0], [2 / 3, 0, 0.7 / 3, 0.7 / 3, 0, 0]),
    ]
    for total, rq, re, counts, shares in cases:
        for fn in (O.split_history, class_token_counts):
            got_shares, got_counts = fn(total, rq.clone(), re.clone())
            assert got_counts.tolist() == counts, (fn.__name__, total)
            assert int(got_counts.sum()) == total
            assert torch.allclose(got_shares, torch.tensor(shares, dtype=torch.float32), atol=1e-6)
    # next increment: history 320 -> 32 tokens are added to reach 352; the evicted share becomes 32 * 0.25 / 352 = 1/44,
    # the three quantised shares (equal) take (1 - 1/44) / 3 = 43/132 each
    e, q = ratios_for_next_increment(320, t(0.25), t(0.25, 0.25, 0.25))
    assert torch.allclose(e, t(1 / 44), atol=1e-7) and torch.allclose(q, t(43 / 132, 43 / 132, 43 / 132), atol=1e-7)
    # history 330 (not on the block grid): 22 tokens reach 352; 22 * 0.25 / 352 = 1/64; shares 0.2/0.3/0.5 scaled by 63/64
    e, q = ratios_for_next_increment(330, t(0.25), t(0.2, 0.3, 0.5))
    assert torch.allclose(e, t(1 / 64), atol=1e-7)
    assert torch.allclose(q, t(0.196875, 0.2953125, 0.4921875), atol=1e-7)
    # the oracle's layer applies the same update after a compression: one prompt of 352 tokens with the shipped
    # shares -> 11 blocks: (2, 0, 2.25 x 4 * ...) worked below
    orc = O.DecodeLayerOracle(32, bit_0=0.25, bit_4=0.25, bit_2=0.25, bit_1=0.25, max_length=400)
    g = torch.Generator().manual_seed(1)
    q_, k_, v_ = (torch.randn(1, h, 352, 32, generator=g).half() for h in (2, 1, 1))
    mask = torch.triu(torch.full((352, 352), torch.finfo(torch.float16).min, dtype=torch.float16), 1)[None, None]
    _, _, pkv, aux = orc.step(q_, k_, v_, mask, None, None)
    # 352 tokens = 11 blocks: fp16 64/352 = 2/11; rest 9/11 * 0.25 = 9/44 each; 11 * 9/44 = 2.25 -> (2, 0, 2, 2, 2, 2) = 10,
    # one short -> 1-bit entry 3: (64, 0, 64, 64, 96, 64) tokens, 64 evicted, history 288
    assert aux[1].tolist() == [64, 0, 64, 64, 96, 64] and orc.history_reserve_length == 288
    # next: 288 + 32 = 320: evicted share 32 * 0.25 / 320 = 1/40, quantised (1 - 1/40) / 3 = 13/40 each
    assert torch.allclose(orc.ratio_e, t(1 / 40), atol=1e-7) and torch.allclose(orc.ratio_q, t(0.325, 0.325, 0.325), atol=1e-7)


def test_layer_state_machine_bookkeeping():
    """Prompt + decode steps through the oracle's layer: every token is in exactly one class or the
    residual or was evicted, probabilities sum to one, class sizes follow the ratios."""
    D, B, Hq, Hkv, T0 = 128, 1, 4, 2, 400
    orc = O.DecodeLayerOracle(D, bit_0=0.25, bit_4=0.25, bit_2=0.5, max_length=T0 + 40)
    g = torch.Generator().manual_seed(5)
    pkv, evicted = None, 0
    for step in range(41):
        L = T0 if step == 0 else 1
        q = torch.randn(B, Hq, L, D, generator=g).half()
        k = torch.randn(B, Hkv, L, D, generator=g).half()
        v = torch.randn(B, Hkv, L, D, generator=g).half()
        mask = torch.triu(torch.full((L, L), torch.finfo(torch.float16).min, dtype=torch.float16), 1)[None, None] if step == 0 else None
        out, w, pkv, aux = orc.step(q, k, v, mask, pkv, None)
        assert torch.allclose(w.float().sum(-1), torch.ones(B, Hq, L), atol=2e-2)
        if aux is not None:
            evicted += int(aux[1][-1])
            assert int(aux[1].sum()) % 32 == 0 and int(aux[1][0]) == 64 and int(aux[1][1]) == 0
            # every token of the re-ranked history gets a class: the sizes add up to history + compressed tokens
            assert int(aux[1].sum()) == orc.history_reserve_length + int(aux[1][-1])
        kept = sum(pkv[s].shape[2] for s in (O.V16, O.V_BASE[8], O.V_BASE[4], O.V_BASE[2], O.V_BASE[1]) if pkv[s] is not None)
        resid = 0 if pkv[O.NEW_V] is None else pkv[O.NEW_V].shape[2]
        assert kept == orc.history_reserve_length and resid == orc.current_length
        assert kept + resid + evicted == T0 + step == int(pkv[O.KV_SEQ_LEN])
        idx = torch.cat([pkv[s + 1] for s in (O.V16, O.V_BASE[8], O.V_BASE[4], O.V_BASE[2], O.V_BASE[1]) if pkv[s] is not None])
        assert torch.equal(torch.sort(idx)[0], torch.arange(kept))
    assert evicted > 0


# ------------------------------------------------------------------ 1-bit normal-quantile class
def test_normal1_known_answer_and_closed_form():
    """arange(32): mean 15.5, unbiased std sqrt(88) = 9.3808 -> fp16 9.3828; code = [k > 15.5]; the two
    dequantised values are rnd16(mean -+ rnd16(fp16(0.6745) * std)), worked out with numpy float16."""
    import numpy as np
    x = torch.arange(0, 32, dtype=torch.float16).reshape(1, 1, 1, 32)
    code, std, mean = O.normal_group_quantize_pack_last_dim(x, 32, 1)
    assert (code.item() & 0xFFFFFFFF) == 0xFFFF0000
    assert mean.item() == 15.5 and std.item() == float(np.float16(np.sqrt(88.0)))
    k16 = np.float16(0.6744897501960817)
    assert float(k16) == 0.67431640625
    a = np.float16(k16 * np.float16(std.item()))
    lo, hi = np.float16(np.float16(15.5) - a), np.float16(np.float16(15.5) + a)
    dq = O.normal_group_dequantize_unpack_last_dim(code, std, mean, 32, 1).flatten().tolist()
    assert dq == [float(lo)] * 16 + [float(hi)] * 16


def test_normal1_statistics_and_sign_rule():
    import numpy as np
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(2, 2, 8, 128, generator=g) * 3 + 1).half()
    code, std, mean = O.normal_group_quantize_pack_last_dim(x, 32, 1)
    xg = x.reshape(-1, 32).double().numpy()
    # unbiased (n - 1) standard deviation and plain mean, within one fp16 step of the float64 values
    ref_std, ref_mean = xg.std(axis=1, ddof=1), xg.mean(axis=1)
    assert np.all(np.abs(std.flatten().double().numpy() - ref_std) <= ref_std * 2 ** -10)
    assert np.all(np.abs(mean.flatten().double().numpy() - ref_mean) <= np.maximum(np.abs(ref_mean), 2 ** -10) * 2 ** -10)
    # the code is the sign of x - mean (fp16), ties and negatives to 0
    c = O.unpack_codes(code, 1).reshape(-1, 32)
    u = (x.reshape(-1, 32) - mean.reshape(-1, 1))
    assert torch.equal(c, (u > 0).to(torch.int32))
    # a constant group stores code 0 everywhere
    z = torch.full((1, 1, 1, 32), 2.5, dtype=torch.float16)
    assert O.normal_group_quantize_pack_last_dim(z, 32, 1)[0].item() == 0


def test_kivi_layer_bookkeeping_and_equivalence_to_plain_attention():
    """The KIVI-style state machine (model/llama_kivi.py:96-266): closed-form lengths after every step, and
    its decode step -- per-class GEMV + dense tails + concatenation -- equals plain attention over the
    reconstructed cache (dequantised class followed by the fp16 tail)."""
    R, D, B, Hq, Hkv = 64, 128, 1, 4, 2
    lay = O.KiviLayerOracle(D, k_bits=4, v_bits=2, residual_length=R)
    g = torch.Generator().manual_seed(3)

    def qkv(L):
        return [torch.randn(B, h, L, D, generator=g).half() for h in (Hq, Hkv, Hkv)]

    T = 150
    q, k, v = qkv(T)
    _, _, pkv = lay.step(q, k, v, None, None)
    for step in range(1, 80):
        T += 1
        q, k, v = qkv(1)
        prev = pkv
        out, w, pkv = lay.step(q, k, v, None, prev)
        # K: whole blocks of R quantised, the rest fp16; V: everything but the last R tokens quantised
        n_kq = 0 if pkv[0] is None else pkv[0].shape[3] * 8
        n_kf = 0 if pkv[1] is None else pkv[1].shape[2]
        assert (n_kq, n_kf) == (T // R * R, T % R) and pkv[8] == T
        assert pkv[4].shape[2] == T - R and pkv[5].shape[2] == R
        assert torch.equal(pkv[5][:, :, -1:], v) and (n_kf == 0 or torch.equal(pkv[1][:, :, -1:], k))
        # the same step as plain attention over the reconstructed cache (dequantised class, then the tail)
        kq, k_full, ks, kz, vq, v_full, vs, vz, _ = prev
        k_full = k if k_full is None else torch.cat((k_full, k), 2)
        v_full = torch.cat((v_full, v), 2)
        k_all = k_full if kq is None else torch.cat(
            (O.uniform_group_dequantize_unpack_last_dim(kq, ks, kz, 32, 4).transpose(2, 3), k_full), 2)
        v_all = torch.cat((O.uniform_group_dequantize_unpack_last_dim(vq, vs, vz, 32, 2), v_full), 2)
        assert k_all.shape[2] == v_all.shape[2] == T
        sc = torch.matmul(q.float(), O.repeat_kv(k_all, Hq // Hkv).transpose(2, 3).float()).half()
        w2 = torch.softmax((sc.float() * (torch.tensor(1.0) / torch.tensor(D ** 0.5))).half().float(), -1).half()
        out2 = torch.matmul(w2.float(), O.repeat_kv(v_all, Hq // Hkv).float()).half()
        assert w.shape == (B, Hq, 1, T) and torch.allclose(w.float(), w2.float(), rtol=1e-3, atol=1e-4)
        assert torch.allclose(out.float(), out2.float(), rtol=1e-3, atol=1e-3)


def test_gpu_tree_statistics_restatement():
    """``std_mean_gpu_tree`` (torch's GPU reduction order for a 32-element row, restated): a hand-worked first
    level, the closed form on arange(32), agreement with a float64 two-pass evaluation to one fp16 step, and
    near-agreement with this host's ``torch.std_mean`` (another order: the std may differ in the last place)."""
    # by hand, 2 elements per level: (1, 3) -> delta 2, mean 2, M2 = 2*2*1*0.5 = 2; (5, 9) -> delta 4, mean 7, M2 = 8;
    # merge (n_half = 2): delta 5, mean 4.5, M2 = (2 + 8) + 25 * 2 * 0.5 = 35 = sum (x - 4.5)^2 = 12.25 + 2.25 + 0.25 + 20.25
    x = torch.tensor([[1.0, 3.0, 5.0, 9.0] * 8]).half()
    std, mean = O.std_mean_gpu_tree(x)
    assert float(mean) == 4.5 and float(std) == float(torch.tensor((35.0 * 8 / 31) ** 0.5).half())
    a = torch.arange(32).half()[None]
    std, mean = O.std_mean_gpu_tree(a)
    assert float(mean) == 15.5 and float(std) == float(torch.tensor(88.0 ** 0.5).half())
    g = (torch.randn(20000, 32, generator=torch.Generator().manual_seed(3)) * 2 + 0.5).half()
    std, mean = O.std_mean_gpu_tree(g)
    d = g.double()
    m64 = d.mean(-1, keepdim=True)
    s64 = ((d - m64) ** 2).sum(-1, keepdim=True).div(31).sqrt()
    step = lambda v: torch.exp2(torch.floor(torch.log2(v.abs().clamp_min(2.0 ** -14))) - 10)
    assert bool(((std.double() - s64).abs() <= step(s64)).all()) and bool(((mean.double() - m64).abs() <= step(m64)).all())
    t_std, t_mean = torch.std_mean(g, dim=-1, keepdim=True)
    assert float((t_std != std).float().mean()) < 0.005 and float((t_mean != mean).float().mean()) < 0.005


def test_gpu_tree_statistics_known_answer_next_to_a_rounding_boundary():
    """A group whose std lies 5e-9 below the midpoint of two fp16 numbers (fp32 std 0.88549799, midpoint
    0.88549805): ``torch.std_mean`` on the GPU and the HIP quantiser both give 0.88525390625 / 0.09979248046875
    (recorded from a run on an MI355X).  A square root that is one fp32 unit off -- torch.sqrt on one AVX-512 host
    was -- lands on the other side; the restatement takes it through float64."""
    vals = [0.2332763671875, -0.167236328125, -0.96826171875, -0.53662109375, 1.751953125, 1.48046875, -0.126953125,
            0.1861572265625, -1.0458984375, -1.5888671875, 1.720703125, 0.2330322265625, -1.201171875, 1.0595703125,
            -0.75244140625, -0.381591796875, 0.8837890625, -0.1619873046875, 0.9853515625, -0.08868408203125,
            -0.2069091796875, 0.73486328125, 1.580078125, 0.5078125, -0.798828125, 0.023773193359375, -0.2061767578125,
            -0.11798095703125, 0.1656494140625, -0.93408203125, -0.221435546875, 1.15234375]
    g = torch.tensor(vals, dtype=torch.float16).reshape(1, 1, 32)
    std, mean = O.std_mean_gpu_tree(g)
    assert std.dtype == torch.float16 and float(std) == 0.88525390625 and float(mean) == 0.09979248046875
