"""The KIVI-style caller (every token kept; K quantised per channel in blocks of 128 tokens, V per token one
token at a time, fp16 tails) on the HIP path, in lockstep with the oracle's restatement of
model/llama_kivi.py:96-266.  Cache tuples must be bit-identical; probabilities and outputs within
1e-3 relative + 2e-3 absolute."""
import pytest
import torch

from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 2e-3
D = 128


def _qkv(B, Hq, Hkv, L, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, L, D, generator=g)
    k = torch.randn(B, Hkv, L, D, generator=g)
    for ch in (3, 35, 67, 99):
        k[..., ch] *= 10.0
    v = torch.randn(B, Hkv, L, D, generator=g)
    return q.half(), k.half(), v.half()


def _same_tuple(got, want, where):
    assert len(got) == len(want) == 9
    assert int(got[8]) == int(want[8]), where
    for i, (a, b) in enumerate(zip(got[:8], want[:8])):
        assert (a is None) == (b is None), (where, i)
        if a is None:
            continue
        a = a.cpu()
        assert a.shape == b.shape and a.dtype == b.dtype, (where, i, a.shape, b.shape)
        if a.dtype == torch.float16:
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (where, i)
        else:
            assert torch.equal(a, b), (where, i)


@pytest.mark.parametrize("B,Hq,Hkv,T0,steps,k_bits,v_bits,R", [
    (1, 8, 2, 300, 140, 2, 2, 128),   # upstream's setting; crosses a K block boundary, V grows every step
    (2, 4, 4, 100, 70, 4, 2, 128),    # prompt shorter than the residual: nothing quantised at first
    (1, 8, 2, 256, 12, 2, 4, 128),    # prompt a multiple of the residual: no fp16 K tail after it
    (1, 4, 1, 70, 80, 8, 1, 32),      # short residual, 8-bit K, 1-bit V
])
def test_kivi_layer_in_lockstep_with_oracle(dev, B, Hq, Hkv, T0, steps, k_bits, v_bits, R):
    from hqekv_amd.kivi_layer import KiviAttentionLayer
    layer = KiviAttentionLayer(D, k_bits, v_bits, 32, R)
    orc = O.KiviLayerOracle(D, k_bits, v_bits, 32, R)
    pkv_g = pkv_o = None
    for step in range(steps + 1):
        L = T0 if step == 0 else 1
        q, k, v = _qkv(B, Hq, Hkv, L, 9100 + step)
        mask = None
        if step == 0:
            mask = torch.triu(torch.full((T0, T0), torch.finfo(torch.float16).min, dtype=torch.float16), 1)[None, None]
        out_g, w_g, pkv_g = layer(q.to(dev), k.to(dev), v.to(dev), None if mask is None else mask.to(dev), pkv_g)
        # the oracle's output is formed from the layer's own probabilities: each stage is compared on equal inputs
        out_o, w_o, pkv_o = orc.step(q, k, v, mask, pkv_o, observed=None if step == 0 else w_g.cpu())
        where = f"step {step}"
        if step == 0:   # torch's fused attention for the prompt (outside the quantised path): looser
            assert w_g is None
            assert torch.allclose(out_g.cpu().float(), out_o.float(), rtol=1e-2, atol=1e-2), where
        else:
            assert w_g.shape == w_o.shape == (B, Hq, 1, T0 + step), where
            assert torch.allclose(w_g.cpu().float(), w_o.float(), rtol=RTOL, atol=ATOL), where
            assert torch.allclose(out_g.cpu().float(), out_o.float(), rtol=RTOL, atol=ATOL), where
        _same_tuple(pkv_g, pkv_o, where)
    assert int(pkv_g[8]) == T0 + steps
    # what is quantised and what is still fp16 adds up to the sequence, on both sides
    pf_k = 32 // k_bits
    n_kq = 0 if pkv_g[0] is None else pkv_g[0].shape[3] * pf_k
    n_kf = 0 if pkv_g[1] is None else pkv_g[1].shape[2]
    assert n_kq + n_kf == T0 + steps and n_kq % R == 0 and n_kf < R
    n_vq = 0 if pkv_g[4] is None else pkv_g[4].shape[2]
    assert n_vq + pkv_g[5].shape[2] == T0 + steps and pkv_g[5].shape[2] <= R


def test_kivi_in_place_steps_grow_slide_and_mix_with_the_plain_sequence(dev, monkeypatch):
    """The in-place decode step with tiny buffers -- the V class outgrows its capacity several times, the V tail window
    wraps -- and with steps of upstream's plain sequence in between (an all-zero additive mask sends a step there; the
    next step takes the tuple over into fresh buffers): the tuples stay bit-identical to the oracle's, and a second
    layer that only ever runs the plain sequence sees the same tuples and outputs."""
    from hqekv_amd.kivi_layer import KiviAttentionLayer
    monkeypatch.setattr(KiviAttentionLayer, "MIN_V_ROWS", 8)
    B, Hq, Hkv, T0, steps, R = 2, 8, 2, 45, 150, 32
    fast, plain = KiviAttentionLayer(D, 2, 2, 32, R), KiviAttentionLayer(D, 2, 2, 32, R)
    plain.in_place = False
    orc = O.KiviLayerOracle(D, 2, 2, 32, R)
    pf = pp = po = None
    for step in range(steps + 1):
        L = T0 if step == 0 else 1
        q, k, v = _qkv(B, Hq, Hkv, L, 5200 + step)
        mask = None
        if step in (7, 8, 60, 111):
            mask = torch.zeros(B, 1, 1, T0 + step, dtype=torch.float16, device=dev)
        out_f, w_f, pf = fast(q.to(dev), k.to(dev), v.to(dev), mask, pf)
        out_p, w_p, pp = plain(q.to(dev), k.to(dev), v.to(dev), mask, pp)
        _, _, po = orc.step(q, k, v, None, po, observed=None if step == 0 else w_f.cpu())
        where = f"step {step}"
        _same_tuple(pf, po, where)
        _same_tuple(pp, po, where)
        if step and mask is None:
            assert torch.allclose(w_f.float(), w_p.float(), rtol=RTOL, atol=ATOL), where
            assert torch.allclose(out_f.float(), out_p.float(), rtol=RTOL, atol=ATOL), where
    assert fast._st is not None and fast._st.vcode.shape[2] >= pf[4].shape[2] > 8 * 8   # grown more than once


def test_kivi_decode_with_mask(dev):
    """An additive mask on a decode step takes the general path (scale, mask, clamp, softmax as its own launch)."""
    from hqekv_amd.kivi_layer import KiviAttentionLayer
    B, Hq, Hkv, T0 = 1, 8, 2, 200
    layer, orc = KiviAttentionLayer(D), O.KiviLayerOracle(D)
    q, k, v = _qkv(B, Hq, Hkv, T0, 1)
    _, _, pkv_g = layer(q.to(dev), k.to(dev), v.to(dev), None, None)
    _, _, pkv_o = orc.step(q, k, v, None, None)
    q, k, v = _qkv(B, Hq, Hkv, 1, 2)
    mask = torch.zeros(B, 1, 1, T0 + 1, dtype=torch.float16)
    mask[..., 5:40] = torch.finfo(torch.float16).min
    out_g, w_g, _ = layer(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), pkv_g)
    out_o, w_o, _ = orc.step(q, k, v, mask, pkv_o)
    assert float(w_g[..., 5:40].abs().max()) == 0.0
    assert torch.allclose(w_g.cpu().float(), w_o.float(), rtol=RTOL, atol=ATOL)
    assert torch.allclose(out_g.cpu().float(), out_o.float(), rtol=RTOL, atol=ATOL)


def test_kivi_layer_argument_errors(dev):
    from hqekv_amd.kivi_layer import KiviAttentionLayer
    with pytest.raises(ValueError):
        KiviAttentionLayer(D, residual_length=100)
    with pytest.raises(ValueError):
        KiviAttentionLayer(D, k_bits=3)
    with pytest.raises(ValueError):
        KiviAttentionLayer(D, group_size=64)
