"""The decode caller (prompt -> cache tuple -> decode steps with periodic compression) on the HIP path
against the oracle's restatement of the same layer, in lockstep.

The oracle's ring is fed with the probabilities the GPU produced (and, after each call, aligned to the
GPU ring bit for bit), so both sides take their policy decisions from identical importance values and the
caches can be compared bit for bit after every call; the probabilities and outputs themselves are compared
with the attention tolerance (1e-3 relative + 2e-3 absolute)."""
import pytest
import torch

from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 2e-3


def _qkv(B, Hq, Hkv, L, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, L, D, generator=g)
    k = torch.randn(B, Hkv, L, D, generator=g)
    for ch in (3, 35, 67, 99):
        k[..., ch] *= 10.0
    v = torch.randn(B, Hkv, L, D, generator=g)
    return q.half(), k.half(), v.half()


def _causal_mask(T):
    m = torch.full((T, T), torch.finfo(torch.float16).min, dtype=torch.float16)
    return torch.triu(m, diagonal=1)[None, None]


def _same_tuple(got, want, where, normal=False):
    assert len(got) == len(want) == 42
    for i, (a, b) in enumerate(zip(got, want)):
        if i == 41:
            assert int(a) == int(b), (where, i)
            continue
        assert (a is None) == (b is None), (where, i)
        if a is None:
            continue
        a = a.cpu()
        assert a.shape == b.shape and a.dtype == b.dtype, (where, i, a.shape, b.shape)
        if a.dtype == torch.float16:
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (where, i)
        else:
            assert torch.equal(a, b), (where, i)


@pytest.mark.parametrize("B,Hq,Hkv,T0,steps,strategy,bit_1", [
    (1, 8, 2, 300, 72, "uniform_group", 0.0),
    (2, 4, 4, 96, 40, "uniform_group", 0.0),
    (1, 8, 2, 300, 72, "high_uniform_group_low_normal_group", 0.25),   # the reference's shipped default
    (1, 4, 2, 20, 70, "uniform_group", 0.0),                            # prompt shorter than one block
    (2, 16, 4, 511, 40, "high_uniform_group_low_normal_group", 0.1),    # ragged prompt, GQA 4, two batch rows
    (1, 6, 2, 200, 40, "uniform_group", 0.0),                           # three query heads per KV head
    (2, 12, 2, 130, 40, "high_uniform_group_low_normal_group", 0.1),    # six per KV head
])
def test_layer_in_lockstep_with_oracle(dev, B, Hq, Hkv, T0, steps, strategy, bit_1):
    from hqekv_amd.decode_layer import HqeAttentionLayer
    D = 128
    ratios = dict(bit_0=0.2, bit_4=0.3, bit_2=0.5 - bit_1, bit_1=bit_1)
    layer = HqeAttentionLayer(D, **ratios, quant_strategy=strategy)
    layer.set_max_length(T0 + steps)
    orc = O.DecodeLayerOracle(D, **ratios, max_length=T0 + steps, quant_strategy=strategy)

    pkv_g = pkv_o = None
    compressions = 0
    for step in range(steps + 1):
        L = T0 if step == 0 else 1
        q, k, v = _qkv(B, Hq, Hkv, L, D, 4200 + step)
        mask = _causal_mask(T0) if step == 0 else None
        out_g, w_g, pkv_g, aux_g = layer(q.to(dev), k.to(dev), v.to(dev),
                                         None if mask is None else mask.to(dev), pkv_g, None)
        w_obs = w_g.cpu()
        out_o, w_o, pkv_o, aux_o = orc.step(q, k, v, mask, pkv_o, None,
                                            observed=w_obs if step else None)
        if step == 0:   # the oracle keeps every prompt row, the layer the last 20
            w_o = w_o[:, :, -w_obs.shape[2]:, :]
        where = f"step {step}"
        assert torch.allclose(w_obs.float(), w_o.float(), rtol=RTOL, atol=ATOL), where
        # the prompt's output comes from torch's fused attention (outside the quantised path): looser there
        o_rtol, o_atol = (RTOL, ATOL) if step else (1e-2, 1e-2)
        assert torch.allclose(out_g.cpu().float(), out_o.float(), rtol=o_rtol, atol=o_atol), where
        assert (aux_g is None) == (aux_o is None), where
        if aux_g is not None:
            compressions += 1
            assert torch.equal(aux_g[1], aux_o[1]) and torch.equal(aux_g[2], aux_o[2]), where
        assert layer.current_length == orc.current_length, where
        assert layer.history_reserve_length == orc.history_reserve_length, where
        assert torch.equal(layer.ratio_e, orc.ratio_e) and torch.equal(layer.ratio_q, orc.ratio_q), where
        # rings: the same rows summed on the GPU and on the CPU, then aligned exactly
        ring_g = layer.last_weights.weights.cpu()
        assert torch.allclose(ring_g.float(), orc.ring.weights.float(), rtol=2e-3, atol=1e-3), where
        assert layer.last_weights.next_line == orc.ring.next_line, where
        orc.ring.weights.copy_(ring_g)
        _same_tuple(pkv_g, pkv_o, where, normal=strategy != "uniform_group")
    assert compressions >= 2
    kept = sum(pkv_g[s].shape[2] for s in (2, 8, 16, 24, 32) if pkv_g[s] is not None)
    assert kept == layer.history_reserve_length
    assert int(pkv_g[41]) == T0 + steps
