"""Two decoder layers around the decode caller, the way the reference's model loop drives it
(model/llama_hqe.py:211-214, 241: layer 0 sizes the precision classes and hands its ``auxiliary_parameters``
to every later layer of the same step), against one ``DecodeLayerOracle`` per layer in lockstep.

The projections, rotary embedding and MLP are a random-weight Llama-shaped stack (32 query heads over 8 KV heads of
128 channels, narrow hidden size) that runs on the GPU for both sides: each layer's q, k, v are copied to the host for
the oracle, the residual stream continues from the GPU layer's output.  Cache tuples are compared bit for bit after
every call of every layer, probabilities and outputs with the attention tolerance (1e-3 relative + 2e-3 absolute)."""
import pytest
import torch

from oracle import hqe_oracle as O
from tests.test_decode_layer_gpu import ATOL, RTOL, _causal_mask, _same_tuple

pytestmark = pytest.mark.gpu


def _close(got, want, rtol, atol, where):
    got, want = got.float(), want.float()
    excess = ((got - want).abs() - (atol + rtol * want.abs())).max().item()
    assert excess <= 0, f"{where}: {excess:.3e} over the tolerance"


def _small_llama(n_layers, dev):
    import bench

    class Small(bench._RandomLlama):
        HID, FFN, VOCAB = 512, 1024, 2048

    m = Small(n_layers, dev, seed=77)
    for lw in m.layers:          # wider q and k than N(0, 0.02) weights give: the softmax should not be flat
        lw["qkv"][: (m.HQ + m.HKV) * m.D] *= 3.0
    return m


@pytest.mark.parametrize("B,T0,steps,strategy,bit_1", [
    (2, 300, 40, "uniform_group", 0.0),
    (1, 301, 72, "high_uniform_group_low_normal_group", 0.2),
])
def test_two_layers_share_layer0_class_sizes(dev, B, T0, steps, strategy, bit_1):
    from hqekv_amd.decode_layer import HqeAttentionLayer
    NL = 2
    m = _small_llama(NL, dev)
    ratios = dict(bit_0=0.2, bit_4=0.3, bit_2=0.5 - bit_1, bit_1=bit_1)
    att = [HqeAttentionLayer(m.D, **ratios, quant_strategy=strategy) for _ in range(NL)]
    orc = [O.DecodeLayerOracle(m.D, **ratios, max_length=T0 + steps, quant_strategy=strategy) for _ in range(NL)]
    for a in att:
        a.set_max_length(T0 + steps)
    g = torch.Generator(device=dev).manual_seed(5)
    nxt = torch.randint(0, m.VOCAB, (B, T0), generator=g, device=dev)
    pkv_g, pkv_o = [None] * NL, [None] * NL
    handed_down = 0
    for step in range(steps + 1):
        L = T0 if step == 0 else 1
        pos = torch.arange(T0, device=dev) if step == 0 else torch.full((1,), T0 + step - 1, device=dev)
        mask = _causal_mask(T0) if step == 0 else None
        x, rot = m.embed[nxt], m.rot(pos)
        aux_g = aux_o = None
        for l, lw in enumerate(m.layers):
            where = f"step {step} layer {l}"
            q, k, v = m.qkv(lw, x, rot)
            out_g, w_g, pkv_g[l], aux_g = att[l](q, k, v, None if mask is None else mask.to(dev), pkv_g[l],
                                                 aux_g if l > 0 else None)
            w_obs = w_g.cpu()
            out_o, w_o, pkv_o[l], aux_o = orc[l].step(q.cpu().contiguous(), k.cpu().contiguous(), v.cpu().contiguous(),
                                                      mask, pkv_o[l], aux_o if l > 0 else None,
                                                      observed=w_obs if step else None)
            if step == 0:
                w_o = w_o[:, :, -w_obs.shape[2]:, :]
            _close(w_obs, w_o, RTOL, ATOL, where + " probabilities")
            o_rtol, o_atol = (RTOL, ATOL) if step else (1e-2, 1e-2)
            _close(out_g.cpu(), out_o, o_rtol, o_atol, where + " output")
            assert (aux_g is None) == (aux_o is None), where
            if aux_g is not None:
                assert all(torch.equal(a.cpu(), b) for a, b in zip(aux_g, aux_o)), where
                handed_down += l > 0
            assert att[l].current_length == orc[l].current_length, where
            assert att[l].history_reserve_length == orc[l].history_reserve_length, where
            assert torch.equal(att[l].ratio_e, orc[l].ratio_e) and torch.equal(att[l].ratio_q, orc[l].ratio_q), where
            ring_g = att[l].last_weights.weights.cpu()
            _close(ring_g, orc[l].ring.weights, 2e-3, 1e-3, where + " ring")
            assert att[l].last_weights.next_line == orc[l].ring.next_line, where
            orc[l].ring.weights.copy_(ring_g)
            _same_tuple(pkv_g[l], pkv_o[l], where)
            x = m.after_attention(lw, x, out_g)
        # every layer evicts what layer 0 sized, so all keep the same number of tokens (the split of the kept ones over
        # the classes may differ: a block never moves back up to a higher precision, and each layer ranks its own)
        assert len({a.history_reserve_length for a in att}) == 1, step
        nxt = m.logits(x[:, -1:]).argmax(-1)
    assert handed_down >= 2
    # a later layer keeps the ratios it was built with: only layer 0 rescales them (model/llama_hqe.py:233-239)
    assert torch.equal(att[1].ratio_e, att[1].ratio_e_0) and not torch.equal(att[0].ratio_e, att[0].ratio_e_0)
