"""The prompt-side kernels against plain torch fp32 attention and against the reference's own op chain for the last
rows [model/llama_hqe.py:141-188], both evaluated on the device.  Tolerances: the output of the whole-prompt attention
within 2e-3 (absolute and relative) of the fp32 result -- probabilities enter the second product as fp16, as in
flash-attention --; the last rows' probabilities within 2 fp16 steps (relative 2e-3, absolute 2e-6) of the torch chain,
whose matmul accumulates in another order before the same roundings."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


def _qkv(B, Hq, Hkv, T, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, T, 128, generator=g) * spread).half()
    k = (torch.randn(B, Hkv, T, 128, generator=g) * spread).half()
    v = torch.randn(B, Hkv, T, 128, generator=g).half()
    return q.to(_dev()), k.to(_dev()), v.to(_dev())


def _dense(q, k, v, scale, causal):
    B, Hq, T, D = q.shape
    n_rep = Hq // k.shape[1]
    k32 = k.float().repeat_interleave(n_rep, dim=1)
    v32 = v.float().repeat_interleave(n_rep, dim=1)
    s = torch.matmul(q.float(), k32.transpose(2, 3)) * scale
    if causal:
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool, device=q.device).triu(1), float("-inf"))
    return torch.matmul(torch.softmax(s, dim=-1), v32)


@pytest.mark.parametrize("B,Hq,Hkv,T", [(1, 4, 1, 64), (1, 4, 4, 129), (2, 8, 2, 300), (1, 32, 8, 777), (1, 8, 1, 1), (1, 2, 2, 20),
                                        (3, 4, 2, 1024), (1, 8, 8, 2049)])
@pytest.mark.parametrize("causal", [True, False])
def test_prompt_attention_matches_fp32(B, Hq, Hkv, T, causal):
    from hqekv_amd.prompt_attention import prompt_attention
    q, k, v = _qkv(B, Hq, Hkv, T, 1000 + T)
    scale = 1.0 / math.sqrt(128)
    out = prompt_attention(q, k, v, scale, causal=causal)
    ref = _dense(q, k, v, scale, causal)
    torch.testing.assert_close(out.float(), ref, rtol=2e-3, atol=2e-3)


def test_prompt_attention_reads_strided_inputs():
    """Slices of a fused (B, T, (Hq + 2 Hkv) * 128) projection, as a model hands them over."""
    from hqekv_amd.prompt_attention import prompt_attention
    B, Hq, Hkv, T = 2, 8, 2, 333
    g = torch.Generator().manual_seed(5)
    fused = torch.randn(B, T, (Hq + 2 * Hkv) * 128, generator=g).half().to(_dev())
    q = fused[..., :Hq * 128].view(B, T, Hq, 128).transpose(1, 2)
    k = fused[..., Hq * 128:(Hq + Hkv) * 128].view(B, T, Hkv, 128).transpose(1, 2)
    v = fused[..., (Hq + Hkv) * 128:].view(B, T, Hkv, 128).transpose(1, 2)
    scale = 0.1
    out = prompt_attention(q, k, v, scale)
    torch.testing.assert_close(out.float(), _dense(q, k, v, scale, True), rtol=2e-3, atol=2e-3)


def test_prompt_attention_sharp_rows():
    """Large logits: rows dominated by one key, running maximum replaced many times along the row."""
    from hqekv_amd.prompt_attention import prompt_attention
    q, k, v = _qkv(1, 4, 2, 600, 77, spread=4.0)
    out = prompt_attention(q, k, v, 0.5)
    torch.testing.assert_close(out.float(), _dense(q, k, v, 0.5, True), rtol=2e-3, atol=2e-3)


def _reference_last_rows(q, k, scale, rows, mask):
    """model/llama_hqe.py:156-168 in torch on the device."""
    n_rep = q.shape[1] // k.shape[1]
    kt = k.transpose(2, 3).contiguous()
    w = torch.matmul(q[:, :, -rows:, :], kt.repeat_interleave(n_rep, dim=1)) * scale
    w = w + mask[:, :, -rows:, :]
    w = torch.max(w, torch.tensor(torch.finfo(w.dtype).min, dtype=w.dtype, device=w.device))
    return torch.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)


def _causal_mask(T, dev):
    m = torch.full((T, T), torch.finfo(torch.float16).min, dtype=torch.float16, device=dev).triu(1)
    return m[None, None]


@pytest.mark.parametrize("B,Hq,Hkv,T,rows", [(1, 4, 1, 64, 20), (2, 8, 2, 300, 20), (1, 32, 8, 4111, 20), (1, 4, 4, 20, 20),
                                             (1, 4, 2, 7, 7), (2, 4, 1, 1000, 32), (1, 8, 2, 33, 1)])
@pytest.mark.parametrize("with_mask", [True, False])
def test_last_rows_match_the_reference_chain(B, Hq, Hkv, T, rows, with_mask):
    from hqekv_amd.prompt_attention import prompt_last_rows
    q, k, _ = _qkv(B, Hq, Hkv, T, 2000 + T)
    scale = 1.0 / math.sqrt(128)
    mask = _causal_mask(T, q.device)
    got = prompt_last_rows(q, k, scale, rows, attention_mask=mask if with_mask else None)
    want = _reference_last_rows(q, k, scale, rows, mask)
    assert got.shape == want.shape == (B, Hq, rows, T)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-3, atol=2e-6)
    torch.testing.assert_close(got.float().sum(-1), torch.ones(B, Hq, rows, device=q.device), rtol=0, atol=2e-3)


def test_last_rows_with_a_padding_mask():
    """A mask that is not causal: the first keys of batch row 1 are padding."""
    from hqekv_amd.prompt_attention import prompt_last_rows
    B, Hq, Hkv, T, rows = 2, 4, 2, 200, 20
    q, k, _ = _qkv(B, Hq, Hkv, T, 31)
    mask = _causal_mask(T, q.device).repeat(B, 1, 1, 1).contiguous()
    mask[1, :, :, :37] = torch.finfo(torch.float16).min
    got = prompt_last_rows(q, k, 0.09, rows, attention_mask=mask)
    want = _reference_last_rows(q, k, 0.09, rows, mask)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-3, atol=2e-6)
    assert float(got[1, :, :, :37].abs().max()) == 0.0


def test_prompt_entries_refuse_bad_arguments():
    from hqekv_amd.prompt_attention import prompt_attention, prompt_last_rows
    q, k, v = _qkv(1, 4, 2, 40, 3)
    with pytest.raises(NotImplementedError):
        prompt_attention(q.float(), k.float(), v.float(), 0.1)
    with pytest.raises(ValueError):
        prompt_last_rows(q, k, 0.1, 33)
    with pytest.raises(ValueError):
        prompt_last_rows(q, k, 0.1, 0)
    with pytest.raises(ValueError):
        prompt_last_rows(q, k, 0.1, 20, attention_mask=torch.zeros(1, 4, 40, 40, dtype=torch.float16, device=q.device))   # a mask per head
    with pytest.raises(Exception):
        prompt_attention(q, k[:, :1].expand(1, 3, 40, 128), v, 0.1)   # 4 query heads over 3 KV heads
    with pytest.raises(Exception):
        prompt_attention(q, k, v, -0.1)                               # the running maximum assumes a positive scale


def test_layer_prompt_without_a_mask_equals_the_causal_mask():
    """The attention layer's prompt call: no mask (the library's kernels, causal rule) against an explicit causal mask
    (torch's fused attention for the output), same probabilities for the ring and the same cache tuple."""
    from hqekv_amd.decode_layer import HqeAttentionLayer
    B, Hq, Hkv, T = 2, 8, 2, 157
    q, k, v = _qkv(B, Hq, Hkv, T, 404)
    outs = []
    for mask in (None, _causal_mask(T, q.device)):
        layer = HqeAttentionLayer(128, bit_0=0.2, bit_4=0.4, bit_2=0.4, bit_1=0.0)
        layer.set_max_length(T + 8)
        outs.append(layer(q, k, v, mask, None, None))
    (o_a, w_a, pkv_a, _), (o_b, w_b, pkv_b, _) = outs
    torch.testing.assert_close(o_a.float(), o_b.float(), rtol=2e-3, atol=2e-3)
    assert w_a.shape == w_b.shape == (B, Hq, 20, T)
    torch.testing.assert_close(w_a.float(), w_b.float(), rtol=2e-3, atol=2e-6)
    assert len(pkv_a) == len(pkv_b) == 42
    for fa, fb in zip(pkv_a, pkv_b):
        assert (fa is None) == (fb is None)


def test_prompt_attention_at_full_size_against_torch_fused_attention():
    """The benchmark's shape (B=1, 32 query heads over 8 KV heads, 32768 tokens): against torch's own fused attention
    on the device -- two fp16-probability implementations, so the tolerance is twice the one against fp32 --, and the
    rows of the last block against the fp32 definition."""
    from hqekv_amd.prompt_attention import prompt_attention
    B, Hq, Hkv, T = 1, 32, 8, 32768
    g = torch.Generator(device=_dev()).manual_seed(99)
    q = torch.randn(B, Hq, T, 128, generator=g, device=_dev(), dtype=torch.float16)
    k = torch.randn(B, Hkv, T, 128, generator=g, device=_dev(), dtype=torch.float16)
    v = torch.randn(B, Hkv, T, 128, generator=g, device=_dev(), dtype=torch.float16)
    scale = 1.0 / math.sqrt(128)
    out = prompt_attention(q, k, v, scale)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale, enable_gqa=True)
    torch.testing.assert_close(out.float(), ref.float(), rtol=4e-3, atol=4e-3)
    # the last 64 rows of two heads, dense in fp32
    for h in (0, 31):
        s = (q[0, h, -64:].float() @ k[0, h // 4].float().T) * scale
        keep = torch.arange(T, device=_dev())[None, :] <= torch.arange(T - 64, T, device=_dev())[:, None]
        want = torch.softmax(s.masked_fill(~keep, float("-inf")), dim=-1) @ v[0, h // 4].float()
        torch.testing.assert_close(out[0, h, -64:].float(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("B,Hq,Hkv,T,rows", [(1, 4, 1, 9000, 20), (1, 32, 8, 32768, 20), (2, 8, 2, 4097, 32)])
def test_last_rows_in_key_slices_equal_the_single_workgroup_form(B, Hq, Hkv, T, rows):
    """Few heads: the keys are cut into slices over more workgroups (two launches and a workspace).  Same
    probabilities as one workgroup per head, to the last fp16 step or two (the slices' sums are merged in another
    order), and both within tolerance of the reference chain."""
    from hqekv_amd import _lib
    from hqekv_amd.prompt_attention import prompt_last_rows
    assert _lib.load().hqekv_prompt_last_rows_workspace_bytes(B, Hq, T) > 0
    q, k, _ = _qkv(B, Hq, Hkv, T, 3000 + T)
    scale = 1.0 / math.sqrt(128)
    a = prompt_last_rows(q, k, scale, rows, sliced=True)
    b = prompt_last_rows(q, k, scale, rows, sliced=False)
    torch.testing.assert_close(a.float(), b.float(), rtol=2e-3, atol=2e-6)
    want = _reference_last_rows(q, k, scale, rows, _causal_mask(T, q.device))
    torch.testing.assert_close(a.float(), want.float(), rtol=2e-3, atol=2e-6)
