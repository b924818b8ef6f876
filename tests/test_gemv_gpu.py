"""Per-class fused dequantize-GEMV against dequantise-then-matmul (the reference's own definition of
correct, quant/cuda_hq_test.py:82,242).  Tolerance: 1e-3 relative + 2e-3 absolute, fp32 accumulation."""
import pytest
import torch

from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 2e-3


def _close(a, b):
    torch.testing.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("T", [32, 992, 4096])
def test_qk_shape(dev, bit, T):
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    g = torch.Generator().manual_seed(100 + bit + T)
    B, Hq, Hkv, D = 2, 8, 2, 128
    k = torch.randn(B, Hkv, D, T, generator=g)
    k[:, :, 3] *= 10
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    code, s, z = O.uniform_group_quantize_pack_last_dim(k.half(), 32, bit)
    out = cuda_bmm_fA_qB_uniform_group(32, q.to(dev), code.to(dev), s.to(dev), z.to(dev), bit)
    assert out.shape == (B, Hq, 1, T) and out.dtype == torch.float16
    _close(out, O.gemv_uniform_group(32, q, code, s, z, bit))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("T", [32, 160, 2080])
def test_pv_shape(dev, bit, T):
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    g = torch.Generator().manual_seed(200 + bit + T)
    B, Hq, Hkv, D = 2, 8, 2, 128
    v = torch.randn(B, Hkv, T, D, generator=g).half()
    p = torch.softmax(torch.randn(B, Hq, 1, T, generator=g) * 3, -1).half()
    code, s, z = O.uniform_group_quantize_pack_last_dim(v, 32, bit)
    out = cuda_bmm_fA_qB_uniform_group(32, p.to(dev), code.to(dev), s.to(dev), z.to(dev), bit)
    assert out.shape == (B, Hq, 1, D)
    _close(out, O.gemv_uniform_group(32, p, code, s, z, bit))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("T", [1, 2, 31, 37, 129, 513, 2081])
def test_pv_shape_any_token_count(dev, bit, T):
    """V is grouped along the channels, so a V class may hold any number of tokens (a KIVI-style cache
    quantises V one token at a time, model/llama_kivi.py:190-203): odd counts, counts below one group of
    lanes, counts that end a chunk with a single token."""
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    g = torch.Generator().manual_seed(250 + bit + T)
    B, Hq, Hkv, D = 2, 8, 2, 128
    v = torch.randn(B, Hkv, T, D, generator=g).half()
    p = torch.softmax(torch.randn(B, Hq, 1, T, generator=g) * 3, -1).half()
    code, s, z = O.uniform_group_quantize_pack_last_dim(v, 32, bit)
    out = cuda_bmm_fA_qB_uniform_group(32, p.to(dev), code.to(dev), s.to(dev), z.to(dev), bit)
    assert out.shape == (B, Hq, 1, D)
    _close(out, O.gemv_uniform_group(32, p, code, s, z, bit))


@pytest.mark.parametrize("n_rep", [1, 2, 3, 4, 6, 7, 8, 11])   # (11: served as slices of 8 + 3 heads)
def test_gqa_group_sizes(dev, n_rep):
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    g = torch.Generator().manual_seed(300 + n_rep)
    B, Hkv, D, T = 1, 2, 128, 256
    Hq = Hkv * n_rep
    k = torch.randn(B, Hkv, D, T, generator=g).half()
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    code, s, z = O.uniform_group_quantize_pack_last_dim(k, 32, 4)
    _close(cuda_bmm_fA_qB_uniform_group(32, q.to(dev), code.to(dev), s.to(dev), z.to(dev), 4),
           O.gemv_uniform_group(32, q, code, s, z, 4))
    v = torch.randn(B, Hkv, T, D, generator=g).half()
    p = torch.rand(B, Hq, 1, T, generator=g).half()
    code, s, z = O.uniform_group_quantize_pack_last_dim(v, 32, 2)
    _close(cuda_bmm_fA_qB_uniform_group(32, p.to(dev), code.to(dev), s.to(dev), z.to(dev), 2),
           O.gemv_uniform_group(32, p, code, s, z, 2))


def test_integer_special_case_is_exact(dev):
    """scale = 1, zero = 0, 8-bit codes, integer q: the GEMV is an exact integer mat-vec."""
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    g = torch.Generator().manual_seed(7)
    B, Hq, Hkv, D, T = 1, 4, 1, 128, 64
    c = torch.randint(0, 8, (B, Hkv, D, T), generator=g, dtype=torch.int32)
    q = torch.randint(-2, 3, (B, Hq, 1, D), generator=g).half()
    code = O.pack_along_last_dim(c, 8)
    s = torch.ones(B, Hkv, D, T // 32, dtype=torch.float16)
    z = torch.zeros_like(s)
    out = cuda_bmm_fA_qB_uniform_group(32, q.to(dev), code.to(dev), s.to(dev), z.to(dev), 8)
    exact = torch.matmul(q.long(), c.long().expand(B, Hq, D, T))
    assert torch.equal(out.cpu().long(), exact)


def test_gemv_errors(dev):
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    q = torch.zeros(1, 4, 1, 128, dtype=torch.float16, device=dev)
    code = torch.zeros(1, 1, 128, 4, dtype=torch.int32, device=dev)
    s = torch.zeros(1, 1, 128, 2, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        cuda_bmm_fA_qB_uniform_group(32, q, code, s, s, 3)
    with pytest.raises(ValueError):
        cuda_bmm_fA_qB_uniform_group(16, q, code, s, s, 2)
    with pytest.raises(ValueError):
        cuda_bmm_fA_qB_uniform_group(32, q, code, s[..., :1], s[..., :1], 2)
    with pytest.raises(TypeError):
        cuda_bmm_fA_qB_uniform_group(32, q.float(), code, s, s, 2)


@pytest.mark.parametrize("shape", ["qk", "pv"])
@pytest.mark.parametrize("T", [32, 992, 2080])
def test_normal_group_gemv(dev, shape, T):
    """cuda_bmm_fA_qB_normal_group (quant/matmul.py:72-95) and its p.V twin over the 1-bit normal-quantile class
    against the reference's criterion: dequantise with the library's own unpack (quant/pack_unpack.py:356-376),
    repeat_kv, matmul.  The stored (std, mean) are the oracle's, so the comparison is of the GEMV alone."""
    from hqekv_amd.matmul import cuda_bmm_fA_qB_normal_group, cuda_bmm_fA_qB_wv_normal_group
    g = torch.Generator().manual_seed(300 + T)
    B, Hq, Hkv, D = 2, 8, 2, 128
    if shape == "qk":
        x = torch.randn(B, Hkv, D, T, generator=g)
        x[:, :, 3] *= 10
        a = torch.randn(B, Hq, 1, D, generator=g).half()
        fn = cuda_bmm_fA_qB_normal_group
    else:
        x = torch.randn(B, Hkv, T, D, generator=g)
        a = torch.softmax(torch.randn(B, Hq, 1, T, generator=g) * 3, -1).half()
        fn = cuda_bmm_fA_qB_wv_normal_group
    code, std, mean = O.normal_group_quantize_pack_last_dim(x.half(), 32, 1)
    out = fn(32, a.to(dev), code.to(dev), std.to(dev), mean.to(dev), 1)
    dq = O.normal_group_dequantize_unpack_last_dim(code, std, mean, 32, 1)
    ref = torch.matmul(a.float(), O.repeat_kv(dq, Hq // Hkv).float())
    assert out.shape == ref.shape and out.dtype == torch.float16
    _close(out, ref)
    # the uniform reading of the same bytes is a different function: the entry points are told apart
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    other = cuda_bmm_fA_qB_uniform_group(32, a.to(dev), code.to(dev), std.to(dev), mean.to(dev), 1)
    assert not torch.allclose(other.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    with pytest.raises(NotImplementedError):
        fn(32, a.to(dev), code.to(dev), std.to(dev), mean.to(dev), 2)
