"""HIP quantise/pack/unpack kernels against the CPU oracle: bit-exact codes, scales and zeros."""
import pytest
import torch

from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu


def _data(shape, seed, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    if outliers:
        x[..., 3::32, :] *= 10.0
    return x.half()


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_quant_rows_bit_exact(dev, bit):
    from hqekv_amd import pack_unpack as P
    x = _data((2, 3, 96, 256), 10 + bit)
    code, scale, mn = P.uniform_group_quantize_pack_last_dim(x.to(dev), 32, bit)
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(x, 32, bit)
    assert code.dtype == torch.int32 and scale.dtype == torch.float16
    assert torch.equal(code.cpu(), oc)
    assert torch.equal(scale.cpu().view(torch.int16), os_.view(torch.int16))
    assert torch.equal(mn.cpu().view(torch.int16), om.view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_quant_k_transposed_view_bit_exact(dev, bit):
    """K reaches the quantiser as the transpose(2, 3) view of token-major memory (quant/hqe_2.py:32-35)."""
    from hqekv_amd import pack_unpack as P
    k = _data((2, 2, 160, 128), 20 + bit, outliers=False)  # (B, H, T, D)
    k[..., 5] *= 10.0
    kd = k.to(dev)
    before = kd.clone()
    code, scale, mn = P.uniform_group_quantize_pack_last_dim(kd.transpose(2, 3), 32, bit)
    assert torch.equal(kd, before), "the input must not be modified"
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(k.transpose(2, 3).contiguous(), 32, bit)
    assert torch.equal(code.cpu(), oc)
    assert torch.equal(scale.cpu().view(torch.int16), os_.view(torch.int16))
    assert torch.equal(mn.cpu().view(torch.int16), om.view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_quant_matches_torch_chain_on_device(dev, bit):
    """The reference's own torch op chain (quant/pack_unpack.py:166-175) evaluated ON THE GPU, which pins
    the tensor / python-int rule and the fp32 divide of the device against the HIP kernel."""
    from hqekv_amd import pack_unpack as P
    x = _data((1, 8, 128, 1024), 30 + bit).to(dev)
    code, scale, mn = P.uniform_group_quantize_pack_last_dim(x, 32, bit)
    g = x.reshape(8 * 128, 1024 // 32, 32).clone()
    t_mn = torch.min(g, dim=-1, keepdim=True)[0]
    t_mx = torch.max(g, dim=-1, keepdim=True)[0]
    t_scale = (t_mx - t_mn) / (2 ** bit - 1)
    g.sub_(t_mn)
    g.div_(t_scale)
    q = g.clamp_(0, 2 ** bit - 1).round_().to(torch.int32).view(1, 8, 128, 1024)
    assert torch.equal(scale.reshape(-1), t_scale.reshape(-1))
    assert torch.equal(mn.reshape(-1), t_mn.reshape(-1))
    assert torch.equal(code.cpu(), O.pack_along_last_dim(q.cpu(), bit))


def test_quant_degenerate_and_extreme_groups(dev):
    from hqekv_amd import pack_unpack as P
    x = torch.zeros(1, 1, 4, 64, dtype=torch.float16)
    x[0, 0, 0, :32] = 1.5                      # constant group -> scale 0, codes 0
    x[0, 0, 1, :] = torch.linspace(-60000, 60000, 64).half()
    x[0, 0, 2, 0] = 6e-8                       # denormal range
    x[0, 0, 3, :] = torch.arange(64).half() / 1024
    for bit in (1, 2, 4, 8):
        code, scale, mn = P.uniform_group_quantize_pack_last_dim(x.to(dev), 32, bit)
        oc, os_, om = O.uniform_group_quantize_pack_last_dim(x, 32, bit)
        assert torch.equal(code.cpu(), oc), bit
        assert torch.equal(scale.cpu().view(torch.int16), os_.view(torch.int16)), bit
        assert torch.equal(mn.cpu().view(torch.int16), om.view(torch.int16)), bit
        dq = P.uniform_group_dequantize_unpack_last_dim(code, scale, mn, 32, bit)
        assert torch.equal(dq.cpu()[0, 0, 0, :32], x[0, 0, 0, :32])


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_dequant_and_unpack_bit_exact(dev, bit):
    from hqekv_amd import pack_unpack as P
    x = _data((1, 2, 64, 512), 40 + bit)
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(x, 32, bit)
    dq = P.uniform_group_dequantize_unpack_last_dim(oc.to(dev), os_.to(dev), om.to(dev), 32, bit)
    ref = O.uniform_group_dequantize_unpack_last_dim(oc, os_, om, 32, bit)
    assert torch.equal(dq.cpu().view(torch.int16), ref.view(torch.int16))
    un = P.unpack_along_last_dim(oc.to(dev), bit)
    assert torch.equal(un.cpu(), O.unpack_along_last_dim(oc, bit))
    fq = P.uniform_group_fake_quant(x.to(dev), 32, bit)
    assert torch.equal(fq.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_pack_roundtrip(dev, bit):
    from hqekv_amd import pack_unpack as P
    g = torch.Generator().manual_seed(bit)
    q = torch.randint(0, 2 ** bit, (2, 2, 16, 128), generator=g, dtype=torch.int32)
    code = P.pack_along_last_dim(q.to(dev), bit)
    assert torch.equal(code.cpu(), O.pack_along_last_dim(q, bit))
    assert torch.equal(P.unpack_along_last_dim(code, bit).cpu().to(torch.int32), q)


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_append_into_capacity_window(dev, bit):
    """Quantise new tokens straight into a window of capacity-sized cache buffers: the bytes written
    equal a stand-alone quantisation and nothing outside the window changes."""
    from hqekv_amd import pack_unpack as P
    pf = 32 // bit
    B, H, D, cap, old, new = 1, 2, 128, 512, 192, 128
    k_new = _data((B, H, new, D), 50 + bit, outliers=False)
    code = torch.full((B, H, D, cap // pf), -1, dtype=torch.int32, device=dev)
    scale = torch.full((B, H, D, cap // 32), -1.0, dtype=torch.float16, device=dev)
    mn = torch.full_like(scale, -1.0)
    P.quantize_pack_into(k_new.to(dev).transpose(2, 3), bit,
                         code[..., old // pf:(old + new) // pf], scale[..., old // 32:(old + new) // 32],
                         mn[..., old // 32:(old + new) // 32])
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(k_new.transpose(2, 3).contiguous(), 32, bit)
    assert torch.equal(code[..., old // pf:(old + new) // pf].cpu(), oc)
    assert torch.equal(scale[..., old // 32:(old + new) // 32].cpu(), os_)
    assert torch.equal(mn[..., old // 32:(old + new) // 32].cpu(), om)
    assert (code[..., :old // pf] == -1).all() and (code[..., (old + new) // pf:] == -1).all()
    assert (scale[..., :old // 32] == -1).all() and (scale[..., (old + new) // 32:] == -1).all()
    # V: token rows appended into (B, H, cap, D/pf)
    v_new = _data((B, H, new, D), 60 + bit, outliers=False)
    vcode = torch.full((B, H, cap, D // pf), -1, dtype=torch.int32, device=dev)
    vs = torch.full((B, H, cap, D // 32), -1.0, dtype=torch.float16, device=dev)
    vz = torch.full_like(vs, -1.0)
    P.quantize_pack_into(v_new.to(dev), bit, vcode[:, :, old:old + new], vs[:, :, old:old + new], vz[:, :, old:old + new])
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(v_new, 32, bit)
    assert torch.equal(vcode[:, :, old:old + new].cpu(), oc)
    assert torch.equal(vs[:, :, old:old + new].cpu(), os_) and torch.equal(vz[:, :, old:old + new].cpu(), om)
    assert (vcode[:, :, :old] == -1).all() and (vcode[:, :, old + new:] == -1).all()


def test_argument_errors(dev):
    from hqekv_amd import pack_unpack as P
    x = torch.zeros(1, 1, 2, 64, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        P.uniform_group_quantize_pack_last_dim(x, 32, 3)
    with pytest.raises(ValueError):
        P.uniform_group_quantize_pack_last_dim(x, 64, 2)
    with pytest.raises(ValueError):
        P.uniform_group_quantize_pack_last_dim(x[..., :48], 32, 2)
    with pytest.raises(TypeError):
        P.uniform_group_quantize_pack_last_dim(x.float(), 32, 2)
    with pytest.raises(RuntimeError):
        P.uniform_group_quantize_pack_last_dim(x.cpu(), 32, 2)


def test_dequant_keeps_the_two_fp16_roundings(dev):
    """10 * fp16(0.1) is a tie that rounds to 1.0 and 2050 + 1.0 is a tie that rounds to 2052; a fused
    multiply-add (one rounding) would give 2050.  The same values must come out of the attention kernels."""
    from hqekv_amd import pack_unpack as P
    from hqekv_amd.matmul import cuda_bmm_fA_qB_uniform_group
    codes = torch.zeros(1, 1, 128, 32, dtype=torch.int32)
    codes[..., 0] = 10
    code = O.pack_along_last_dim(codes, 4)
    s = torch.full((1, 1, 128, 1), 0.0999755859375, dtype=torch.float16)
    z = torch.full((1, 1, 128, 1), 2050.0, dtype=torch.float16)
    dq = P.uniform_group_dequantize_unpack_last_dim(code.to(dev), s.to(dev), z.to(dev), 32, 4)
    assert (dq[..., 0] == 2052.0).all() and (dq[..., 1] == 2050.0).all()
    # q = e_0 picks K[d=0][t]: the GEMV must see 2052 for token 0 (exactly representable in the fp16 output)
    q = torch.zeros(1, 1, 1, 128, dtype=torch.float16)
    q[..., 0] = 1.0
    out = cuda_bmm_fA_qB_uniform_group(32, q.to(dev), code.to(dev), s.to(dev), z.to(dev), 4)
    assert out[0, 0, 0, 0].item() == 2052.0 and out[0, 0, 0, 1].item() == 2050.0


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("magnitude", [2.0 ** -21, 2.0 ** -14, 9000.0])
def test_quant_denormal_and_near_overflow_ranges_both_layouts(dev, bit, magnitude):
    """Scales that are fp16 denormals, underflow to zero, or sit next to overflow; constant and one-hot groups."""
    from hqekv_amd import pack_unpack as P
    g = torch.Generator().manual_seed(int(magnitude * 2 ** 22) % 9973 + bit)
    x = (torch.randn(1, 2, 64, 128, generator=g) * magnitude).half()
    x[0, 0, :8] = x[0, 0, :8, :1]                      # constant rows
    x[0, 1, :, 5] = x[0, 1, :1, 5]                     # constant column
    x[0, 1, 7, 40] += torch.tensor(magnitude * 2 ** -3).half()
    for data in (x, x.transpose(2, 3)):                # rows kernel, token-major K kernel
        code, scale, mn = P.uniform_group_quantize_pack_last_dim(data.to(dev), 32, bit)
        oc, os_, om = O.uniform_group_quantize_pack_last_dim(data.contiguous(), 32, bit)
        assert torch.equal(code.cpu(), oc)
        assert torch.equal(scale.cpu().view(torch.int16), os_.view(torch.int16))
        assert torch.equal(mn.cpu().view(torch.int16), om.view(torch.int16))


def test_reciprocal_division_matches_true_division_for_every_fp16_pair(dev):
    """The quantiser's u * (1/scale) against the correctly rounded u / scale, all 2^32 operand pairs."""
    from hqekv_amd import _lib
    counts = torch.zeros(4, dtype=torch.int64, device=dev)
    _lib.check(_lib.load().hqekv_selftest_quant_division(counts.data_ptr(), _lib.stream_ptr(counts.device)),
               "selftest_quant_division")
    torch.cuda.synchronize()
    c = counts.cpu().tolist()
    assert c[1] == 0, f"{c[1]} code mismatches in the quantiser's domain"
    assert c[0] == 0, f"{c[0]} code mismatches over all pairs"
    # the quotients themselves may differ only on exact ties among fp16 denormals (|v| < 2^-14)
    assert c[3] < 0x0400, f"quotients differ at |v| bits {c[3]:#06x} ({c[2]} pairs)"


# ------------------------------------------------------------------ 1-bit normal-quantile class
def _ulp16(x):
    """Spacing of the fp16 grid at |x| (fp32 tensor in, fp32 out)."""
    e = torch.floor(torch.log2(x.abs().clamp_min(2.0 ** -14)))
    return torch.exp2(e - 10)


@pytest.mark.parametrize("layout", ["rows", "token_major"])
def test_normal1_quantiser_against_oracle(dev, layout):
    """Codes, std and mean bit-identical to the oracle, whose statistics follow the tree order of torch's GPU
    reduction (the order the kernels use).  Against ``torch.std_mean`` as THIS host's CPU evaluates it the std may
    differ in the last fp16 place in rare groups (another accumulation order): asserted <= 1 step, < 0.5 %."""
    from hqekv_amd import pack_unpack as P
    x = (_data((2, 2, 64, 256), 77) * 2 + 0.5)
    data = x if layout == "rows" else x.transpose(2, 3)
    code, std, mean = P.normal_group_quantize_pack_last_dim(data.to(dev), 32, 1)
    oc, os_, om = O.normal_group_quantize_pack_last_dim(data.contiguous(), 32, 1)
    code, std, mean = code.cpu(), std.cpu(), mean.cpu()
    assert torch.equal(code, oc)
    assert torch.equal(std.view(torch.int16), os_.view(torch.int16)) and torch.equal(mean.view(torch.int16), om.view(torch.int16))
    B, nh, R, L = data.shape
    g = data.contiguous().reshape(B * nh * R, L // 32, 32)
    c_std, c_mean = torch.std_mean(g, dim=-1)
    for got, want in ((std, c_std.reshape(std.shape)), (mean, c_mean.reshape(mean.shape))):
        d = (got.float() - want.float()).abs()
        assert bool((d <= _ulp16(want.float())).all())
        assert float((d > 0).float().mean()) < 0.005


@pytest.mark.parametrize("layout", ["rows", "token_major"])
def test_normal1_matches_torch_std_mean_on_device(dev, layout):
    """The reference computes the 1-bit class's statistics with ``torch.std_mean`` on the GPU
    (quant/pack_unpack.py:227).  Its accumulation order is not documented, so the kernel's std / mean are
    compared here with torch's own result executed on this device, bit for bit; the mismatch rate is printed
    and the codes must follow the element-wise rule for the values the kernel stored."""
    from hqekv_amd import pack_unpack as P
    x = (_data((2, 4, 128, 1024), 91) * 2 + 0.5)
    data = (x if layout == "rows" else x.transpose(2, 3)).to(dev)
    code, std, mean = P.normal_group_quantize_pack_last_dim(data, 32, 1)
    B, nh, R, L = data.shape
    g = data.contiguous().reshape(B * nh * R, L // 32, 32)
    t_std, t_mean = torch.std_mean(g, dim=-1, keepdim=True)
    t_std, t_mean = t_std.reshape(std.shape), t_mean.reshape(mean.shape)
    bad_std = int((std.view(torch.int16) != t_std.view(torch.int16)).sum())
    bad_mean = int((mean.view(torch.int16) != t_mean.view(torch.int16)).sum())
    print(f"normal1 {layout}: {bad_std} of {std.numel()} std and {bad_mean} of {mean.numel()} mean values differ "
          f"from torch.std_mean on the device")
    step = lambda a, b: (a.view(torch.int16).to(torch.int32) - b.view(torch.int16).to(torch.int32)).abs().max()
    assert int(step(std, t_std)) <= 1 and int(step(mean, t_mean)) <= 1
    assert bad_std == 0 and bad_mean == 0
    v = (g - mean.reshape(B * nh * R, L // 32, 1)) / std.reshape(B * nh * R, L // 32, 1)
    assert torch.equal(P.unpack_along_last_dim(code, 1).to(torch.int32), (v > 0).to(torch.int32).reshape(B, nh, R, L))


def test_normal1_dequantiser_bit_exact_and_edges(dev):
    from hqekv_amd import pack_unpack as P
    g = torch.Generator().manual_seed(5)
    code = torch.randint(-2 ** 31, 2 ** 31 - 1, (1, 2, 16, 4), generator=g, dtype=torch.int64).to(torch.int32)
    std = (torch.rand(1, 2, 16, 4, generator=g) * 3).half()
    mean = torch.randn(1, 2, 16, 4, generator=g).half()
    std[0, 0, 0, 0], std[0, 0, 0, 1] = 0.0, 6e-8          # zero and denormal spread
    dq = P.normal_group_dequantize_unpack_last_dim(code.to(dev), std.to(dev), mean.to(dev), 32, 1)
    ref = O.normal_group_dequantize_unpack_last_dim(code, std, mean, 32, 1)
    assert torch.equal(dq.cpu().view(torch.int16), ref.view(torch.int16))
    # quantiser edges: constant group -> code 0; tiny spread under a large offset; huge values (std -> inf)
    x = torch.zeros(1, 1, 4, 32, dtype=torch.float16)
    x[0, 0, 0] = 2.5
    x[0, 0, 1] = 1000.0
    x[0, 0, 1, 3] = 1000.5
    x[0, 0, 2] = torch.linspace(-60000, 60000, 32).half()
    x[0, 0, 3, 7] = 6e-8
    c, s, m = P.normal_group_quantize_pack_last_dim(x.to(dev), 32, 1)
    oc, os_, om = O.normal_group_quantize_pack_last_dim(x, 32, 1)
    assert torch.equal(c.cpu(), oc)
    assert torch.equal(s.cpu().view(torch.int16), os_.view(torch.int16))
    assert torch.equal(m.cpu().view(torch.int16), om.view(torch.int16))
    with pytest.raises(NotImplementedError):
        P.normal_group_quantize_pack_last_dim(x.to(dev), 32, 2)


def test_wave_reductions_on_integer_data(dev):
    """The DPP / lane-row-swap reductions of the attention kernels: exact on integer-valued inputs, for
    every position of the maximum and with negative values, and equal to the plain shuffle butterfly."""
    from hqekv_amd import _lib
    g = torch.Generator().manual_seed(9)
    n_waves = 4096 + 3
    x = torch.randint(-1000, 1000, (n_waves, 64), generator=g).float()
    x[:64] = -5.0
    x[torch.arange(64), torch.arange(64)] = 7.0          # the maximum visits every lane
    out = torch.empty(n_waves, 4, dtype=torch.float32, device=dev)
    xd = x.to(dev)
    _lib.check(_lib.load().hqekv_selftest_wave_reduce(xd.data_ptr(), out.data_ptr(), n_waves, _lib.stream_ptr(xd.device)),
               "selftest_wave_reduce")
    o = out.cpu()
    assert torch.equal(o[:, 0], x.sum(1)) and torch.equal(o[:, 1], x.max(1)[0])
    assert torch.equal(o[:, 2], o[:, 0]) and torch.equal(o[:, 3], o[:, 1])


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("layout", ["rows", "token_major"])
def test_signed_zero_extremes_follow_torch_tie_rule(dev, bit, layout):
    """torch.min / torch.max return the lowest-indexed element among equal ones, so a group whose minimum (or
    maximum) is zero stores the sign of its FIRST zero when it holds both +0 and -0.  Zero point, scale and codes
    are compared bit for bit, sign bits included, with torch's op chain on the device and with the oracle."""
    from hqekv_amd import pack_unpack as P
    g = torch.Generator().manual_seed(40 + bit)
    x = torch.randn(1, 2, 16, 64, generator=g).abs().half()           # groups of positive values ...
    nz = torch.tensor(-0.0, dtype=torch.float16)
    x[0, 0, 0, 3], x[0, 0, 0, 9] = 0.0, nz                            # ... minimum zero: +0 first
    x[0, 0, 1, 3], x[0, 0, 1, 9] = nz, 0.0                            # -0 first
    x[0, 0, 2, 31], x[0, 0, 2, 0] = nz, 0.0                           # first and last element of a group
    x[0, 0, 3, 8], x[0, 0, 3, 7] = 0.0, nz                            # across the lanes that share a group
    x[0, 1, 0, :32] = -x[0, 1, 0, :32]                                # maximum zero
    x[0, 1, 0, 5], x[0, 1, 0, 20] = nz, 0.0
    x[0, 1, 1, 32:] = 0.0                                             # a group of zeros only, mixed signs
    x[0, 1, 1, 40], x[0, 1, 1, 63] = nz, nz
    x[0, 1, 2, :32] = nz                                              # all -0
    x[0, 1, 3, :32] = 0.0
    x[0, 1, 3, 0] = nz                                                # -0 first, +0 after
    data = x if layout == "rows" else x.transpose(2, 3).contiguous().transpose(2, 3)
    code, scale, mn = P.uniform_group_quantize_pack_last_dim(data.to(dev), 32, bit)
    t = x.to(dev).reshape(2 * 16, 2, 32).clone()
    t_mn = torch.min(t, dim=-1, keepdim=True)[0]
    t_mx = torch.max(t, dim=-1, keepdim=True)[0]
    t_scale = (t_mx - t_mn) / (2 ** bit - 1)
    bits = lambda a: a.reshape(-1).view(torch.int16)
    assert torch.equal(bits(mn), bits(t_mn)), "zero point (sign of a zero minimum)"
    assert torch.equal(bits(scale), bits(t_scale)), "scale (sign of a zero range)"
    oc, os_, om = O.uniform_group_quantize_pack_last_dim(x, 32, bit)
    assert torch.equal(code.cpu(), oc)
    assert torch.equal(bits(scale.cpu()), bits(os_)) and torch.equal(bits(mn.cpu()), bits(om))


def test_dequant_keeps_the_sign_of_zero_products(dev):
    """rnd16(c * s) is -0 for code 0 and a negative (or -0) scale, and for the -0.6745 centre times a std of +0;
    with a zero point of -0 the value then stays -0, as torch's ``mul_`` / ``add_`` chain on the device gives it
    (a mixed-precision fma with a +0 addend would answer +0).  Arbitrary fp16 bit patterns for scale and zero
    (infinities, NaNs, denormals) ride along."""
    from hqekv_amd import pack_unpack as P
    nz = -0.0
    scale = torch.tensor([-1.5, nz, 0.0, 2.0, -6e-8, float("inf"), 65504.0, 3e-7], dtype=torch.float16).reshape(1, 1, 1, 8)
    zero = torch.tensor([nz, nz, nz, nz, nz, 1.0, nz, nz], dtype=torch.float16).reshape(1, 1, 1, 8)
    g = torch.Generator().manual_seed(3)
    for bit in (1, 2, 4, 8):
        code = torch.randint(-2 ** 31, 2 ** 31 - 1, (1, 1, 1, 8 * bit), generator=g, dtype=torch.int64).to(torch.int32)
        code[..., ::2] = 0                                   # every other word: zero codes
        out = P.uniform_group_dequantize_unpack_last_dim(code.to(dev), scale.to(dev), zero.to(dev), 32, bit)
        c = O.unpack_codes(code, bit).to(dev).to(torch.float16).reshape(1, 1, 1, 8, 32)
        ref = (c * scale.to(dev).unsqueeze(-1) + zero.to(dev).unsqueeze(-1)).reshape(1, 1, 1, 256)
        nan = torch.isnan(ref)
        assert torch.equal(torch.isnan(out), nan)
        assert torch.equal(out[~nan].view(torch.int16), ref[~nan].view(torch.int16)), bit
        assert bool((out[..., :32 // bit].view(torch.int16) == -32768).all())   # code 0, scale -1.5, zero -0  ->  -0
    code = torch.tensor([[[[0x0000FFFF] * 8]]], dtype=torch.int32)
    out = P.normal_group_dequantize_unpack_last_dim(code.to(dev), scale.abs().to(dev), zero.to(dev), 32, 1)
    c = O.unpack_codes(code, 1).to(dev).reshape(1, 1, 1, 8, 32)
    k = torch.tensor(O.NORMAL1_CENTER, dtype=torch.float16, device=dev)
    ref = (torch.where(c > 0, k, -k) * scale.abs().to(dev).unsqueeze(-1) + zero.to(dev).unsqueeze(-1)).reshape(1, 1, 1, 256)
    nan = torch.isnan(ref)
    assert torch.equal(torch.isnan(out), nan)
    assert torch.equal(out[~nan].view(torch.int16), ref[~nan].view(torch.int16))
    assert bool((out[0, 0, 0, 32 + 16:64].view(torch.int16) == -32768).all())   # std +0, mean -0, code 0  ->  -0
