"""Hybrid decode attention (all precision classes in one launch, evicted tokens absent) against the
CPU oracle.  Probabilities and outputs: 1e-3 relative + 2e-3 absolute with fp32 accumulation."""
import pytest
import torch

from hqekv_amd import synth
from oracle import hqe_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 2e-3


def _close(a, b, what=""):
    torch.testing.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, msg=lambda m: f"{what}: {m}")


def _case(B, Hq, Hkv, T, D, fractions, residual, seed, permute=False):
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, seed)
    classes = synth.split_blocks(T - residual, fractions, seed)
    override = None
    if permute:  # arbitrary int64 positions, as the reference's kernel scripts feed (quant/cuda_hq_test.py:21-22)
        pos, kept = synth.survivor_positions(classes, T - residual)
        perm = torch.randperm(kept, generator=torch.Generator().manual_seed(seed))
        override, start = {}, 0
        for b, p in pos.items():
            override[b] = perm[start:start + p.numel()]
            start += p.numel()
    cache = synth.build_cache(K, V, classes, residual, O.uniform_group_quantize_pack_last_dim, override)
    return q, cache


CASES = [
    dict(B=1, Hq=8, Hkv=2, T=1024, D=128, fractions=(0.1, 0.2, 0.3, 0.3, 0.1), residual=0, seed=1),
    dict(B=2, Hq=8, Hkv=2, T=2048 + 17, D=128, fractions=(0.05, 0.15, 0.3, 0.3, 0.2), residual=17, seed=2),
    dict(B=1, Hq=32, Hkv=8, T=4096, D=128, fractions=(0.0, 0.0, 0.0, 1.0, 0.0), residual=128, seed=1235),  # config 1
    dict(B=1, Hq=4, Hkv=4, T=512 + 31, D=128, fractions=(0.25, 0.0, 0.5, 0.0, 0.25), residual=31, seed=4),
    dict(B=1, Hq=16, Hkv=2, T=1024, D=128, fractions=(0.0, 1.0, 0.0, 0.0, 0.0), residual=0, seed=5),
    dict(B=3, Hq=8, Hkv=1, T=640 + 5, D=128, fractions=(0.1, 0.2, 0.3, 0.3, 0.1), residual=5, seed=6),
    # with the uniform 1-bit class of the 'uniform_group' strategy (32 codes per word)
    dict(B=1, Hq=8, Hkv=2, T=2048 + 9, D=128, fractions=(0.05, 0.1, 0.2, 0.25, 0.3, 0.1), residual=9, seed=7),
    dict(B=2, Hq=4, Hkv=1, T=1024, D=128, fractions=(0.0, 0.0, 0.0, 0.0, 1.0, 0.0), residual=0, seed=8),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c['B']}Hq{c['Hq']}T{c['T']}D{c['D']}s{c['seed']}")
@pytest.mark.parametrize("permute", [False, True], ids=["blockidx", "randperm"])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "general"])
def test_hqe2_matches_oracle(dev, case, permute, fused, monkeypatch):
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    monkeypatch.setenv("HQEKV_UNFUSED", "0" if fused else "1")
    q, cache = _case(permute=permute, **case)
    w_ref, o_ref = O.qkv_matmul(q, cache, None, case["D"], use_mask=False)
    _, o_ref32 = O.qkv_matmul(q, cache, None, case["D"], use_mask=False, round_per_class=False)
    w, o = qkv_matmul_hqe_2(q.to(dev), synth.cache_to(cache, dev), None, case["D"], "uniform_group")
    assert w.shape == w_ref.shape and o.shape == o_ref.shape and w.dtype == torch.float16
    _close(w, w_ref, "attn_weights")
    _close(o, o_ref, "attn_output vs per-class fp16 accumulation")
    _close(o, o_ref32, "attn_output vs fp32 accumulation")
    # the probabilities of every (b, h) row sum to one
    torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(case["B"], case["Hq"], 1), rtol=0, atol=5e-3)


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "general"])
def test_low_normal_strategy_one_bit_class(dev, fused, monkeypatch):
    """'high_uniform_group_low_normal_group': the 1-bit class holds normal-quantile codes with (std, mean)."""
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    from hqekv_amd.quant_matmul_hq import qkv_matmul
    monkeypatch.setenv("HQEKV_UNFUSED", "0" if fused else "1")
    strategy = "high_uniform_group_low_normal_group"
    B, Hq, Hkv, T, D, residual = 1, 8, 2, 2048 + 11, 128, 11
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, 21)
    classes = synth.split_blocks(T - residual, (0.05, 0.1, 0.2, 0.25, 0.3, 0.1), 21)
    cache = synth.build_cache(K, V, classes, residual, lambda x, g, b: O.class_quantize(x, b, low_normal=True))
    w_ref, o_ref = O.qkv_matmul(q, cache, None, D, strategy, use_mask=False)
    w, o = qkv_matmul_hqe_2(q.to(dev), synth.cache_to(cache, dev), None, D, strategy)
    _close(w, w_ref, "attn_weights")
    _close(o, o_ref, "attn_output")
    # the same cache read as uniform 1-bit is a different function: the layouts are told apart
    w_u, _ = qkv_matmul_hqe_2(q.to(dev), synth.cache_to(cache, dev), None, D, "uniform_group")
    assert not torch.allclose(w_u.float().cpu(), w_ref.float(), rtol=RTOL, atol=ATOL)
    w2, o2 = qkv_matmul(q.to(dev), synth.cache_to(cache, dev), None, D, strategy)
    _close(w2, w_ref, "qkv_matmul attn_weights")
    _close(o2, o_ref, "qkv_matmul attn_output")


def test_qkv_matmul_with_mask(dev):
    from hqekv_amd.quant_matmul_hq import qkv_matmul, qkv_matmul_hq
    case = CASES[1]
    q, cache = _case(**case)
    Tall = cache[41]
    g = torch.Generator().manual_seed(3)
    mask = torch.zeros(case["B"], 1, 1, Tall, dtype=torch.float16)
    mask[..., torch.randperm(Tall, generator=g)[:Tall // 4]] = torch.finfo(torch.float16).min
    w_ref, o_ref = O.qkv_matmul(q, cache, mask, case["D"])
    for fn in (qkv_matmul, qkv_matmul_hq):
        w, o = fn(q.to(dev), synth.cache_to(cache, dev), mask.to(dev), case["D"], "uniform_group")
        _close(w, w_ref, "attn_weights")
        _close(o, o_ref, "attn_output")
        assert (w.cpu()[mask.expand_as(w_ref) < 0] == 0).all()
    w0, o0 = qkv_matmul(q.to(dev), synth.cache_to(cache, dev), 0, case["D"], "uniform_group")
    w_ref0, o_ref0 = O.qkv_matmul(q, cache, None, case["D"])
    _close(w0, w_ref0)
    _close(o0, o_ref0)


def test_fused_wrappers_match_oracle(dev):
    """cuda_bmm_forward_qk_group_hq / wv_group_hq with shuffled idx, the shape of quant/cuda_hq_test.py."""
    from hqekv_amd.matmul import cuda_bmm_forward_qk_group_hq, cuda_bmm_forward_wv_group_hq
    case = dict(B=1, Hq=32, Hkv=8, T=2048 + 95, D=128, fractions=(0.05, 0.0, 0.15, 0.8, 0.0), residual=95, seed=9)
    q, cache = _case(permute=True, **case)
    c = synth.cache_to(cache, dev)
    Tall = cache[41]
    scores = cuda_bmm_forward_qk_group_hq(32, 8, q.to(dev), c[0], c[1], c[4], c[5], c[6], c[7], c[12], c[13], c[14],
                                          c[15], c[20], c[21], c[22], c[23], None, None, None, None, c[39])
    # reference definition: dequantise everything, place by idx, matmul
    D = case["D"]
    dqK = torch.zeros(1, 8, Tall, D, dtype=torch.float16)
    dqK[:, :, cache[1]] = cache[0].transpose(2, 3)
    for b, base in ((4, 12), (2, 20)):
        dq = O.uniform_group_dequantize_unpack_last_dim(cache[base], cache[base + 2], cache[base + 3], 32, b)
        dqK[:, :, cache[base + 1]] = dq.transpose(2, 3)
    dqK[:, :, Tall - 95:] = cache[39]
    ref = torch.matmul(q.float(), O.repeat_kv(dqK, 4).transpose(2, 3).float())
    torch.testing.assert_close(scores.float().cpu(), ref, rtol=2e-3, atol=2e-2)  # raw scores are O(50)

    p = torch.softmax(torch.randn(1, 32, 1, Tall, generator=torch.Generator().manual_seed(1)) * 2, -1).half()
    out = cuda_bmm_forward_wv_group_hq(32, 8, p.to(dev), c[2], c[3], c[8], c[9], c[10], c[11], c[16], c[17], c[18],
                                       c[19], c[24], c[25], c[26], c[27], None, None, None, None, c[40])
    dqV = torch.zeros(1, 8, Tall, D, dtype=torch.float16)
    dqV[:, :, cache[3]] = cache[2]
    for b, base in ((4, 16), (2, 24)):
        dqV[:, :, cache[base + 1]] = O.uniform_group_dequantize_unpack_last_dim(
            cache[base], cache[base + 2], cache[base + 3], 32, b)
    dqV[:, :, Tall - 95:] = cache[40]
    ref = torch.matmul(p.float(), O.repeat_kv(dqV, 4).float())
    _close(out, ref, "attn_output")


def test_shape_of_the_reference_kernel_script(dev):
    """The one configuration the reference's own kernel script runs (quant/cuda_hq_test.py:340-355 with the
    class bounds of :27 and :296-304): B=1, 32 query heads over 8 KV heads, 8192 quantised tokens + 1023 new
    ones, inputs uniform in [0, 1), shuffled positions; fp16 [0,64), 4 bit [64,256), 2 bit [256,7168), 1 bit
    normal-quantile [7168,8192), no 8-bit class.  Its criterion is ours: dequantise with the library's own
    unpack, place by idx, matmul."""
    from hqekv_amd.matmul import cuda_bmm_forward_qk_group_hq, cuda_bmm_forward_wv_group_hq
    g = torch.Generator().manual_seed(77)
    quant_len, new_len, D = 8192, 1023, 128
    T = quant_len + new_len
    q = torch.rand(1, 32, 1, D, generator=g).half()
    k = torch.rand(1, 8, T, D, generator=g).half()
    v = torch.rand(1, 8, T, D, generator=g).half()
    idx = torch.randperm(quant_len, generator=g)
    bounds = [0, 64, 256, 7168, quant_len]          # fp16 | 4 bit | 2 bit | 1 bit
    sl = [slice(bounds[i], bounds[i + 1]) for i in range(4)]

    def classes(x, is_k):
        """-> per class (codes or fp16 data, scale/std, zero/mean) in the stored layout, and the dequantised rows"""
        out, dq = [], torch.zeros_like(x)
        for s_, bits in zip(sl, (16, 4, 2, 1)):
            part = x[:, :, s_, :].contiguous()
            src = part.transpose(2, 3).contiguous() if is_k else part
            if bits == 16:
                out.append((src, None, None))
                rows = part
            else:
                if bits == 1:
                    c, a, b = O.normal_group_quantize_pack_last_dim(src, 32, 1)
                    r = O.normal_group_dequantize_unpack_last_dim(c, a, b, 32, 1)
                else:
                    c, a, b = O.uniform_group_quantize_pack_last_dim(src, 32, bits)
                    r = O.uniform_group_dequantize_unpack_last_dim(c, a, b, 32, bits)
                out.append((c, a, b))
                rows = r.transpose(2, 3) if is_k else r
            dq[:, :, idx[s_], :] = rows
        dq[:, :, quant_len:, :] = x[:, :, quant_len:, :]
        return out, dq

    def to(x):
        return None if x is None else x.to(dev)

    (k16, k4, k2, k1), dq_k = classes(k, True)
    i16, i4, i2, i1 = (to(idx[s_]) for s_ in sl)
    scores = cuda_bmm_forward_qk_group_hq(
        32, 8, to(q), to(k16[0]), i16, None, None, None, None, to(k4[0]), i4, to(k4[1]), to(k4[2]),
        to(k2[0]), i2, to(k2[1]), to(k2[2]), to(k1[0]), i1, to(k1[1]), to(k1[2]), to(k[:, :, quant_len:, :].contiguous()))
    ref = torch.matmul(q.float(), O.repeat_kv(dq_k, 4).transpose(2, 3).float())
    assert scores.shape == (1, 32, 1, T)
    torch.testing.assert_close(scores.float().cpu(), ref, rtol=1e-3, atol=2e-2)   # raw scores are O(30)

    w = torch.softmax((ref / D ** 0.5), dim=-1).half()
    (v16, v4, v2, v1), dq_v = classes(v, False)
    out = cuda_bmm_forward_wv_group_hq(
        32, 8, to(w), to(v16[0]), i16, None, None, None, None, to(v4[0]), i4, to(v4[1]), to(v4[2]),
        to(v2[0]), i2, to(v2[1]), to(v2[2]), to(v1[0]), i1, to(v1[1]), to(v1[2]), to(v[:, :, quant_len:, :].contiguous()))
    _close(out, torch.matmul(w.float(), O.repeat_kv(dq_v, 4).float()), "attn_output")


def test_all_fp16_equals_dense_attention(dev):
    """Permutation invariance: with every class at fp16 and tokens shuffled between positions, the
    result must equal dense attention over the permuted sequence."""
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    q, K, V = synth.make_qkv(1, 8, 2, 512, 128, 77)
    perm = torch.randperm(480, generator=torch.Generator().manual_seed(5))
    t = [None] * 42
    t[0], t[1] = K[:, :, :480].transpose(2, 3).contiguous(), perm
    t[2], t[3] = V[:, :, :480].contiguous(), perm.clone()
    t[39], t[40], t[41] = K[:, :, 480:].contiguous(), V[:, :, 480:].contiguous(), 512
    w, o = qkv_matmul_hqe_2(q.to(dev), synth.cache_to(tuple(t), dev), None, 128, "uniform_group")
    Kp, Vp = K.clone(), V.clone()
    Kp[:, :, perm], Vp[:, :, perm] = K[:, :, :480], V[:, :, :480]
    s = torch.matmul(q.float(), O.repeat_kv(Kp, 4).transpose(2, 3).float()).half()
    s = (s.float() * (1.0 / 128 ** 0.5)).half()
    pr = torch.softmax(s.float(), -1).half()
    _close(w, pr)
    _close(o, torch.matmul(pr.float(), O.repeat_kv(Vp, 4).float()))


def test_unsupported_head_dim_is_an_error(dev):
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    q, K, V = synth.make_qkv(1, 4, 2, 64, 64, 3)
    cache = O.empty_cache(K, V, 64)
    with pytest.raises(ValueError, match="head_dim"):
        qkv_matmul_hqe_2(q.to(dev), synth.cache_to(cache, dev), None, 64, "uniform_group")


def test_errors(dev):
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    from hqekv_amd.quant_matmul_hq import qkv_matmul
    q = torch.zeros(1, 4, 1, 128, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError, match="invalid past_key_value"):
        qkv_matmul_hqe_2(q, (None,) * 41 + (0,), None, 128, "uniform_group")
    with pytest.raises(ValueError, match="invalid quant_strategy"):
        qkv_matmul_hqe_2(q, (None,) * 41 + (0,), None, 128, "bogus")
    with pytest.raises(ValueError, match="invalid quant_strategy"):
        qkv_matmul(q, (None,) * 41 + (0,), None, 128, "bogus")
    with pytest.raises(ValueError, match="invalid past_key_value"):
        qkv_matmul(q, (None,) * 41 + (0,), None, 128, "uniform_group")


def test_positions_that_are_no_partition_take_the_general_path(dev):
    """The softmax fused into the GEMV launches needs every position written exactly once.  A cache whose K
    positions name one position twice (and so leave another out) must not take that path: the call falls back
    to the separate softmax over a zero-initialised buffer, so every probability is finite and rows sum to one."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import DecodePlan, classes_partition_positions
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    case = CASES[0]
    q, cache = _case(**case)
    c = list(synth.cache_to(cache, dev))
    assert classes_partition_positions(tuple(c))
    bad = c[21].clone()
    bad[5] = bad[6]
    c[21] = bad
    assert not classes_partition_positions(tuple(c))
    w, o = qkv_matmul_hqe_2(q.to(dev), tuple(c), None, case["D"], "uniform_group")
    assert torch.isfinite(w.float()).all() and torch.isfinite(o.float()).all()
    torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(case["B"], case["Hq"], 1), rtol=0, atol=5e-3)
    plan = DecodePlan(q.to(dev), tuple(c), flags=_lib.FUSE_SOFTMAX)
    assert not (plan.flags & _lib.FUSE_SOFTMAX)
    w2, _ = plan.run(q.to(dev))
    torch.testing.assert_close(w2.float().sum(-1).cpu(), torch.ones(case["B"], case["Hq"], 1), rtol=0, atol=5e-3)
    # an in-place edit of a position array is noticed (the remembered verdict is tied to the tensor's version)
    good = list(synth.cache_to(cache, dev))
    assert classes_partition_positions(tuple(good))
    good[21][5] = good[21][6]
    assert not classes_partition_positions(tuple(good))


@pytest.mark.parametrize("Tall", [1, 7, 8, 1000, 8191, 8200, 26225, 70001, 140003])
@pytest.mark.parametrize("with_mask", [False, True])
def test_scale_softmax_rows(dev, Tall, with_mask):
    """The epilogue alone, through the C ABI, on aligned and odd row lengths (register-resident and
    generic kernels) against the oracle's fp16-scale / fp32-softmax chain."""
    from hqekv_amd import _lib
    g = torch.Generator().manual_seed(Tall)
    rows = 5
    s = (torch.randn(rows, Tall, generator=g) * 30).half()
    mask = None
    if with_mask:
        mask = torch.zeros(rows, Tall, dtype=torch.float16)
        mask[:, torch.randperm(Tall, generator=g)[:Tall // 3]] = torch.finfo(torch.float16).min
    ref = O._scale_clamp_softmax(s.view(1, rows, 1, Tall), 128, None if mask is None else mask.view(1, rows, 1, Tall),
                                 "recip").view(rows, Tall)
    sd = s.to(dev)
    md = mask.to(dev) if with_mask else None
    rc = _lib.load().hqekv_scale_softmax(sd.data_ptr(), None if md is None else md.data_ptr(), Tall, rows, Tall,
                                         1.0 / 128 ** 0.5, _lib.stream_ptr(dev))
    _lib.check(rc, "scale_softmax")
    torch.testing.assert_close(sd.float().cpu(), ref.float(), rtol=RTOL, atol=1e-5)


def test_fused_path_is_deterministic_and_reusable(dev):
    """Repeated calls on one plan (same workspace, uninitialised at first) give bit-identical results,
    and the fused path matches the general path within the tolerance."""
    from hqekv_amd.attention import DecodePlan
    q, cache = _case(**CASES[1])
    c = synth.cache_to(cache, dev)
    plan = DecodePlan(q.to(dev), c, flags=1)
    ref = DecodePlan(q.to(dev), c, flags=0)
    w0, o0 = [x.clone() for x in plan.run(q.to(dev))]
    for _ in range(5):
        w, o = plan.run(q.to(dev))
        assert torch.equal(w, w0) and torch.equal(o, o0)
    wr, orr = ref.run(q.to(dev))
    _close(w0, wr.cpu(), "fused vs general attn_weights")
    _close(o0, orr.cpu(), "fused vs general attn_output")


def test_segment_memo_gives_the_same_bits(dev):
    """A caller that keeps a SegmentMemo per layer (class entries built once, only the residual entry per
    step, workspace reused) gets bit-identical results to the memo-less call: while the residual grows
    token by token, after the classes are replaced by another cache, and for a cache without a residual."""
    from hqekv_amd.attention import SegmentMemo
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    memo = SegmentMemo()
    g = torch.Generator().manual_seed(11)
    for ci in (1, 6, 0):
        case = CASES[ci]
        q, cache = _case(**case)
        c = list(synth.cache_to(cache, dev))
        for step in range(4):
            if step:  # the caller appends one token to the residual; the class tensors stay the same objects
                nk = torch.randn(case["B"], case["Hkv"], 1, case["D"], generator=g).half().to(dev)
                nv = torch.randn(case["B"], case["Hkv"], 1, case["D"], generator=g).half().to(dev)
                c[39] = nk if c[39] is None else torch.cat((c[39], nk), 2)
                c[40] = nv if c[40] is None else torch.cat((c[40], nv), 2)
                c[41] = int(c[41]) + 1
            qd = torch.randn(case["B"], case["Hq"], 1, case["D"], generator=g).half().to(dev)
            w0, o0 = qkv_matmul_hqe_2(qd, tuple(c), None, case["D"], "uniform_group")
            w1, o1 = qkv_matmul_hqe_2(qd, tuple(c), None, case["D"], "uniform_group", memo=memo)
            assert torch.equal(w0, w1) and torch.equal(o0, o1), (ci, step)
            assert memo.lookup(tuple(c), torch.device(dev), True)


@pytest.mark.parametrize("ci", [0, 1, 6])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "general"])
def test_step_tokens_as_a_tail_segment(dev, ci, fused, monkeypatch):
    """A decode step may hand its new key / value rows over beside the tuple (``tail``) instead of appending them to
    the residual first.  Same probabilities bit for bit on the general path (every logit is computed alike and the
    softmax runs over the whole row), the oracle's result to tolerance on both paths, with and without a memo, for
    a cache with and without a residual."""
    from hqekv_amd.attention import SegmentMemo
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    if not fused:
        monkeypatch.setenv("HQEKV_UNFUSED", "1")
    case = CASES[ci]
    q, cache = _case(**case)
    g = torch.Generator().manual_seed(31 + ci)
    nk = torch.randn(case["B"], case["Hkv"], 1, case["D"], generator=g).half()
    nv = torch.randn(case["B"], case["Hkv"], 1, case["D"], generator=g).half()
    appended = list(cache)
    appended[39] = nk if cache[39] is None else torch.cat((cache[39], nk), 2)
    appended[40] = nv if cache[40] is None else torch.cat((cache[40], nv), 2)
    appended[41] = int(cache[41]) + 1
    w_ref, o_ref = O.qkv_matmul(q, tuple(appended), None, case["D"], use_mask=False, round_per_class=False)
    c, ca = synth.cache_to(cache, dev), synth.cache_to(tuple(appended), dev)
    w0, o0 = qkv_matmul_hqe_2(q.to(dev), ca, None, case["D"], "uniform_group")
    memo = SegmentMemo()
    for m in (None, memo, memo):
        w, o = qkv_matmul_hqe_2(q.to(dev), c, None, case["D"], "uniform_group", memo=m,
                                tail=(nk.to(dev), nv.to(dev)))
        assert w.shape == w0.shape
        if not fused:
            assert torch.equal(w, w0)
        _close(w, w_ref, "attn_weights")
        _close(o, o_ref, "attn_output")
        _close(o, o0.cpu(), "tail vs appended")


@pytest.mark.parametrize("case", [CASES[1], CASES[2], CASES[5], CASES[6]], ids=lambda c: f"B{c['B']}Hq{c['Hq']}T{c['T']}")
@pytest.mark.parametrize("fused", [1, 0], ids=["fused", "general"])
def test_folded_combine_equals_the_combine_launch(dev, case, fused):
    """The split-K partials are added up by the last p.V workgroup of each (b, kv head) (HQEKV_FOLD_COMBINE; the
    default for long launches) or by a launch of their own (HQEKV_SEPARATE_COMBINE): same order of additions, so
    the outputs are bit-identical -- on repeated calls over one workspace as well (the arrival counters are
    re-armed by every call)."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import DecodePlan
    q, cache = _case(**case)
    c = synth.cache_to(cache, dev)
    folded = DecodePlan(q.to(dev), c, flags=fused | _lib.FOLD_COMBINE)
    apart = DecodePlan(q.to(dev), c, flags=fused | _lib.SEPARATE_COMBINE)
    g = torch.Generator().manual_seed(5)
    for rep in range(4):
        qn = torch.randn(q.shape, generator=g).half().to(dev)
        w0, o0 = [x.clone() for x in folded.run(qn)]
        w1, o1 = [x.clone() for x in apart.run(qn)]
        assert torch.equal(w0, w1) and torch.equal(o0, o1), rep
    w_ref, o_ref = O.qkv_matmul(qn.cpu(), cache, None, case["D"], use_mask=False, round_per_class=False)
    _close(o0, o_ref, "attn_output")


@pytest.mark.parametrize("flags", [1, 0], ids=["fused", "general"])
def test_plan_replayed_from_a_hip_graph(dev, flags):
    """A captured decode step (no allocation, no memset inside) replayed several times with new queries,
    eager launches and synchronisations in between: every replay equals the eager result bit for bit."""
    from hqekv_amd.attention import DecodePlan
    q, cache = _case(**CASES[1])
    c = synth.cache_to(cache, dev)
    plan = DecodePlan(q.to(dev), c, flags=flags)
    eager = DecodePlan(q.to(dev), c, flags=flags)
    q_static = q.to(dev).clone()
    plan.run(q_static)                       # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.run(q_static)
    g = torch.Generator().manual_seed(99)
    for rep in range(4):
        q_new = torch.randn(q.shape, generator=g).half().to(dev)
        q_static.copy_(q_new)
        graph.replay()
        torch.cuda.synchronize()
        w_g, o_g = plan.weights.clone(), plan.out.clone()
        w_e, o_e = [x.clone() for x in eager.run(q_new)]   # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(w_g, w_e) and torch.equal(o_g, o_e), rep


def test_config2_full_size_against_oracle(dev):
    """Benchmark configuration 2 at its full size (B=1, 32 query heads, 8 KV heads, context 32768, hybrid split with
    20 % evicted): caches built by the HIP quantiser are bit-identical to the oracle's, attention within
    tolerance, and the probabilities of every head sum to one."""
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    from hqekv_amd.pack_unpack import uniform_group_quantize_pack_last_dim as hip_quant
    cfg = synth.CONFIGS["c2"]
    q, K, V = synth.make_qkv(cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["T"], cfg["D"], cfg["seed"])
    classes = synth.split_blocks(cfg["T"], cfg["fractions"], cfg["seed"])
    assert [classes[b].numel() for b in (16, 8, 4, 2, 0)] == [1632, 4928, 9824, 9824, 6560]
    cache_cpu = synth.build_cache(K, V, classes, 0, O.uniform_group_quantize_pack_last_dim)
    cache_gpu = synth.build_cache(K.to(dev), V.to(dev), classes, 0, hip_quant)
    for i, (a, b) in enumerate(zip(cache_cpu[:41], cache_gpu[:41])):
        if torch.is_tensor(a):
            assert torch.equal(a, b.cpu()), f"cache slot {i}"
    w_ref, o_ref = O.qkv_matmul(q, cache_cpu, None, 128, use_mask=False)
    w, o = qkv_matmul_hqe_2(q.to(dev), cache_gpu, None, 128, "uniform_group")
    assert w.shape == (1, 32, 1, 26208)
    _close(w, w_ref, "attn_weights")
    _close(o, o_ref, "attn_output")
    torch.testing.assert_close(w.float().sum(-1).cpu(), torch.ones(1, 32, 1), rtol=0, atol=5e-3)


def test_linearity_in_v_at_scale(dev):
    """Size-independent property: with q = 0 every probability is 1/T, so the output is the mean of the
    dequantised V rows -- checked against the HIP dequantiser at 16k tokens, batch 2."""
    from hqekv_amd.hqe_matmul import qkv_matmul_hqe_2
    from hqekv_amd import pack_unpack as P
    g = torch.Generator().manual_seed(8)
    B, Hkv, T, D = 2, 2, 16384, 128
    V = torch.randn(B, Hkv, T, D, generator=g).half().to(dev)
    K = torch.randn(B, Hkv, T, D, generator=g).half().to(dev)
    kc, ks, kz = P.uniform_group_quantize_pack_last_dim(K.transpose(2, 3), 32, 2)
    vc, vs, vz = P.uniform_group_quantize_pack_last_dim(V, 32, 4)
    idx = torch.arange(T, device=dev)
    t = [None] * 42
    t[20], t[21], t[22], t[23] = kc, idx, ks, kz
    t[16], t[17], t[18], t[19] = vc, idx.clone(), vs, vz
    t[41] = T
    q = torch.zeros(B, 8, 1, D, dtype=torch.float16, device=dev)
    w, o = qkv_matmul_hqe_2(q, tuple(t), None, D, "uniform_group")
    assert torch.allclose(w.float(), torch.full_like(w, 1.0 / T, dtype=torch.float32), rtol=2e-3, atol=0)
    dq = P.uniform_group_dequantize_unpack_last_dim(vc, vs, vz, 32, 4).float()
    expect = (dq * w[0, 0, 0, 0].float()).sum(2, keepdim=True)                     # (B,Hkv,1,D)
    expect = expect[:, :, None].expand(B, Hkv, 4, 1, D).reshape(B, 8, 1, D)
    torch.testing.assert_close(o.float(), expect, rtol=2e-3, atol=2e-3)


def _random_configurations(dev, n_cases, seed0, ratios, kv_heads, least):
    import random
    from hqekv_amd.attention import decode_attention
    checked = 0
    for case in range(seed0, seed0 + n_cases):
        rnd = random.Random(1000 + case)
        B = rnd.choice([1, 1, 2, 3])
        Hkv = rnd.choice(kv_heads)
        Hq = Hkv * rnd.choice(ratios)
        nblocks = rnd.choice([1, 2, 3, 8, 17, 40, 64, 100])
        residual = rnd.choice([0, 0, 1, 5, 31, 32, 97, 200])
        nfr = 6 if rnd.random() < 0.5 else 5
        raw = [rnd.random() ** 2 if rnd.random() < 0.7 else 0.0 for _ in range(nfr)]
        if sum(raw) == 0:
            raw[2] = 1.0
        fr = [x / sum(raw) for x in raw]
        if sum(fr[:-1]) == 0 and residual == 0:   # everything evicted and no residual: nothing to attend over
            fr = [0.0] * nfr
            fr[1] = 1.0
        T = nblocks * 32 + residual
        permute = rnd.random() < 0.4
        low_uniform = rnd.random() < 0.5
        use_mask = rnd.random() < 0.2
        flags = rnd.choice([None, None, 0])
        what = f"case {case}: B={B} Hq={Hq} Hkv={Hkv} T={T} residual={residual} shares={[round(f, 2) for f in fr]} " \
               f"shuffled={permute} low_uniform={low_uniform} mask={use_mask} flags={flags}"
        try:
            classes = synth.split_blocks(T - residual, fr, 7000 + case)
        except AssertionError:   # shares that do not round to whole blocks
            continue
        q, K, V = synth.make_qkv(B, Hq, Hkv, T, 128, 5000 + case)
        override = None
        if permute:
            pos, kept = synth.survivor_positions(classes, T - residual)
            perm = torch.randperm(kept, generator=torch.Generator().manual_seed(case))
            override, start = {}, 0
            for b, p_ in pos.items():
                override[b] = perm[start:start + p_.numel()]
                start += p_.numel()

        def quant(x, g, bits):
            if bits == 1 and not low_uniform:
                return O.normal_group_quantize_pack_last_dim(x, 32, 1)
            return O.uniform_group_quantize_pack_last_dim(x, 32, bits)

        cache = synth.build_cache(K, V, classes, residual, quant, override)
        Tall = cache[41]
        if Tall == 0:
            continue
        mask = None
        if use_mask:
            mask = torch.zeros(B, 1, 1, Tall, dtype=torch.float16)
            mask[..., : max(1, Tall // 3)] = torch.finfo(torch.float16).min
        strategy = "uniform_group" if low_uniform else "high_uniform_group_low_normal_group"
        w_ref, _ = O.qkv_matmul(q, cache, mask, 128, strategy, use_mask=True, round_per_class=False)
        w, o = decode_attention(q.to(dev), synth.cache_to(cache, dev), None if mask is None else mask.to(dev), Tall,
                                zero_init=True, flags=flags, low_uniform=low_uniform)
        w, o = w.cpu(), o.cpu()
        assert torch.isfinite(o).all(), what
        assert torch.allclose(w.float(), w_ref.float(), rtol=RTOL, atol=ATOL), what
        _, v_dense = O.reconstruct_cache(cache, strategy)
        o_stage = torch.matmul(w.float(), O.repeat_kv(v_dense, Hq // Hkv).float())
        assert torch.allclose(o.float(), o_stage, rtol=RTOL, atol=ATOL), what
        checked += 1
    assert checked >= least


def test_random_configurations(dev):
    """200 seeded random configurations: batch, GQA ratio 1..8, context 32..3500, class shares (with and
    without the 1-bit class, either 1-bit coding), residual lengths, shuffled positions, masks, fused and
    general path.  Probabilities against the oracle; the output against the oracle's p.V of the SAME
    probabilities (a raw score on an fp16 rounding boundary may round the other way in another summation
    order and move a peaked row by half a percent, which the first check tolerates and the second one
    would otherwise inherit)."""
    _random_configurations(dev, 200, 0, [1, 2, 4, 4, 8], [1, 2, 4, 8], 150)


def test_random_configurations_of_sliced_head_ratios(dev):
    """The same draw for the other head ratios up to 8 and for ratios that run as slices of at most eight heads (9, 12)."""
    _random_configurations(dev, 60, 5000, [3, 5, 6, 7, 9, 12], [1, 2, 4], 40)


@pytest.mark.parametrize("ratio", [3, 5, 6, 7, 12, 13])
@pytest.mark.parametrize("fused", [1, 0], ids=["fused", "general"])
@pytest.mark.parametrize("tiling", ["8waves", "wave512"])
def test_other_head_ratios(dev, ratio, fused, tiling):
    """Query heads per KV head other than 1, 2, 4, 8 (repeat_kv takes any ratio: model/public_func.py:127-135): 3, 5,
    6, 7 have kernels of their own, 12 and 13 run as slices of at most eight heads, one launch pair each: every head
    row against the oracle, with the matrix-core slice of four and without it, with and without an additive mask, and
    again over the same plan (slices share one workspace)."""
    from hqekv_amd import _lib
    from hqekv_amd.attention import DecodePlan, decode_attention
    B, Hkv, T, residual = 2, 2, 1024 + 37, 37
    q, cache = _case(B, ratio * Hkv, Hkv, T, 128, (0.1, 0.2, 0.3, 0.3, 0.1), residual, 300 + ratio)
    c = synth.cache_to(cache, dev)
    Tall = cache[41]
    w_ref, o_ref = O.qkv_matmul(q, cache, None, 128, use_mask=False, round_per_class=False)
    for dot in (0, _lib.DOT_VALU):
        plan = DecodePlan(q.to(dev), c, flags=fused | dot | _lib.qk_tiling(_lib.QK_TILINGS[tiling]))
        for rep in range(2):
            w, o = plan.run(q.to(dev))
            _close(w, w_ref, f"attn_weights dot={dot} rep={rep}")
            _close(o, o_ref, f"attn_output dot={dot} rep={rep}")
    mask = torch.zeros(B, 1, 1, Tall, dtype=torch.float16)
    mask[..., : Tall // 3] = torch.finfo(torch.float16).min
    wm_ref, om_ref = O.qkv_matmul(q, cache, mask, 128, use_mask=True, round_per_class=False)
    wm, om = decode_attention(q.to(dev), c, mask.to(dev), Tall, zero_init=True, flags=fused)
    _close(wm, wm_ref, "masked attn_weights")
    _close(om, om_ref, "masked attn_output")


@pytest.mark.parametrize("tiling", ["8waves", "4waves", "wave512", "wave256"])
@pytest.mark.parametrize("dot", ["mfma", "valu"])
def test_score_scaling_matches_torch_division_on_device(dev, tiling, dot):
    """``attn_weights /= math.sqrt(head_dim)`` (quant/quant_matmul_hq.py:100) pinned on the device: the scaled fp16
    logits the fused q.K^T launch stores must equal, bit for bit, the raw fp16 scores of the same launch (same tiling,
    same form of the dot products) followed by torch's own in-place division executed on the GPU, which multiplies by
    the fp32 reciprocal and rounds to fp16.  Data like configuration 2: hybrid classes, K outlier channels, logits of
    a hundred and more, where one fp16 place is 0.06."""
    import math
    from hqekv_amd import _lib
    from hqekv_amd.attention import DecodePlan
    B, Hq, Hkv, T, D = 2, 32, 8, 4096, 128
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, D, 4242)
    classes = synth.split_blocks(T, (0.05, 0.15, 0.30, 0.30, 0.20), 4242)
    cache = synth.cache_to(synth.build_cache(K, V, classes, 0, O.uniform_group_quantize_pack_last_dim), dev)
    form = _lib.DOT_MFMA if dot == "mfma" else _lib.DOT_VALU
    plan = DecodePlan(q.to(dev), cache, flags=_lib.FUSE_SOFTMAX | _lib.qk_tiling(_lib.QK_TILINGS[tiling]) | form)
    assert plan.flags & _lib.FUSE_SOFTMAX
    qd = q.to(dev).contiguous()
    plan.run(qd, only=_lib.ONLY_QK)
    scaled = plan.weights.clone()
    plan.run(qd, only=_lib.ONLY_RAW_QK)
    raw = plan.weights.clone()
    torch.cuda.synchronize()
    assert float(raw.float().abs().max()) > 100.0
    expect = raw.clone()
    expect /= math.sqrt(D)                                  # torch's own op, on the device
    assert torch.equal(scaled.view(torch.int16), expect.view(torch.int16))
    # and the rule itself on every fp16 bit pattern: x / sqrt(128) on the device == rnd16(x * fp32(1 / sqrt(128)))
    allx = torch.arange(0, 65536, dtype=torch.int32, device=dev).to(torch.int16).view(torch.float16)
    finite = torch.isfinite(allx)
    by_torch = allx.clone()
    by_torch /= math.sqrt(D)
    inv = torch.tensor(1.0, dtype=torch.float32, device=dev) / torch.tensor(float(D), dtype=torch.float32, device=dev).sqrt()
    by_rule = (allx.float() * inv).half()
    assert torch.equal(by_torch[finite].view(torch.int16), by_rule[finite].view(torch.int16))
