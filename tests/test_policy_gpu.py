"""The product cache policy (HIP quantise/dequantise kernels + host logic) against the oracle: every
field of the 42-tuple bit-identical after each of three compressions with demotion and eviction."""
import pytest
import torch

from oracle import hqe_oracle as O
from tests import policy_cases as PC

pytestmark = pytest.mark.gpu


def _same(a, b, what):
    if a is None or b is None:
        assert a is None and b is None, what
        return
    if torch.is_tensor(a):
        a = a.cpu()
        assert a.shape == b.shape and a.dtype == b.dtype, (what, a.shape, b.shape, a.dtype, b.dtype)
        if a.dtype == torch.float16:
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), what
        else:
            assert torch.equal(a, b), what
    else:
        assert a == b, what


@pytest.mark.parametrize("strategy", ["uniform_group", "high_uniform_group_low_normal_group"])
def test_hqe2_policy_bit_exact_over_three_compressions(dev, strategy):
    """Under the second strategy the 1-bit class is quantised with the normal-quantile rule (std, mean in the
    scale / zero slots); everything else is unchanged."""
    from hqekv_amd.hqe_2 import KV_cache_hqe_2
    from hqekv_amd.public_func import get_block_token_idx, last_attn_weights

    lw = last_attn_weights(20)
    lw.set_max_length(4096)
    ring0 = torch.rand(20, 4096, generator=torch.Generator().manual_seed(2)).half()
    lw.weights = ring0.to(dev).clone()
    ring = {"cpu": ring0.clone()}

    def prod(pkv, cl, hist, ks, kb, vb, imp):
        return KV_cache_hqe_2(pkv, cl, hist, ks, kb, vb, imp, strategy, lw)

    def orac(pkv, cl, hist, ks, kb, vb, imp):
        out, ring["cpu"] = O.compress_cache(pkv, cl, hist, ks, kb, vb, imp, weights_ring=ring["cpu"],
                                            quant_strategy=strategy)
        return out

    got, _, _ = PC.run(prod, to_dev=lambda x: x.to(dev),
                       rank_blocks=lambda bs, bn, imp: get_block_token_idx(bs, bn, imp.to(dev)).cpu())
    want, _, _ = PC.run(orac)
    for step, (g, w) in enumerate(zip(got, want)):
        for slot in range(42):
            _same(g[slot], w[slot], f"step {step} slot {slot}")
    _same(lw.weights, ring["cpu"], "ring of recent attention rows after eviction")


def test_compress_without_eviction_and_reconstruct(dev):
    from hqekv_amd.hybrid_quant import KV_cache_compress, KV_cache_compress_1, KV_cache_reconstruct
    g = torch.Generator().manual_seed(21)
    K = torch.randn(2, 2, 128 + 9, 128, generator=g).half()
    V = torch.randn(2, 2, 128 + 9, 128, generator=g).half()
    imp = torch.rand(128, generator=g)
    ks = O.get_block_token_idx(32, 4, imp)
    counts = torch.tensor([32, 32, 32, 32, 0], dtype=torch.int32)
    pkv = O.empty_cache(K, V, 137)
    want, _ = O.compress_cache(pkv, 128, 0, ks, counts, counts.clone(), imp)
    dpkv = tuple(x.to(dev) if torch.is_tensor(x) else x for x in pkv)
    got = KV_cache_compress(dpkv, 128, 0, ks.to(dev), counts, counts.clone(), imp.to(dev), "uniform_group")
    for slot in range(42):
        _same(got[slot], want[slot], f"slot {slot}")
    rng = O.calculate_token_range(V[:, :, :128], None)
    got1 = KV_cache_compress_1(dpkv, 128, 0, ks.to(dev), counts, counts.clone(), imp.to(dev), rng.to(dev), "uniform_group")
    for slot in range(42):
        _same(got1[slot], want[slot], f"compress_1 slot {slot}")
    rK, rV = KV_cache_reconstruct(got, "uniform_group")
    wK, wV = O.reconstruct_cache(want)
    _same(rK, wK, "reconstructed K")
    _same(rV, wV, "reconstructed V")
    # the fp16 class and the residual come back exactly
    assert torch.equal(rK[:, :, 128:].cpu(), K[:, :, 128:])
    assert torch.equal(rV[:, :, want[3]].cpu(), V[:, :, want[3]])


def test_policy_errors(dev):
    from hqekv_amd.hqe_2 import KV_cache_hqe_2
    K = torch.zeros(1, 1, 64, 128, dtype=torch.float16, device=dev)
    pkv = (None,) * 39 + (K, K.clone(), 64)
    imp = torch.rand(64, device=dev).half()
    ks = torch.arange(64, device=dev)
    six = torch.tensor([32, 0, 0, 32, 0, 0], dtype=torch.int32)
    with pytest.raises(ValueError, match="invalid quant_strategy"):
        KV_cache_hqe_2(pkv, 64, 0, ks, six, six, imp, "bogus")
    with pytest.raises(NotImplementedError):
        # the per-row / all-normal quantiser families are not part of this library
        KV_cache_hqe_2(pkv, 64, 0, ks, six, six, imp, "normal_group")
    with pytest.raises(ValueError):
        KV_cache_hqe_2(pkv, 48, 0, ks, six, six, imp, "uniform_group")
    with pytest.raises(ValueError):
        KV_cache_hqe_2((None,) * 41 + (0,), 64, 0, ks, six, six, imp, "uniform_group")


@pytest.mark.parametrize("strategy", ["uniform_group", "high_uniform_group_low_normal_group"])
def test_gather_engine_equals_step_engine(dev, strategy):
    """The one-launch-per-side gather (block-level plan on the host, hqekv_cache_migrate on the device) and the
    step-by-step engine (the reference's sequence of moves) leave bit-identical tuples behind after each of three
    compressions with demotions and evictions; the gather really ran (engine='gather' raises when it cannot)."""
    from hqekv_amd import cache_policy
    from hqekv_amd.public_func import get_block_token_idx

    def runner(engine):
        def f(pkv, cl, hist, ks, kb, vb, imp):
            return cache_policy.compress(pkv, cl, hist, ks, kb, vb, imp, strategy, n_targets=6, engine=engine)
        return PC.run(f, to_dev=lambda x: x.to(dev), rank_blocks=lambda bs, bn, imp: get_block_token_idx(bs, bn, imp.to(dev)))[0]

    fast, slow = runner("gather"), runner("steps")
    for step, (a, b) in enumerate(zip(fast, slow)):
        for slot in range(42):
            x, y = a[slot], b[slot]
            _same(x, None if y is None else (y.cpu() if torch.is_tensor(y) else y), f"step {step} slot {slot}")


def test_gather_engine_declines_selections_that_split_blocks(dev):
    """V selections need not be made of whole blocks at this interface (a caller may hand in any ranking): the
    gather engine then declines and the step-by-step engine does the compression; forcing the gather raises."""
    from hqekv_amd import cache_policy
    g = torch.Generator().manual_seed(31)
    K = torch.randn(1, 2, 128, 128, generator=g).half()
    V = torch.randn(1, 2, 128, 128, generator=g).half()
    imp = torch.rand(128, generator=g)
    ks = O.get_block_token_idx(32, 4, imp.clone())
    ragged = torch.cat((ks[1:], ks[:1]))            # the same tokens, cut one token off the block grid
    counts = torch.tensor([32, 32, 32, 32, 0], dtype=torch.int32)
    pkv = tuple(x.to(dev) if torch.is_tensor(x) else x for x in O.empty_cache(K, V, 128))
    with pytest.raises(ValueError, match="whole aligned"):
        cache_policy.compress(pkv, 128, 0, ragged.to(dev), counts, counts.clone(), imp.to(dev), "uniform_group",
                              n_targets=5, engine="gather")
    # the same call without forcing: the step-by-step engine takes it, bit-identical to the oracle
    got = cache_policy.compress(pkv, 128, 0, ragged.to(dev), counts, counts.clone(), imp.to(dev), "uniform_group", n_targets=5)
    want, _ = O.compress_cache(O.empty_cache(K, V, 128), 128, 0, ragged, counts, counts.clone(), imp)
    for slot in range(42):
        _same(got[slot], want[slot], f"slot {slot}")


@pytest.mark.parametrize("is_k", [True, False], ids=["K", "V"])
@pytest.mark.parametrize("low_normal", [False, True], ids=["uniform1", "normal1"])
@pytest.mark.parametrize("D", [128, 64, 256])
def test_cache_migrate_random_plans(dev, is_k, low_normal, D):
    """hqekv_cache_migrate through the C ABI on plans drawn at random: every (source class, destination class)
    pair with destination bits <= source bits, sources in any order, more blocks than one workgroup's 16 (K side),
    a last workgroup that is not full, new tokens read from the head of a longer token-major tensor.  Expected
    bytes from the oracle: a block that keeps its width is copied, any other is dequantised (two roundings) and
    quantised again; the position arrays are the plan's block numbers expanded to tokens."""
    from hqekv_amd import _lib
    B, H = 2, 2
    bits_of = (16, 8, 4, 2, 1)
    g = torch.Generator().manual_seed(5 + (2 if is_k else 0) + (1 if low_normal else 0) + D)
    def rnd(*s):   # (B, H, tokens, D) values with a few groups whose minimum is a zero of either sign
        x = torch.randn(*s, generator=g).half()
        x[..., :8] = x[..., :8].abs()                       # K groups (32 tokens of a channel) of channels 0-7 ...
        x[:, :, 3::32, :8] = 0.0                            # ... hold +0 first,
        x[:, :, 9::32, :8] = -0.0                           # then -0
        x[:, :, 5::32, :32] = x[:, :, 5::32, :32].abs()     # V groups (32 channels of a token): -0 first
        x[:, :, 5::32, 2] = -0.0
        x[:, :, 5::32, 6] = 0.0
        return x
    n_src = [int(x) for x in torch.randint(6, 20, (5,), generator=g)] + [9]     # blocks per source; last: new tokens
    tail = 7                                                                      # residual tokens behind the new ones
    quant = lambda x, b: (O.normal_group_quantize_pack_last_dim(x, 32, 1) if (b == 1 and low_normal)
                          else O.uniform_group_quantize_pack_last_dim(x, 32, b))
    dequant = lambda c, s, z, b: (O.normal_group_dequantize_unpack_last_dim(c, s, z, 32, 1) if (b == 1 and low_normal)
                                  else O.uniform_group_dequantize_unpack_last_dim(c, s, z, 32, b))
    grp = (lambda x: x.transpose(2, 3).contiguous()) if is_k else (lambda x: x)   # groups along the last dim
    ungrp = grp if is_k else (lambda x: x)
    # sources as token-major fp16 values (B,H,n,D) and as stored
    src_vals, src_store = [], []
    for si, b in enumerate(bits_of):
        x = rnd(B, H, n_src[si] * 32, D)
        if b == 16:
            src_vals.append(x)
            src_store.append((grp(x), None, None))
        else:
            c, s, z = quant(grp(x), b)
            src_vals.append(ungrp(dequant(c, s, z, b)))
            src_store.append((c, s, z))
    new_full = rnd(B, H, n_src[5] * 32 + tail, D)
    src_vals.append(new_full[:, :, :n_src[5] * 32])
    # plan: every source block goes somewhere it may go (or nowhere: evicted), in random order
    cand = [(si, j) for si in range(6) for j in range(n_src[si])]
    perm = torch.randperm(len(cand), generator=g).tolist()
    dest_blocks = {di: [] for di in range(5)}
    for p in perm:
        si, j = cand[p]
        lo = 0 if si == 5 else si                       # new tokens may go anywhere, a class only down or stay
        di = int(torch.randint(lo, 6, (1,), generator=g))
        if di < 5:
            dest_blocks[di].append((si, j))
    total = sum(len(v) for v in dest_blocks.values())
    assert total > 16   # more than one workgroup on the K side
    pos = torch.randperm(total, generator=g).tolist()   # new block numbers, any bijection
    # expected stores
    want, plan_src, plan_pos, u = {}, [], [], 0
    for di, b in enumerate(bits_of):
        blocks = dest_blocks[di]
        if not blocks:
            continue
        vals = torch.cat([src_vals[si][:, :, 32 * j:32 * j + 32] for si, j in blocks], dim=2)
        if b == 16:
            c, s, z = grp(vals), None, None
        else:
            c, s, z = quant(grp(vals), b)
            c, s, z = c.clone(), s.clone(), z.clone()
            pf = 32 // b
            for k, (si, j) in enumerate(blocks):        # same width: the stored bytes move
                if si < 5 and bits_of[si] == b:
                    sc, ss, sz = src_store[si]
                    if is_k:
                        c[..., k * 32 // pf:(k + 1) * 32 // pf] = sc[..., j * 32 // pf:(j + 1) * 32 // pf]
                        s[..., k], z[..., k] = ss[..., j], sz[..., j]
                    else:
                        c[:, :, 32 * k:32 * k + 32] = sc[:, :, 32 * j:32 * j + 32]
                        s[:, :, 32 * k:32 * k + 32], z[:, :, 32 * k:32 * k + 32] = ss[:, :, 32 * j:32 * j + 32], sz[:, :, 32 * j:32 * j + 32]
        idx = torch.cat([torch.arange(32) + 32 * pos[u + k] for k in range(len(blocks))]).to(torch.int64)
        want[b] = (c, s, z, idx)
        plan_src += [(si << 24) | j for si, j in blocks]
        plan_pos += pos[u:u + len(blocks)]
        u += len(blocks)
    # device side
    keep = []
    def up(t):
        t = t.to(dev).contiguous()
        keep.append(t)
        return t
    src = (_lib.CacheClass * 6)()
    for si, b in enumerate(bits_of):
        c, s, z = src_store[si]
        e = src[si]
        e.bits, e.n_tokens, e.data = b, n_src[si] * 32, up(c).data_ptr()
        if b != 16:
            e.scale, e.zero = up(s).data_ptr(), up(z).data_ptr()
            e.layout = _lib.LAYOUT_NORMAL1 if (b == 1 and low_normal) else 0
    newd = up(new_full)
    e = src[5]
    e.bits, e.n_tokens, e.slab_tokens, e.data = 16, n_src[5] * 32, new_full.shape[2], newd.data_ptr()
    e.layout = _lib.LAYOUT_TOKEN_MAJOR if is_k else 0
    dst = (_lib.CacheClass * 5)()
    got, n_dst = {}, 0
    for di, b in enumerate(bits_of):
        if b not in want:
            continue
        c, s, z, idx = want[b]
        oc = torch.empty_like(c, device=dev)
        oi = torch.empty_like(idx, device=dev)
        d = dst[n_dst]
        n_dst += 1
        d.bits, d.n_tokens, d.data, d.idx = b, idx.numel(), oc.data_ptr(), oi.data_ptr()
        os_ = oz = None
        if b != 16:
            os_, oz = torch.empty_like(s, device=dev), torch.empty_like(z, device=dev)
            d.scale, d.zero = os_.data_ptr(), oz.data_ptr()
            d.layout = _lib.LAYOUT_NORMAL1 if (b == 1 and low_normal) else 0
        got[b] = (oc, os_, oz, oi)
    plan = torch.tensor(plan_src + plan_pos, dtype=torch.int32).to(dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    rc = _lib.load().hqekv_cache_migrate(1 if is_k else 0, src, 6, dst, n_dst, plan.data_ptr(), B * H, D,
                                         status.data_ptr(), _lib.stream_ptr(torch.device(dev)))
    _lib.check(rc, "cache_migrate")
    torch.cuda.synchronize()
    assert int(status) == 0
    for b in want:
        for name, a, w in zip(("code", "scale", "zero", "idx"), got[b], want[b]):
            _same(a, w, f"{b}-bit class {name}")
    # A plan that is wrong in every way the kernel can be told: a slot past the table, an empty slot, a block past
    # the end of its class, a position outside the new sequence.  Those entries are refused -- their destination
    # blocks keep the sentinel, the status word is set -- and every other entry is served as before.
    n_all = len(plan_src)
    bad_src, bad_pos = list(plan_src), list(plan_pos)
    victims = [0, n_all // 3, n_all // 2, n_all - 1]
    bad_src[victims[0]] = (7 << 24) | 0                       # slot 7 of a table of 7 entries (6 populated + 1 empty)
    bad_src[victims[1]] = (6 << 24) | 0                       # the empty slot
    bad_src[victims[2]] = (1 << 24) | (n_src[1] + 3)          # past the end of the 8-bit class
    bad_pos[victims[3]] = n_all + 5                           # position outside the new sequence
    src7 = (_lib.CacheClass * 7)()
    for i in range(6):
        C_ = src[i]
        for f, _t in _lib.CacheClass._fields_:
            setattr(src7[i], f, getattr(C_, f))
    sent_i, sent_h = -1234567, -3.0
    for b in got:
        oc, os_, oz, oi = got[b]
        oc.fill_(sent_i if oc.dtype == torch.int32 else sent_h)
        oi.fill_(-7)
        if os_ is not None:
            os_.fill_(sent_h)
            oz.fill_(sent_h)
    plan_bad = torch.tensor(bad_src + bad_pos, dtype=torch.int32).to(dev)
    rc = _lib.load().hqekv_cache_migrate(1 if is_k else 0, src7, 7, dst, n_dst, plan_bad.data_ptr(), B * H, D,
                                         status.data_ptr(), _lib.stream_ptr(torch.device(dev)))
    _lib.check(rc, "cache_migrate")
    torch.cuda.synchronize()
    assert int(status) != 0
    u = 0
    for b in bits_of:
        if b not in want:
            continue
        oi, wi = got[b][3].cpu(), want[b][3]
        for k in range(wi.numel() // 32):
            sl = slice(32 * k, 32 * k + 32)
            if u + k in victims:
                assert bool((oi[sl] == -7).all()), f"{b}-bit class: refused block {k} was written"
            else:
                assert torch.equal(oi[sl], wi[sl]), f"{b}-bit class: block {k} of a plan with refused entries"
        u += wi.numel() // 32
