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
