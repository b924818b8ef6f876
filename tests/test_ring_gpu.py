"""The importance ring's decode row on the device (hqekv_ring_row, and the same code inside hqekv_decode_step) against
torch's own ``attn_weights.sum(0).sum(0)`` executed on the GPU, bit for bit -- the row's last place decides block
rankings (model/public_func.py:92-106, 243-257), so the kernels follow the order in which torch's reduction adds the
rows.  Shapes: 32 heads, batch 1..8, rows from 256 tokens up, every residue of the length modulo 4, aligned and
unaligned slots of the ring store."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _order_sensitive(B, H, T, g):
    """Small values everywhere plus, in every column, big values that cancel exactly in pairs: what is left depends on
    which small values met a big partial sum before its partner arrived -- any other order of additions shows."""
    m = torch.randint(1024, 2048, (B * H, T), generator=g).float() / 1024.0
    e = torch.randint(8, 15, (B * H, T), generator=g).float()
    X = m * torch.exp2(-e)
    order = torch.rand(B * H, T, generator=g).argsort(0)
    cols = torch.arange(T)
    for k in range(max(1, B * H // 8)):
        big = (torch.randint(1024, 2048, (T,), generator=g).float() / 1024.0) * 1024.0
        X[order[2 * k], cols] = big
        X[order[2 * k + 1], cols] = -big
    return X.half().view(B, H, 1, T)


def _probabilities(B, H, T, g):
    return torch.softmax(torch.randn(B, H, 1, T, generator=g) * 4.0, dim=-1).half()


@pytest.mark.parametrize("B", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("kind", ["order_sensitive", "probabilities"])
def test_ring_row_equals_torch_sum_on_device(dev, B, kind):
    from hqekv_amd import _lib
    from hqekv_amd.attention import ring_order, ring_row_on_device_applies
    H = 32
    g = torch.Generator().manual_seed(100 * B + len(kind))
    lib = _lib.load()
    for T in (256, 257, 258, 259, 260, 1000, 1023, 4096, 4099, 8200, 26208, 26209, 26210, 26211, 52449, 104864):
        w = (_order_sensitive if kind == "order_sensitive" else _probabilities)(B, H, T, g).to(dev)
        assert ring_row_on_device_applies(w)
        expect = w.sum(0).sum(0).reshape(T)                       # torch's own reductions, on the device
        for max_len, row in ((T + 8, 0), (T + 9, 1), (T + 10, 3), (T + 11, 7)):   # slots of every alignment
            store = torch.full((20, max_len), -5.0, dtype=torch.float16, device=dev)
            line = store[row, :T]
            rc = lib.hqekv_ring_row(w.data_ptr(), B, H, T, line.data_ptr(), ring_order(T, w), _lib.stream_ptr(dev))
            _lib.check(rc, "ring_row")
            torch.cuda.synchronize()
            assert torch.equal(line.view(torch.int16), expect.view(torch.int16)), (B, T, max_len, row)
            assert bool((store[row, T:] == -5.0).all()) and bool((store[row - 1] == -5.0).all())   # nothing else written
    # the class that keeps the ring takes this route for such rows, and torch's for the others
    from hqekv_amd.public_func import last_attn_weights
    ring = last_attn_weights()
    ring.set_max_length(5000)
    for T in (100, 255, 256, 4099):
        w = _probabilities(B, H, T, g).to(dev)
        slot = ring.next_line
        ring.update(w)
        assert torch.equal(ring.weights[slot, :T].view(torch.int16), w.sum(0).sum(0).reshape(T).view(torch.int16)), T


def _row_sum_in_kernel_order(rows, by):
    """The documented order on the host in float32: the rows are dealt round-robin to ``by`` walkers, a walker adds its
    k-th row to accumulator k mod 4 and closes with ((a0 + a1) + a2) + a3, two walkers are added at the end."""
    parts = []
    for y in range(by):
        acc = [torch.zeros(rows.shape[1], dtype=torch.float32) for _ in range(4)]
        for k, r in enumerate(range(y, rows.shape[0], by)):
            acc[k % 4] = acc[k % 4] + rows[r].float()
        parts.append(((acc[0] + acc[1]) + acc[2]) + acc[3])
    return parts[0] if by == 1 else parts[0] + parts[1]


@pytest.mark.parametrize("B,H,T", [(9, 32, 300), (2, 80, 300), (2, 32, 3), (1, 32, 2), (3, 7, 1031)])
@pytest.mark.parametrize("by", [1, 2])
def test_ring_row_shapes_outside_the_tiled_path(dev, B, H, T, by):
    """More than 8 batch rows, more than 64 heads, rows shorter than one 4-column load: the kernel walks such columns
    one load at a time.  torch's order is not pinned for these shapes, so the check is the documented order itself."""
    from hqekv_amd import _lib
    g = torch.Generator().manual_seed(B * 1000 + H + T)
    w = _order_sensitive(B, H, T, g)
    per_head = w[0, :, 0] if B == 1 else torch.stack([_row_sum_in_kernel_order(w[:, h, 0], 1).half() for h in range(H)])
    expect = _row_sum_in_kernel_order(per_head, by).half()
    line = torch.full((T + 3,), -5.0, dtype=torch.float16, device=dev)
    wd = w.to(dev)
    _lib.check(_lib.load().hqekv_ring_row(wd.data_ptr(), B, H, T, line.data_ptr(), by, _lib.stream_ptr(dev)), "ring_row")
    torch.cuda.synchronize()
    assert torch.equal(line[:T].cpu().view(torch.int16), expect.view(torch.int16))
    assert bool((line[T:] == -5.0).all())


def test_ring_row_rejects_bad_arguments(dev):
    from hqekv_amd import _lib
    lib = _lib.load()
    w = torch.zeros(1, 32, 1, 256, dtype=torch.float16, device=dev)
    line = torch.zeros(256, dtype=torch.float16, device=dev)
    assert lib.hqekv_ring_row(w.data_ptr(), 1, 32, 256, line.data_ptr(), 3, None) == -1
    assert lib.hqekv_ring_row(None, 1, 32, 256, line.data_ptr(), 1, None) == -1
    assert lib.hqekv_ring_row(w.data_ptr(), 1, 32, 0, line.data_ptr(), 1, None) == -1


@pytest.mark.parametrize("B,T0", [(1, 300), (2, 257), (4, 512)])
def test_layer_step_in_one_call_equals_the_separate_launches(dev, B, T0):
    """Two layers in lockstep over a prompt and 70 decode steps (two compressions): one runs a decode step as ONE call
    (attention + ring row + residual appends, hqekv_decode_step), the other as the reference's sequence of separate
    operations.  Every field of the cache tuples, the ring stores, the probabilities and the outputs are identical
    bit for bit, and each ring row equals torch's own attn_weights.sum(0).sum(0) on the device."""
    from hqekv_amd.decode_layer import HqeAttentionLayer
    Hq, Hkv, D, steps = 32, 8, 128, 70
    ratios = dict(bit_0=0.2, bit_4=0.3, bit_2=0.5, bit_1=0.0)
    one, sep = HqeAttentionLayer(D, **ratios), HqeAttentionLayer(D, **ratios)
    sep.fused_step = False
    for l in (one, sep):
        l.set_max_length(T0 + steps)
    g = torch.Generator().manual_seed(7 + B)
    pkv1 = pkv2 = None
    compressions = 0
    for step in range(steps + 1):
        L = T0 if step == 0 else 1
        q = torch.randn(B, Hq, L, D, generator=g).half().to(dev)
        k = torch.randn(B, Hkv, L, D, generator=g).half().to(dev)
        v = torch.randn(B, Hkv, L, D, generator=g).half().to(dev)
        mask = None
        if step == 0:
            mask = torch.triu(torch.full((T0, T0), torch.finfo(torch.float16).min, dtype=torch.float16), diagonal=1)[None, None].to(dev)
        slot = one.last_weights.next_line
        o1, w1, pkv1, aux1 = one(q, k, v, mask, pkv1, None)
        o2, w2, pkv2, aux2 = sep(q, k, v, mask, pkv2, None)
        where = f"step {step}"
        assert torch.equal(w1, w2) and torch.equal(o1, o2), where
        if step and aux1 is None:   # (a compression moves the ring's columns afterwards)
            T = w1.shape[-1]
            assert torch.equal(one.last_weights.weights[slot, :T].view(torch.int16),
                               w1.sum(0).sum(0).reshape(T).view(torch.int16)), where
        assert torch.equal(one.last_weights.weights.view(torch.int16), sep.last_weights.weights.view(torch.int16)), where
        assert (aux1 is None) == (aux2 is None), where
        compressions += aux1 is not None
        for i, (a, b) in enumerate(zip(pkv1, pkv2)):
            if torch.is_tensor(a):
                assert a.shape == b.shape and torch.equal(a, b), (where, i)
            else:
                assert a == b, (where, i)
    assert compressions >= 2


# ------------------------------------------------------------------ what the policy ranks blocks by
def _ring_with_cancelling_columns(n, max_len, g, dev):
    """A 20-row ring store whose column sums are small everywhere except for pairs of columns inside every block of 32
    that hold +big and -big: the block sums then depend on the order the 32 values are added in, the column sums (big
    values that cancel between rows, as in ``_order_sensitive``) on the order of the rows."""
    X = _order_sensitive(1, 20, n, g)[0, :, 0].float()          # (20, n)
    for b0 in range(0, n - 31, 32):
        i, j = (torch.randperm(32, generator=g)[:2] + b0).tolist()
        big = float(torch.randint(1024, 2048, (1,), generator=g)) / 8.0
        X[:, i] = 0
        X[:, j] = 0
        X[3, i], X[3, j] = big, -big
    store = torch.zeros(20, max_len, dtype=torch.float16, device=dev)
    store[:, :n] = X.half().to(dev)
    return store


@pytest.mark.parametrize("max_len,n", [(600, 33), (600, 64), (4099, 320), (4099, 4064 + 5), (32968, 26240),
                                       (32968, 26208 + 19), (131500, 104864)])
def test_importance_and_block_scores_equal_torch_chain_on_device(dev, max_len, n):
    """``ranked_importance`` / ``rank_blocks_weighted`` (one launch each) against the chain of torch operations they
    stand for -- sum over the ring's rows, divide by the counts, copy, divide by 32 in place, sum the blocks; multiply
    with the V ranges, divide, sum -- executed by torch on the device: importance, scores and order bit for bit."""
    from hqekv_amd.public_func import get_block_importance, last_attn_weights, rank_blocks_weighted
    g = torch.Generator().manual_seed(n)
    total, nb = n // 32 * 32, n // 32
    ring = last_attn_weights()
    ring.set_max_length(max_len)
    ring.weights = _ring_with_cancelling_columns(n, max_len, g, dev)
    ring.kv_seq_len = n
    imp_t = ring.calculate_token_importance()[:total].clone()
    sc_t = get_block_importance(32, nb, imp_t)                    # divides imp_t in place, like the reference's helper
    imp_k, ranked = ring.ranked_importance(total)
    torch.cuda.synchronize()
    assert torch.equal(imp_k.view(torch.int16), imp_t.view(torch.int16))
    assert torch.equal(ranked.scores.view(torch.int16), sc_t.view(torch.int16))
    assert torch.equal(ranked.order, torch.sort(sc_t, descending=True, stable=True)[1])
    # the V side: importance (already divided) times the token ranges, divided again, summed per block
    vn = (torch.rand(total, generator=g) * 40 + 0.01).half().to(dev)
    for w in (vn, None):
        v_t = imp_t * w if w is not None else imp_t.clone()
        sv_t = get_block_importance(32, nb, v_t)
        kept = imp_k.clone()
        rw = rank_blocks_weighted(nb, imp_k, w)
        torch.cuda.synchronize()
        assert torch.equal(rw.scores.view(torch.int16), sv_t.view(torch.int16))
        assert torch.equal(imp_k, kept) and (w is None or torch.equal(w, vn))      # arguments untouched


@pytest.mark.parametrize("B,H,T,cap", [(1, 8, 32, 0), (2, 8, 32, 96), (3, 4, 64, 0), (4, 8, 300, 0), (8, 8, 33, 64),
                                       (1, 2, 32, 0), (5, 3, 1, 0), (2, 8, 4099, 0)])
def test_token_range_equals_torch_chain_on_device(dev, B, H, T, cap):
    """``hqekv_token_range`` against (max - min over channels).sum(0).sum(0) executed by torch on the device, bit for
    bit: random tokens, and tokens whose ranges span 25 binades so that fp32 sums lose low bits in an order-dependent
    way; dense tensors and heads of capacity buffers."""
    from hqekv_amd.public_func import calculate_new_token_range
    g = torch.Generator().manual_seed(B * 100 + H * 10 + T)
    D = 128
    for kind in ("random", "wide"):
        x = torch.randn(B, H, T, D, generator=g)
        if kind == "wide":
            x = torch.zeros(B, H, T, D)
            x[..., 5] = torch.exp2(torch.randint(-10, 16, (B, H, T), generator=g).float()) * \
                (torch.randint(1024, 2048, (B, H, T), generator=g).float() / 1024.0)
        x = x.half()
        if cap:
            buf = torch.zeros(B, H, cap + T, D, dtype=torch.float16, device=dev)
            buf[:, :, :T] = x.to(dev)
            xd = buf[:, :, :T]
        else:
            xd = x.to(dev)
        expect = (torch.max(xd, dim=-1)[0] - torch.min(xd, dim=-1)[0]).sum(0).sum(0)
        got = calculate_new_token_range(xd)
        torch.cuda.synchronize()
        assert got.shape == expect.shape and got.dtype == expect.dtype
        assert torch.equal(got.view(torch.int16), expect.view(torch.int16)), (kind, B, H, T)


def test_policy_score_entries_reject_bad_arguments(dev):
    from hqekv_amd import _lib
    lib = _lib.load()
    a = torch.zeros(20, 64, dtype=torch.float16, device=dev)
    o = torch.zeros(64, dtype=torch.float16, device=dev)
    assert lib.hqekv_importance_scores(a.data_ptr(), 20, 64, 64, 48, o.data_ptr(), o.data_ptr(), None) == -1   # not whole blocks
    assert lib.hqekv_importance_scores(a.data_ptr(), 20, 64, 32, 64, o.data_ptr(), o.data_ptr(), None) == -1   # total > n
    assert lib.hqekv_importance_scores(None, 20, 64, 64, 64, o.data_ptr(), o.data_ptr(), None) == -1
    assert lib.hqekv_weighted_block_scores(o.data_ptr(), None, 33, o.data_ptr(), None) == -1
    assert lib.hqekv_token_range(a.data_ptr(), 1, 1, 8, 128, 4, o.data_ptr(), None) == -1                      # slab < T
    assert lib.hqekv_token_range(a.data_ptr(), 40, 40, 8, 128, 8, o.data_ptr(), None) == -4                    # B * H > 1024


@pytest.mark.parametrize("B,Hq,Hkv,T", [(1, 32, 8, 2048 + 9), (4, 32, 8, 1024 + 3)])
def test_step_extras_with_either_combine_route_and_dot_form(dev, B, Hq, Hkv, T):
    """``hqekv_decode_step``'s ring row and appends ride in the combine launch -- or, when the combine is folded into
    the p.V launch, in a launch of their own: both routes (forced by flag), with the dot products on the matrix cores
    and on the vector ALU, give the ring row torch computes from the probabilities and the appended rows, and the
    attention itself is the same bits as without the extras."""
    from hqekv_amd import _lib, synth
    from hqekv_amd.attention import decode_attention, value_length
    from oracle import hqe_oracle as O
    q, K, V = synth.make_qkv(B, Hq, Hkv, T, 128, 77 + B)
    res = T % 32
    classes = synth.split_blocks(T - res, (0.05, 0.15, 0.30, 0.30, 0.20), 5 + B)
    cache = synth.cache_to(synth.build_cache(K, V, classes, res, O.uniform_group_quantize_pack_last_dim), dev)
    Tall = value_length(cache) + 1                      # the step's own token rides as a tail segment
    g = torch.Generator().manual_seed(3)
    k_new = torch.randn(B, Hkv, 1, 128, generator=g).half().to(dev)
    v_new = torch.randn(B, Hkv, 1, 128, generator=g).half().to(dev)
    qd = q.to(dev)
    for route in (_lib.SEPARATE_COMBINE, _lib.FOLD_COMBINE):
        for dot in (_lib.DOT_MFMA, _lib.DOT_VALU):
            flags = _lib.FUSE_SOFTMAX | route | dot
            w0, o0 = decode_attention(qd, cache, None, Tall, zero_init=False, flags=flags, tail=(k_new, v_new))
            kbuf = torch.zeros(B, Hkv, 64, 128, dtype=torch.float16, device=dev)
            vbuf = torch.zeros_like(kbuf)
            line = torch.full((Tall + 5,), -3.0, dtype=torch.float16, device=dev)
            w1, o1 = decode_attention(qd, cache, None, Tall, zero_init=False, flags=flags, tail=(k_new, v_new),
                                      step=dict(ring_line=line[1:Tall + 1], append=(kbuf, vbuf, 7)))
            torch.cuda.synchronize()
            where = (route, dot)
            assert torch.equal(w0, w1) and torch.equal(o0, o1), where
            assert torch.equal(line[1:Tall + 1].view(torch.int16), w1.sum(0).sum(0).reshape(Tall).view(torch.int16)), where
            assert float(line[0]) == -3.0 and bool((line[Tall + 1:] == -3.0).all()), where
            assert torch.equal(kbuf[:, :, 7], k_new[:, :, 0]) and torch.equal(vbuf[:, :, 7], v_new[:, :, 0]), where
            kbuf[:, :, 7] = 0
            vbuf[:, :, 7] = 0
            assert not bool(kbuf.any()) and not bool(vbuf.any()), where   # nothing else written
