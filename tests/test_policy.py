"""The cache-policy oracle against an independent per-block history model (CPU only).

The model knows nothing about tensors of classes: it tracks, for every original 32-token block, the
sequence of precisions it went through and whether it survived, using only the published rules
(targets served low to high, demotion only, whole blocks, survivors re-ranked).  The dense cache the
oracle's tuple reconstructs to must equal the original data pushed through that chain of fake
quantisations, at the position the model predicts."""
import torch

from oracle import hqe_oracle as O
from tests import policy_cases as PC


def _oracle_compress(pkv, cl, hist, ks, kb, vb, imp):
    return O.compress_cache(pkv, cl, hist, ks, kb, vb, imp)[0]


def _model(log, K, V):
    """-> per side, the ordered list of (original block id, [precision chain]) of the survivors."""
    sides = {}
    for side in ("K", "V"):
        order = []      # surviving original blocks in position order: (block id, chain)
        n_seen = 0
        for st in log:
            n_new_blocks = st["compress_length"] // 32
            order = order + [(n_seen + j, None) for j in range(n_new_blocks)]   # chain None = still new
            total_blocks = len(order)
            imp = st["importance"]
            if side == "V":   # V ranks by importance x token range of the (dequantisation-free) originals
                rng = torch.cat([(V[:, :, 32 * b:32 * b + 32].max(-1)[0] - V[:, :, 32 * b:32 * b + 32].min(-1)[0]).sum(0).sum(0)
                                 for b, _ in order])
                imp = imp * rng
            blk = (imp.reshape(total_blocks, 32) / 32).sum(-1)
            ranked = torch.sort(blk, descending=True, stable=True)[1].tolist()
            counts = [c // 32 for c in st["counts"]]
            tgt, pos = {}, 0
            for bits, c in zip((16, 8, 4, 2, 1, 0), counts):
                for p in ranked[pos:pos + c]:
                    tgt[p] = bits
                pos += c
            nxt = []
            for p, (bid, chain) in enumerate(order):
                t = tgt[p]
                if t == 0:
                    continue
                if chain is None:
                    chain = [t]
                elif t < chain[-1]:
                    chain = chain + [t]
                nxt.append((bid, chain))
            order = nxt
            n_seen += n_new_blocks
        sides[side] = order
    return sides


def _expected_block(x_block, chain, is_k):
    """x_block (B,H,32,D) original fp16 -> value after the chain of quantise/dequantise steps."""
    x = x_block
    for bits in chain:
        if bits == 16:
            continue
        if is_k:
            x = O.uniform_group_fake_quant(x.transpose(2, 3).contiguous(), 32, bits).transpose(2, 3)
        else:
            x = O.uniform_group_fake_quant(x.contiguous(), 32, bits)
    return x


def test_oracle_policy_matches_history_model():
    caches, log, (K, V) = PC.run(_oracle_compress)
    # the V ranking needs distinct block scores to be order-independent of sort stability; check that
    final = caches[-1]
    model = _model(log, K, V)
    dK, dV = O.reconstruct_cache(final)
    n_res = 0 if final[39] is None else final[39].shape[2]
    for side, dense, src, is_k in (("K", dK, K, True), ("V", dV, V, False)):
        order = model[side]
        assert dense.shape[2] == 32 * len(order) + n_res
        for p, (bid, chain) in enumerate(order):
            exp = _expected_block(src[:, :, 32 * bid:32 * bid + 32], chain, is_k)
            got = dense[:, :, 32 * p:32 * p + 32]
            assert torch.equal(got, exp), (side, p, bid, chain)
    # class membership: the number of tokens per class equals the model's count of final precisions
    for side, slots in (("K", (0, 4, 12, 20, 28)), ("V", (2, 8, 16, 24, 32))):
        for bits, s in zip((16, 8, 4, 2, 1), slots):
            want = 32 * sum(1 for _, ch in model[side] if ch[-1] == bits)
            have = 0 if final[s + 1] is None else final[s + 1].numel()
            assert have == want, (side, bits, have, want)


def test_oracle_policy_invariants_every_step():
    caches, log, _ = PC.run(_oracle_compress)
    for pkv, st in zip(caches, log):
        kept = st["history"] + st["compress_length"] - st["counts"][5]
        for slots in ((1, 5, 13, 21, 29), (3, 9, 17, 25, 33)):
            idx = torch.cat([pkv[s] for s in slots if pkv[s] is not None])
            assert sorted(idx.tolist()) == list(range(kept)), "class positions partition the survivors"
            for s in slots:
                if pkv[s] is not None:
                    assert pkv[s].numel() % 32 == 0 and pkv[s].dtype == torch.int64
        assert pkv[38].numel() == kept
        # shapes of a quantised class agree with its index
        for b, s in ((8, 4), (4, 12), (2, 20), (1, 28)):
            if pkv[s] is not None:
                n = pkv[s + 1].numel()
                assert pkv[s].shape == (PC.B, PC.H, PC.D, n * b // 32) and pkv[s + 2].shape == (PC.B, PC.H, PC.D, n // 32)
            if pkv[s + 4] is not None:
                assert pkv[s + 4].shape == (PC.B, PC.H, pkv[s + 5].numel(), PC.D * b // 32)


def test_block_planner_against_the_move_sequence_by_brute_force():
    """The library's host-side planner (hqekv_plan_side, through the product's wrapper) against the reference's
    sequence of moves written out with plain loops (quant/hqe_2.py:552-659): for every target from 1 bit up -- its
    members that stay, the new tokens ranked into it, then what comes down from the fp16, 8, 4 and 2-bit classes in
    source order; a block ranked into a higher precision stays; evicted blocks appear nowhere, and the survivors'
    new block numbers are their ranks among the survivors (quant/hqe_2.py:661-670)."""
    import numpy as np
    from hqekv_amd import cache_policy as cp
    rng = np.random.default_rng(0)
    for trial in range(300):
        hist, n_new = int(rng.integers(0, 40)), int(rng.integers(1, 8))
        total = hist + n_new
        parts = np.split(rng.permutation(hist), np.sort(rng.integers(0, hist + 1, 4)))
        old = {b: parts[i].astype(np.int64) for i, b in enumerate(cp.CLASS_BITS) if parts[i].size}
        n_targets = 6 if trial % 3 else 5
        label = rng.integers(0, n_targets, total).astype(np.int8)
        # a ranking and token counts that produce exactly these labels
        order = np.concatenate([rng.permutation(np.flatnonzero(label == t)) for t in range(n_targets)]).astype(np.int64)
        bit_num = [int((label == t).sum()) * 32 for t in range(n_targets)]
        got = cp._plan_side_c(old, hist, n_new, order, bit_num)
        assert got is not None, trial
        counts, words, alive = got
        want = []
        for ti, bits in enumerate(cp.CLASS_BITS):
            for j, p in enumerate(old.get(bits, [])):
                if label[p] <= ti:
                    want.append((ti, ti, j, p))
            for j in range(n_new):
                if label[hist + j] == ti:
                    want.append((ti, 5, j, hist + j))
            for si in range(ti):
                for j, p in enumerate(old.get(cp.CLASS_BITS[si], [])):
                    if label[p] == ti:
                        want.append((ti, si, j, p))
        u = len(want)
        assert words.size == 2 * u, trial
        assert [(w[1] << 24) | w[2] for w in want] == words[:u].tolist(), trial
        survivors = sorted(w[3] for w in want)
        rank = {p: r for r, p in enumerate(survivors)}
        assert [rank[w[3]] for w in want] == words[u:].tolist(), trial
        assert counts.tolist() == [sum(1 for w in want if w[0] == t) for t in range(5)], trial
        if u < total:
            assert alive.tolist() == survivors, trial
        else:
            assert alive is None, trial
    # what the planner refuses: counts that are not whole blocks, a ranking that names a block twice, classes that do
    # not partition the history
    old = {16: np.array([0, 1], dtype=np.int64)}
    order = np.array([0, 1, 2], dtype=np.int64)
    assert cp._plan_side_c(old, 2, 1, order, [32, 0, 0, 0, 64]) is not None
    assert cp._plan_side_c(old, 2, 1, order, [33, 0, 0, 0, 63]) is None
    assert cp._plan_side_c(old, 2, 1, np.array([0, 0, 2], dtype=np.int64), [32, 0, 0, 0, 64]) is None
    assert cp._plan_side_c({16: np.array([0, 0], dtype=np.int64)}, 2, 1, order, [32, 0, 0, 0, 64]) is None
    assert cp._plan_side_c(old, 2, 1, order, [32, 0, 0, 0, 32]) is None


def test_cover_once_verdict_is_not_reused_for_other_tensors():
    """The remembered verdict of ``idx_cover_once`` belongs to the very tensors it was formed on, in the state they
    were in: an array written in place, or another array in the place of one that has been freed, is checked again."""
    from hqekv_amd.attention import idx_cover_once
    a = torch.arange(0, 64, dtype=torch.int32)
    b = torch.arange(64, 128, dtype=torch.int32)
    assert idx_cover_once([a, b], 128) and idx_cover_once([a, b], 128)
    assert a._hq_cover[1] is True
    del b
    for _ in range(8):   # new arrays of the same size, one of which may well land where b was
        c = torch.arange(60, 124, dtype=torch.int32)          # overlaps a: not a partition
        assert not idx_cover_once([a, c], 128)
        del c
    b = torch.arange(64, 128, dtype=torch.int32)
    assert idx_cover_once([a, b], 128)
    b[5] = 3                                                   # written through torch: the version moves
    assert not idx_cover_once([a, b], 128)
    b[5] = 69
    assert idx_cover_once([a, b], 128)
    assert not idx_cover_once([a, b], 129) and not idx_cover_once([a], 128)


def test_class_sizes_and_ratio_update_equal_the_tensor_arithmetic():
    """The layer's class sizes and ratio update run on numpy float32 scalars; the reference does the same float32
    operations on CPU tensors (model/llama_hqe.py:216-224,235-239), restated in the oracle: same shares, same counts,
    same ratios, bit for bit, over random ratios, histories and lengths."""
    import random
    from hqekv_amd.decode_layer import class_token_counts, ratios_for_next_increment
    rnd = random.Random(7)
    for _ in range(3000):
        total = rnd.choice([32, 64, 96, 128, 320, 1024, 26208, 32768, 131072, rnd.randrange(1, 5000) * 32])
        b0 = rnd.random() * 0.5
        a, c, d = rnd.random(), rnd.random(), rnd.random() * rnd.choice([0, 1])
        e0 = torch.tensor([b0], dtype=torch.float32)
        rq = torch.tensor([a, c, d], dtype=torch.float32) * ((1 - b0) / (a + c + d))
        hist = rnd.randrange(0, 4000) * 32
        add = (hist + 32) // 32 * 32 - hist
        re_t = (add * e0) / (hist + add)                       # the reference's lines, on tensors
        rq_t = (1 - re_t) * rq / rq.sum()
        re_n, rq_n = ratios_for_next_increment(hist, e0, rq)
        assert torch.equal(re_t, re_n) and torch.equal(rq_t, rq_n), (hist, b0, a, c, d)
        shares_o, counts_o = O.split_history(total, rq_t, re_t)
        shares_n, counts_n = class_token_counts(total, rq_n, re_n)
        assert torch.equal(shares_o, shares_n) and torch.equal(counts_o, counts_n), (total, b0, a, c, d)
        assert counts_n.dtype == counts_o.dtype and shares_n.dtype == torch.float32
        assert int(counts_n.sum()) == total // 32 * 32 and bool((counts_n % 32 == 0).all())
