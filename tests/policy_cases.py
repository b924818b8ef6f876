"""Shared scenario for the cache-policy tests: three successive compressions with demotions and
evictions, driven by explicit per-step token counts (all multiples of 32)."""
import torch

from oracle import hqe_oracle as O

B, H, D = 1, 2, 128

# (new tokens this step, residual kept fp16, [fp16, 8, 4, 2, 1, evict] token counts over history+new)
STEPS = [
    dict(n_new=256 + 7, counts=[64, 32, 64, 32, 32, 32]),
    dict(n_new=64 + 3, counts=[32, 32, 64, 96, 32, 32]),       # 7 carried + 64+3 new -> compress 64, residual 10
    dict(n_new=96, counts=[32, 0, 64, 128, 64, 64]),
]


def make_inputs(seed=11):
    g = torch.Generator().manual_seed(seed)
    total_new = sum(s["n_new"] for s in STEPS)
    K = torch.randn(B, H, total_new, D, generator=g)
    K[..., 5] *= 10
    V = torch.randn(B, H, total_new, D, generator=g)
    imps = [torch.rand(4096, generator=g) for _ in STEPS]
    return K.half(), V.half(), imps


def run(compress, to_dev=lambda x: x, rank_blocks=O.get_block_token_idx):
    """Drive ``compress(pkv, compress_length, history, K_sorted_idx, K_bit_num, V_bit_num, importance)``
    through STEPS; returns the list of caches after every step plus what each step was given."""
    K, V, imps = make_inputs()
    pkv = tuple([None] * 42)
    history, consumed, carried_K, carried_V = 0, 0, None, None
    out, log = [], []
    for step, imp in zip(STEPS, imps):
        nk = K[:, :, consumed:consumed + step["n_new"]]
        nv = V[:, :, consumed:consumed + step["n_new"]]
        consumed += step["n_new"]
        new_K = nk if carried_K is None else torch.cat((carried_K, nk), dim=2)
        new_V = nv if carried_V is None else torch.cat((carried_V, nv), dim=2)
        cur = new_K.shape[2]
        compress_length = cur - cur % 32
        total = history + compress_length
        counts = torch.tensor(step["counts"], dtype=torch.int32)
        assert int(counts.sum()) == total, (int(counts.sum()), total)
        importance = imp[:total].float()  # fp32 scores: no ties, so the (unstable) block sort has one answer
        K_sorted = rank_blocks(32, total // 32, importance.clone())
        t = list(pkv)
        t[39], t[40], t[41] = to_dev(new_K), to_dev(new_V), history + cur
        pkv = compress(tuple(t), compress_length, history, to_dev(K_sorted), counts, counts.clone(), to_dev(importance))
        log.append(dict(compress_length=compress_length, history=history, counts=step["counts"],
                        K_sorted=K_sorted, importance=importance))
        history = total - step["counts"][5]
        carried_K = None if pkv[39] is None else pkv[39].cpu()
        carried_V = None if pkv[40] is None else pkv[40].cpu()
        # after a compression kv_seq_len is what survives plus the residual
        t = list(pkv)
        t[41] = history + (0 if pkv[39] is None else pkv[39].shape[2])
        pkv = tuple(t)
        out.append(pkv)
    return out, log, (K, V)
