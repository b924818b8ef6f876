"""Synthetic caches of the benchmark shapes (seeded, no datasets or checkpoints).

K, V ~ N(0,1) fp16 with four K channels per head scaled x10 as outliers, q ~ N(0,1).  The
per-token precision split is block-granular (32 tokens), as the reference only ever assigns whole
blocks (model/public_func.py:92-106): blocks are ranked by the mean of a seeded uniform score and
cut into fp16 / 8 / 4 / 2-bit / evicted shares; survivors keep their original order and a token's
position is its rank among survivors (quant/hqe_2.py:661-670).

``quantize`` is injected (the HIP quantiser for the product and bench, the CPU oracle in tests), so
this module contains no arithmetic of its own.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional, Sequence, Tuple

import torch

OUTLIER_CHANNELS = (3, 35, 67, 99)
CLASS_ORDER = (16, 8, 4, 2, 0)  # 0 = evicted
CLASS_ORDER_1BIT = (16, 8, 4, 2, 1, 0)  # six fractions: with the uniform 1-bit class


def make_qkv(B: int, Hq: int, Hkv: int, T: int, D: int, seed: int, device="cpu"):
    """-> q (B,Hq,1,D), K (B,Hkv,T,D), V (B,Hkv,T,D), all fp16, generated on the CPU from ``seed``."""
    g = torch.Generator().manual_seed(seed)
    K = torch.randn(B, Hkv, T, D, generator=g)
    V = torch.randn(B, Hkv, T, D, generator=g)
    q = torch.randn(B, Hq, 1, D, generator=g)
    for c in OUTLIER_CHANNELS:
        if c < D:
            K[..., c] *= 10.0
    return q.half().to(device), K.half().to(device), V.half().to(device)


def block_counts(n_blocks: int, fractions: Sequence[float]) -> list:
    """Blocks per class for ``fractions`` over CLASS_ORDER; the rounding remainder goes to the last
    class with a non-zero share."""
    counts = [int(round(n_blocks * f)) for f in fractions]
    last = max(i for i, f in enumerate(fractions) if f > 0)
    counts[last] += n_blocks - sum(counts)
    assert min(counts) >= 0 and sum(counts) == n_blocks
    return counts


def split_blocks(T: int, fractions: Sequence[float], seed: int, block: int = 32) -> Dict[int, torch.Tensor]:
    """-> {bits: original token indices (ascending)} for bits in CLASS_ORDER (0 = evicted)."""
    assert T % block == 0
    n_blocks = T // block
    g = torch.Generator().manual_seed(seed)
    score = torch.rand(T, generator=g, dtype=torch.float32)
    order = torch.argsort(score.view(n_blocks, block).mean(-1), descending=True, stable=True)
    counts = block_counts(n_blocks, fractions)
    out, start = {}, 0
    ar = torch.arange(block)
    order_of = CLASS_ORDER if len(fractions) == len(CLASS_ORDER) else CLASS_ORDER_1BIT
    assert len(fractions) == len(order_of)
    for bits, c in zip(order_of, counts):
        blocks = torch.sort(order[start:start + c])[0]
        out[bits] = (blocks[:, None] * block + ar[None, :]).reshape(-1)
        start += c
    return out


def survivor_positions(classes: Dict[int, torch.Tensor], T: int) -> Tuple[Dict[int, torch.Tensor], int]:
    """Rank of every kept token among all kept tokens, per class."""
    alive = torch.ones(T, dtype=torch.bool)
    if 0 in classes and classes[0].numel():
        alive[classes[0]] = False
    rank = torch.cumsum(alive.to(torch.int64), 0) - 1
    pos = {b: rank[idx] for b, idx in classes.items() if b != 0}
    return pos, int(alive.sum())


def build_cache(K: torch.Tensor, V: torch.Tensor, classes: Dict[int, torch.Tensor], n_residual: int,
                quantize: Callable, idx_override: Optional[Dict[int, torch.Tensor]] = None) -> tuple:
    """Build the reference's 42-field tuple from full-precision K, V (B,Hkv,T,D).

    The last ``n_residual`` tokens stay in new_K / new_V; ``classes`` partitions the rest.
    ``quantize(x, 32, bits) -> (code, scale, zero)`` over the last dim.  ``idx_override`` replaces
    the positions (used to test arbitrary permutations).
    """
    B, H, T, D = K.shape
    Tq = T - n_residual
    pos, kept = survivor_positions(classes, Tq)
    if idx_override is not None:
        pos = idx_override
    dev = K.device
    t = [None] * 42
    for bits, tok in classes.items():
        if bits == 0 or tok.numel() == 0:
            continue
        tok_d = tok.to(dev)
        k = K[:, :, tok_d, :]
        v = V[:, :, tok_d, :]
        p = pos[bits].to(dev)
        if bits == 16:
            t[0], t[1], t[2], t[3] = k.transpose(2, 3).contiguous(), p, v.contiguous(), p.clone()
        else:
            kb = {8: 4, 4: 12, 2: 20, 1: 28}[bits]
            vb = kb + 4
            kc, ks, kz = quantize(k.transpose(2, 3).contiguous(), 32, bits)
            vc, vs, vz = quantize(v.contiguous(), 32, bits)
            t[kb], t[kb + 1], t[kb + 2], t[kb + 3] = kc, p, ks, kz
            t[vb], t[vb + 1], t[vb + 2], t[vb + 3] = vc, p.clone(), vs, vz
    if n_residual > 0:
        t[39] = K[:, :, Tq:, :].contiguous()
        t[40] = V[:, :, Tq:, :].contiguous()
    t[41] = kept + n_residual
    return tuple(t)


def cache_to(pkv: tuple, device) -> tuple:
    return tuple(x.to(device) if torch.is_tensor(x) else x for x in pkv)


def algorithmic_bytes(pkv: tuple, Hq: int) -> int:
    """Bytes one decode-attention layer-step must move: packed codes + scale/zero, fp16 classes and
    residual, one idx per class for K and for V, q and the output.  The attn_weights buffer the
    caller receives is not counted."""
    n = 0
    for i, x in enumerate(pkv[:41]):
        if torch.is_tensor(x) and i not in (36, 37, 38):
            n += x.numel() * x.element_size()
    some = next(x for x in (pkv[2], pkv[8], pkv[16], pkv[24], pkv[32], pkv[40]) if x is not None)
    B, D = some.shape[0], (pkv[40].shape[3] if pkv[40] is not None else pkv[2].shape[3] if pkv[2] is not None else 128)
    n += 2 * B * Hq * D * 2
    return n


# benchmark configurations (fractions over fp16 / 8 / 4 / 2 / evicted)
CONFIGS = {
    "c1": dict(B=1, Hq=32, Hkv=8, D=128, T=4096, residual=128, fractions=(0.0, 0.0, 0.0, 1.0, 0.0), seed=1235),
    "c2": dict(B=1, Hq=32, Hkv=8, D=128, T=32768, residual=0, fractions=(0.05, 0.15, 0.30, 0.30, 0.20), seed=1236),
    "c4": dict(B=8, Hq=32, Hkv=8, D=128, T=65536, residual=0, fractions=(0.10, 0.0, 0.20, 0.50, 0.20), seed=1238),
    # the decode-attention share of configuration 5: average 2.56 bit per kept-or-evicted element
    "c5": dict(B=4, Hq=32, Hkv=8, D=128, T=131072, residual=0, fractions=(0.02, 0.03, 0.25, 0.50, 0.20), seed=1239),
}


def build_config(name: str, quantize: Callable, device="cpu", layer: int = 0):
    """-> (q, cache tuple) for a named configuration; ``layer`` varies the seed for distinct copies."""
    c = CONFIGS[name]
    q, K, V = make_qkv(c["B"], c["Hq"], c["Hkv"], c["T"], c["D"], c["seed"] + 1000 * layer, device)
    classes = split_blocks(c["T"] - c["residual"], c["fractions"], c["seed"] + 1000 * layer)
    return q, build_cache(K, V, classes, c["residual"], quantize)
