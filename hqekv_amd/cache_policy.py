"""Class assignment and migration of the hybrid cache (host logic; the arithmetic runs in HIP kernels).

One engine serves both generations of the reference's policy:
  * ``KV_cache_hqe_2``      quant/hqe_2.py:456-843        (six targets: 16/8/4/2/1 bit + evict)
  * ``KV_cache_compress``   quant/hybrid_quant.py:318-612  (five targets, no eviction)
  * ``KV_cache_compress_1`` quant/hybrid_quant.py:614-730  (same, V range supplied by the caller)

What is normative, because it fixes the order of tokens inside every class and therefore the packed
bytes: targets are served from the lowest precision up (evict, 1, 2, 4, 8, 16); for each target the
sources are visited as new tokens, then the 16, 8, 4, 2-bit classes, and only sources of HIGHER
precision than the target move (a token is never promoted); moved tokens are appended to the target
in source order; a quantised source is dequantised (two fp16 roundings) and re-quantised; K moves in
whole 32-token groups.  After an eviction every surviving index is replaced by its rank among the
survivors (quant/hqe_2.py:661-670).

Two engines produce the same bytes.  ``gather`` (the default wherever it applies): everything the reference
moves is a whole block of 32 tokens and every block ends in exactly one place, so the host works out, per
block, where each class's blocks come from (``hqekv_plan_side``, the library's host-side planner: one C call
per side over a few thousand entries), and ONE kernel launch per side
(``hqekv_cache_migrate``) rebuilds all classes from the old ones and the new tokens -- survivors copied, demoted
blocks dequantised and re-quantised, new blocks quantised, evicted blocks left out, positions re-ranked; the
device is waited for once, to fetch the two block rankings.  ``steps``: the general engine for selections that
are not made of whole aligned blocks (token-level V selections): the reference's sequence of moves with
``index_select`` gathers and one quantiser call per move.
"""
from __future__ import annotations

import os
import threading
from typing import Dict, List, Optional

import numpy as np
import torch

from . import pack_unpack as PU
from .public_func import RankedBlocks, calculate_token_range, get_block_token_idx, rank_blocks_weighted

BLOCK = 32
CLASS_BITS = (16, 8, 4, 2, 1)
K_SLOT = {16: 0, 8: 4, 4: 12, 2: 20, 1: 28}
V_SLOT = {16: 2, 8: 8, 4: 16, 2: 24, 1: 32}
_STRATEGIES = ("uniform", "normal", "uniform_group", "normal_group", "high_uniform_group_low_normal_group")


class _Cls:
    """One precision class of one side (K or V): data, positions, scale, zero.

    ``idx_h`` is the host copy (numpy int64) of the positions; the bookkeeping of a compression -- which
    tokens move where -- is done on it, so the device is only asked to gather rows / columns and to quantise.
    ``idx`` (the device tensor the tuple carries) is None while the host copy is ahead of it."""
    __slots__ = ("data", "idx", "scale", "zero", "idx_h")

    def __init__(self, data=None, idx=None, scale=None, zero=None, idx_h=None):
        self.data, self.idx, self.scale, self.zero, self.idx_h = data, idx, scale, zero, idx_h

    @property
    def empty(self) -> bool:
        return self.data is None


def _host_idx(t: torch.Tensor) -> np.ndarray:
    """Host copy of a position tensor.  Tensors made by this module carry theirs along (no device
    round trip) -- token by token, or as the first positions of their 32-token blocks; for anyone else's the
    copy is fetched, which waits for the device."""
    trusted = getattr(t, "_hq_host_version", None) == t._version  # nobody wrote to the tensor since
    h = getattr(t, "_hq_host", None) if trusted else None
    if h is not None and h.shape[0] == t.numel():
        return h
    blocks = getattr(t, "_hq_blocks", None) if trusted else None
    if blocks is not None and blocks.shape[0] * BLOCK == t.numel():
        h = (blocks.astype(np.int64)[:, None] * BLOCK + np.arange(BLOCK, dtype=np.int64)).reshape(-1)
        t._hq_host = h
        return h
    return t.detach().to("cpu", torch.int64).numpy()


def _host_blocks(t: torch.Tensor) -> Optional[np.ndarray]:
    """Block numbers (first position / 32) of a position tensor made of whole aligned blocks, else None."""
    if isinstance(t, RankedBlocks):
        t = t.tokens()
    if getattr(t, "_hq_host_version", None) == t._version:
        blocks = getattr(t, "_hq_blocks", None)
        if blocks is not None and blocks.shape[0] * BLOCK == t.numel():
            return blocks
    if t.numel() % BLOCK:
        return None
    h = _host_idx(t).reshape(-1, BLOCK)
    if h.size and (bool((h[:, 0] % BLOCK).any()) or not bool((h == h[:, :1] + np.arange(BLOCK)).all())):
        return None
    return (h[:, 0] // BLOCK).astype(np.int64)


class _Staging:
    """Page-locked staging area for the small index arrays a compression sends to the device: a copy out of
    pageable memory is synchronous (tens of microseconds each, a dozen per compression), one out of
    page-locked memory is queued like a kernel.  Slices are handed out in ring order; every copy leaves an
    event on the stream that issued it, and before the ring wraps all events of the lap are waited for, so a
    slice is never overwritten while a copy on any stream may still read it.  One lock serialises callers."""
    WORDS = 1 << 20  # int64 entries (8 MiB)

    def __init__(self):
        self.buf = torch.empty(self.WORDS, dtype=torch.int64, pin_memory=True)
        self.view = self.buf.numpy()
        self.pos = 0
        self.events: list = []
        self.lock = threading.Lock()

    def put(self, a: np.ndarray, dev) -> torch.Tensor:
        n = a.size
        if n > self.WORDS // 4:
            return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(dev)
        with self.lock:
            if self.pos + n > self.WORDS:
                for ev in self.events:
                    ev.synchronize()
                self.events.clear()
                self.pos = 0
            lo = self.pos
            self.pos += n
            self.view[lo:lo + n] = a
            out = self.buf[lo:lo + n].to(dev, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record(torch.cuda.current_stream(dev))
            self.events.append(ev)
        return out


_staging: Optional[_Staging] = None


def _to_dev(a: np.ndarray, dev) -> torch.Tensor:
    global _staging
    dev = torch.device(dev)
    if dev.type != "cuda":
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(dev)
    if _staging is None:
        _staging = _Staging()
    return _staging.put(a, dev)


def _dev_idx(h: np.ndarray, dev) -> torch.Tensor:
    t = _to_dev(h, dev)
    t._hq_host = h   # never modified afterwards
    t._hq_host_version = t._version
    return t


def _read_side(pkv: tuple, slots: Dict[int, int], host: bool = False) -> Dict[int, _Cls]:
    out = {}
    for b in CLASS_BITS:
        s = slots[b]
        c = _Cls(pkv[s], pkv[s + 1]) if b == 16 else _Cls(pkv[s], pkv[s + 1], pkv[s + 2], pkv[s + 3])
        if host and c.idx is not None:
            c.idx_h = _host_idx(c.idx)
        out[b] = c
    return out


def _write_side(t: list, side: Dict[int, _Cls], slots: Dict[int, int], dev=None) -> None:
    for b in CLASS_BITS:
        s, c = slots[b], side[b]
        if c.data is not None and c.idx is None:
            c.idx = _dev_idx(c.idx_h, dev)
        t[s], t[s + 1] = c.data, c.idx
        if b != 16:
            t[s + 2], t[s + 3] = c.scale, c.zero


def _cat(a: Optional[torch.Tensor], b: torch.Tensor, dim: int) -> torch.Tensor:
    return b if a is None else torch.cat((a, b), dim=dim)


def _cat_h(a: Optional[np.ndarray], b: np.ndarray) -> np.ndarray:
    return b if a is None else np.concatenate((a, b))


def _none_if_empty(x: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if x is None or x.numel() == 0 else x


LOW_NORMAL = "high_uniform_group_low_normal_group"


def _quantize(x: torch.Tensor, bits: int, strategy: str):
    """8/4/2 bit: the uniform quantiser; 1 bit: uniform under 'uniform_group', normal-quantile under
    'high_uniform_group_low_normal_group' (quant/hqe_2.py:482-492)."""
    if bits == 1 and strategy == LOW_NORMAL:
        return PU.normal_group_quantize_pack_last_dim(x, BLOCK, 1)
    return PU.uniform_group_quantize_pack_last_dim(x, BLOCK, bits)


def _dequantize(c: "_Cls", bits: int, strategy: str) -> torch.Tensor:
    if bits == 1 and strategy == LOW_NORMAL:
        return PU.normal_group_dequantize_unpack_last_dim(c.data, c.scale, c.zero, BLOCK, 1)
    return PU.uniform_group_dequantize_unpack_last_dim(c.data, c.scale, c.zero, BLOCK, bits)


def _check_low_bits(bits: int, strategy: str) -> None:
    if strategy not in ("uniform_group", "high_uniform_group_low_normal_group"):
        raise NotImplementedError(f"quant_strategy '{strategy}' uses quantiser families that are not built")


# ----------------------------------------------------------------------------------------------- K side
# K classes are channel-major (B, H, D, X): X = tokens (fp16), tokens/pf (codes), tokens/32 (scale, zero).

def _k_split(c: _Cls, bits: int, mask: np.ndarray):
    """-> (moved class, kept class); ``mask`` (host, bool) marks tokens of ``c`` and must cover whole
    32-token groups."""
    gm = mask.reshape(-1, BLOCK)
    if not bool((gm == gm[:, :1]).all()):
        raise ValueError("K classes move in whole 32-token groups: the selection splits a group")
    g_all = gm[:, 0]
    sel, keep = np.flatnonzero(g_all), np.flatnonzero(~g_all)
    per = BLOCK if bits == 16 else BLOCK // (32 // bits)
    dev = c.data.device

    def part(groups: np.ndarray, m: np.ndarray) -> _Cls:
        if groups.size == 0:
            return _Cls()
        cols = (groups[:, None] * per + np.arange(per)[None, :]).reshape(-1)
        data = c.data.index_select(3, _to_dev(cols, dev))
        if bits == 16:
            return _Cls(data, idx_h=c.idx_h[m])
        g_t = _to_dev(groups, dev)
        return _Cls(data, None, c.scale.index_select(3, g_t), c.zero.index_select(3, g_t), c.idx_h[m])

    return part(sel, mask), part(keep, ~mask)


def _k_to_fp16(c: _Cls, bits: int, strategy: str = "uniform_group") -> torch.Tensor:
    if bits == 16:
        return c.data
    return _dequantize(c, bits, strategy)


def _k_append(dst: _Cls, x: torch.Tensor, idx_h: np.ndarray, bits: int, strategy: str = "uniform_group") -> None:
    """x is (B, H, D, n) fp16, possibly the transposed view of token-major memory."""
    if bits == 16:
        dst.data = _cat(dst.data, x, 3)
    else:
        code, scale, zero = _quantize(x, bits, strategy)
        dst.data, dst.scale, dst.zero = _cat(dst.data, code, 3), _cat(dst.scale, scale, 3), _cat(dst.zero, zero, 3)
    dst.idx_h, dst.idx = _cat_h(dst.idx_h, idx_h), None


# ----------------------------------------------------------------------------------------------- V side
# V classes are token-major (B, H, n, X): X = D (fp16), D/pf (codes), D/32 (scale, zero).

def _v_split(c: _Cls, bits: int, mask: np.ndarray):
    sel, keep = np.flatnonzero(mask), np.flatnonzero(~mask)
    dev = c.data.device

    def part(rows: np.ndarray) -> _Cls:
        if rows.size == 0:
            return _Cls()
        r_t = _to_dev(rows, dev)
        if bits == 16:
            return _Cls(c.data.index_select(2, r_t), idx_h=c.idx_h[rows])
        return _Cls(c.data.index_select(2, r_t), None, c.scale.index_select(2, r_t),
                    c.zero.index_select(2, r_t), c.idx_h[rows])

    return part(sel), part(keep)


def _v_to_fp16(c: _Cls, bits: int, strategy: str = "uniform_group") -> torch.Tensor:
    if bits == 16:
        return c.data
    return _dequantize(c, bits, strategy)


def _v_append(dst: _Cls, x: torch.Tensor, idx_h: np.ndarray, bits: int, strategy: str = "uniform_group") -> None:
    if bits == 16:
        dst.data = _cat(dst.data, x, 2)
    else:
        code, scale, zero = _quantize(x, bits, strategy)
        dst.data, dst.scale, dst.zero = _cat(dst.data, code, 2), _cat(dst.scale, scale, 2), _cat(dst.zero, zero, 2)
    dst.idx_h, dst.idx = _cat_h(dst.idx_h, idx_h), None


# ----------------------------------------------------------------------------------------------- engine

def _targets(sorted_idx: torch.Tensor, bit_num: torch.Tensor) -> List[Optional[np.ndarray]]:
    """Slices (host) of the ranked token list for (16, 8, 4, 2, 1[, evict]); None where a share is empty."""
    cum = [0] + [int(v) for v in torch.cumsum(bit_num.to(torch.int64).cpu(), 0).tolist()]
    packed = getattr(sorted_idx, "_hq_block_order", None)
    if packed is not None and packed[0].numel() * packed[1] == sorted_idx.numel() \
            and getattr(sorted_idx, "_hq_block_order_version", None) == sorted_idx._version:
        order, bs = packed  # made by get_block_token_idx: whole blocks in ranked order
        sorted_h = (order.detach().to("cpu", torch.int64).numpy()[:, None] * bs + np.arange(bs, dtype=np.int64)).reshape(-1)
    else:
        sorted_h = sorted_idx.detach().to("cpu", torch.int64).numpy()
    return [sorted_h[cum[i]:cum[i + 1]] if cum[i + 1] > cum[i] else None for i in range(len(cum) - 1)]


def _rerank(side: Dict[int, _Cls], total: int) -> None:
    """Survivors keep their order; each index becomes its rank among all survivors."""
    alive = np.zeros(total, dtype=np.int64)
    for b in CLASS_BITS:
        if side[b].idx_h is not None:
            alive[side[b].idx_h] = 1
    rank = np.cumsum(alive) - 1
    for b in CLASS_BITS:
        c = side[b]
        if c.idx_h is not None:
            c.idx_h, c.idx = rank[c.idx_h], None


def _migrate(side: Dict[int, _Cls], new: torch.Tensor, targets: List[Optional[np.ndarray]], history: int,
             is_k: bool, strategy: str, on_evict=None):
    """Run one compression on one side.  ``new`` is (B, H, n_new, D) fp16 (token-major for K and V alike)."""
    dev = new.device
    total = history + new.shape[2]
    new_idx = np.arange(history, total, dtype=np.int64)
    # membership of a position in a target set through one label per position (what the reference asks with
    # torch.isin per class, quant/hqe_2.py:552-659): label[p] = index of the target list that holds p
    label = np.full(total, -1, dtype=np.int8)
    for ti, tgt in enumerate(targets):
        if tgt is not None:
            label[tgt] = ti

    def member(idx_h: np.ndarray, ti: int) -> np.ndarray:
        return label[idx_h] == ti

    split, to16, append = (_k_split, _k_to_fp16, _k_append) if is_k else (_v_split, _v_to_fp16, _v_append)
    evict = targets[5] if len(targets) > 5 else None

    def take_new(mask: np.ndarray) -> torch.Tensor:
        nonlocal new, new_idx
        rows, keep = np.flatnonzero(mask), np.flatnonzero(~mask)
        moved = new.index_select(2, _to_dev(rows, dev))
        new, new_idx = new.index_select(2, _to_dev(keep, dev)), new_idx[keep]
        return moved

    # 1. eviction: dropped tokens leave every tensor
    if evict is not None:
        m = member(new_idx, 5)
        if m.any():
            take_new(m)
        for b in CLASS_BITS:
            c = side[b]
            if c.idx_h is None:
                continue
            m = member(c.idx_h, 5)
            if m.any():
                _, side[b] = split(c, b, m)
        if on_evict is not None:
            on_evict(side, new_idx)

    # 2. demotions, lowest target first; sources: new tokens, then 16, 8, 4, 2 (only above the target)
    for ti in (4, 3, 2, 1, 0):
        tgt_bits, tgt_idx = CLASS_BITS[ti], targets[ti]
        if tgt_idx is None:
            continue
        if new_idx.size:
            m = member(new_idx, ti)
            if m.any():
                if tgt_bits < 16:
                    _check_low_bits(tgt_bits, strategy)
                sel_idx = new_idx[m]
                moved = take_new(m)  # (B, H, n, D)
                append(side[tgt_bits], moved.transpose(2, 3) if is_k else moved, sel_idx, tgt_bits, strategy)
        for src_bits in CLASS_BITS:
            if src_bits <= tgt_bits:
                break
            c = side[src_bits]
            if c.idx_h is None:
                continue
            m = member(c.idx_h, ti)
            if not m.any():
                continue
            _check_low_bits(tgt_bits, strategy)
            moved, side[src_bits] = split(c, src_bits, m)
            append(side[tgt_bits], to16(moved, src_bits, strategy), moved.idx_h, tgt_bits, strategy)

    if evict is not None:
        _rerank(side, total)
    return new, new_idx


# ----------------------------------------------------------------------------------------------- gather engine
# Everything below works on whole 32-token blocks.  A side's state is, per class, the block numbers (first position
# / 32) of its blocks in stored order; a compression turns it into the same thing for the new classes plus, per new
# block, where its bytes come from.

_SRC_NEW = 5   # source slot of the new fp16 tokens (slots 0..4: the old fp16, 8, 4, 2, 1-bit classes)


def _plan_side_c(old_blocks: Dict[int, np.ndarray], hist_blocks: int, n_new_blocks: int, order_h: np.ndarray, bit_num):
    """The block-level plan of one side from the library's host-side planner (``hqekv_plan_side``): which new class
    every block lands in, in which order, and its new position.  -> (blocks per new class (5,), plan words -- source entries then
    new block numbers, ready for the kernel --, surviving old block numbers ascending, or None when nothing was
    evicted), or None when the ranking or the counts are not made of whole blocks covering every block once."""
    from . import _lib
    import ctypes as C
    total = hist_blocks + n_new_blocks
    counts_t = bit_num.tolist() if torch.is_tensor(bit_num) else [int(v) for v in bit_num]
    if order_h is None or order_h.shape[0] != total:
        return None

    def addr(a: np.ndarray) -> int:   # (cheaper than a.ctypes.data, which builds a ctypes object per call)
        return a.__array_interface__["data"][0]
    order64 = order_h if order_h.dtype == np.int64 and order_h.flags.c_contiguous else np.ascontiguousarray(order_h, dtype=np.int64)
    ptrs = (C.c_void_p * 5)()
    cnts = (C.c_int32 * 5)()
    hold = []
    for ci, bits in enumerate(CLASS_BITS):
        b = old_blocks.get(bits)
        if b is not None and b.size:
            b32 = b if b.dtype == np.int32 and b.flags.c_contiguous else np.ascontiguousarray(b, dtype=np.int32)
            hold.append(b32)
            ptrs[ci], cnts[ci] = addr(b32), b32.size
    targets = (C.c_int64 * len(counts_t))(*counts_t)
    out = np.empty(3 * total + 8, dtype=np.int32)   # counts (5, padded to 6), plan words (2 * total), survivors (total)
    counts, plan, alive = out[:5], out[6:6 + 2 * total], out[6 + 2 * total:6 + 3 * total]
    n_alive = C.c_int32(0)
    base = addr(out)
    rc = _lib.load().hqekv_plan_side(ptrs, cnts, hist_blocks, n_new_blocks, addr(order64), targets, len(counts_t),
                                     base, base + 24, base + 4 * (6 + 2 * total), C.byref(n_alive))
    if rc:
        return None
    u = n_alive.value
    return counts, plan[:2 * u], (alive[:u].astype(np.int64) if u < total else None)


_CLASS_SHAPES_K = {b: (lambda B, H, D, n, b=b: [(B, H, D, n)] if b == 16 else [(B, H, D, n * b // 32), (B, H, D, n // 32), (B, H, D, n // 32)]) for b in CLASS_BITS}
_CLASS_SHAPES_V = {b: (lambda B, H, D, n, b=b: [(B, H, n, D)] if b == 16 else [(B, H, n, D * b // 32), (B, H, n, D // 32), (B, H, n, D // 32)]) for b in CLASS_BITS}


def _numel(shape) -> int:
    n = 1
    for v in shape:
        n *= v
    return n


def _gather_side(is_k: bool, side: Dict[int, _Cls], new: torch.Tensor, counts, plan_words: np.ndarray,
                 strategy: str, plan_dev: Optional[torch.Tensor] = None) -> Dict[int, _Cls]:
    """Allocate the new classes of one side (one buffer per element type, the tensors are views of it) and fill
    them with one launch of the migration kernel.  ``plan_words`` (int32): per new block, the classes back to
    back, (source slot << 24) | source block, then every block's new block number; ``plan_dev``: the same words on
    the device when the caller has sent them already."""
    nb = plan_words.size // 2
    pos = plan_words[nb:].astype(np.int64)
    from . import _lib
    B, H, n_new, D = new.shape
    dev = new.device
    low_layout = _lib.LAYOUT_NORMAL1 if strategy == LOW_NORMAL else 0
    # ---- sources
    src = (_lib.CacheClass * (_SRC_NEW + 1))()
    keep = []
    for si, bits in enumerate(CLASS_BITS):
        c = side[bits]
        if c.data is None:
            continue
        data = c.data if c.data.is_contiguous() else c.data.contiguous()
        keep.append(data)
        e = src[si]
        e.bits, e.data = bits, data.data_ptr()
        e.n_tokens = (data.shape[3] * (1 if bits == 16 else 32 // bits)) if is_k else data.shape[2]
        if bits != 16:
            sc, zr = c.scale.contiguous(), c.zero.contiguous()
            keep += [sc, zr]
            e.scale, e.zero = sc.data_ptr(), zr.data_ptr()
            if bits == 1:
                e.layout = low_layout
    # the new tokens are the head of a longer (B, H, T, D) tensor when a residual follows them: read in place
    slab = n_new
    if new.is_contiguous():
        newc = new
    elif new.stride(3) == 1 and new.stride(2) == D and new.stride(1) % D == 0 and new.stride(0) == H * new.stride(1):
        newc, slab = new, new.stride(1) // D
    else:
        newc = new.contiguous()
    keep.append(newc)
    e = src[_SRC_NEW]
    e.bits, e.n_tokens, e.data, e.slab_tokens = 16, n_new, newc.data_ptr(), slab
    e.layout = _lib.LAYOUT_TOKEN_MAJOR if is_k else 0
    # ---- destinations: element counts per type, three allocations, views
    shapes_of = _CLASS_SHAPES_K if is_k else _CLASS_SHAPES_V
    todo, n16, n32, n64 = [], 0, 0, 0
    for ci, bits in enumerate(CLASS_BITS):
        n = int(counts[ci]) * BLOCK
        if n == 0:
            continue
        shp = shapes_of[bits](B, H, D, n)
        if bits == 16:
            todo.append((bits, n, shp, (n16,), n64))
            n16 += (_numel(shp[0]) + 127) // 128 * 128
        else:
            o_s = n16
            n16 += (_numel(shp[1]) + 127) // 128 * 128
            o_z = n16
            n16 += (_numel(shp[2]) + 127) // 128 * 128
            todo.append((bits, n, shp, (n32, o_s, o_z), n64))
            n32 += (_numel(shp[0]) + 63) // 64 * 64
        n64 += (n + 31) // 32 * 32
    out = {b: _Cls() for b in CLASS_BITS}
    if not todo:
        return out
    buf16 = torch.empty(max(n16, 1), dtype=torch.float16, device=dev)
    buf32 = torch.empty(max(n32, 1), dtype=torch.int32, device=dev)
    buf64 = torch.empty(n64, dtype=torch.int64, device=dev)

    def view(buf, shape, off):
        st, acc = [], 1
        for v in reversed(shape):
            st.append(acc)
            acc *= v
        return buf.as_strided(shape, st[::-1], off)

    dst = (_lib.CacheClass * len(CLASS_BITS))()
    n_dst, blk0 = 0, 0
    for bits, n, shp, offs, o_idx in todo:
        d = dst[n_dst]
        n_dst += 1
        idx_t = view(buf64, (n,), o_idx)
        if bits == 16:
            data = view(buf16, shp[0], offs[0])
            sc = zr = None
        else:
            data, sc, zr = view(buf32, shp[0], offs[0]), view(buf16, shp[1], offs[1]), view(buf16, shp[2], offs[2])
            d.scale, d.zero = sc.data_ptr(), zr.data_ptr()
            if bits == 1:
                d.layout = low_layout
        d.bits, d.n_tokens, d.data, d.idx = bits, n, data.data_ptr(), idx_t.data_ptr()
        idx_t._hq_blocks = pos[blk0:blk0 + n // BLOCK]
        idx_t._hq_host_version = idx_t._version
        blk0 += n // BLOCK
        out[bits] = _Cls(data, idx_t, sc, zr)
    plan = plan_dev if plan_dev is not None else \
        _to_dev(np.ascontiguousarray(plan_words).view(np.int64), dev).view(torch.int32)   # int32 pairs ride as int64
    with _lib.on_device(dev):
        # (no status word: this plan was made a few lines up from the classes it names; the kernel still checks it)
        rc = _lib.load().hqekv_cache_migrate(1 if is_k else 0, src, _SRC_NEW + 1, dst, n_dst, plan.data_ptr(), B * H, D,
                                             None, _lib.stream_ptr(dev))
    _lib.check(rc, "cache_migrate")
    # the kernel writes the position arrays behind torch's back: the version stamps taken above still hold, and the
    # host copies describe exactly what the kernel wrote
    return out


def _compress_gather(pkv: tuple, new_K, new_V, res_K, res_V, history: int, compress_length: int, K_sorted_idx,
                     K_bit_num, V_bit_num, V_norm, V_sorted_idx, last_weights, strategy: str, n_targets: int):
    """The whole compression as two gathers; -> new tuple, or None when the inputs are not made of whole blocks."""
    if strategy not in ("uniform_group", LOW_NORMAL) or new_K.device.type != "cuda":
        return None
    if not torch.is_tensor(K_bit_num) or not torch.is_tensor(V_bit_num) or K_bit_num.is_cuda or V_bit_num.is_cuda:
        return None
    total_blocks = (history + compress_length) // BLOCK
    hist_blocks, n_new_blocks = history // BLOCK, compress_length // BLOCK
    k_side, v_side = _read_side(pkv, K_SLOT), _read_side(pkv, V_SLOT)
    old = {}
    for name, side in (("k", k_side), ("v", v_side)):
        blocks = {}
        kept = 0
        for bits in CLASS_BITS:
            c = side[bits]
            if c.data is None:
                continue
            if c.idx is None:
                return None
            b = _host_blocks(c.idx)
            if b is None:
                return None
            blocks[bits] = b
            kept += b.size
        if kept != hist_blocks:
            return None
        old[name] = blocks
    # the two block rankings come down in one transfer when both carry theirs (and out of one sort call when neither
    # has been sorted yet)
    k_order_h = v_order_h = None
    if isinstance(K_sorted_idx, RankedBlocks) and isinstance(V_sorted_idx, RankedBlocks) \
            and K_sorted_idx.scores.numel() == total_blocks == V_sorted_idx.scores.numel() \
            and K_sorted_idx.scores.device == V_sorted_idx.scores.device:
        both = RankedBlocks.sort_together(K_sorted_idx, V_sorted_idx).to("cpu", torch.int64).numpy()
        k_order_h, v_order_h = both[0], both[1]
    k_ord = getattr(K_sorted_idx, "_hq_block_order", None) if k_order_h is None else None
    v_ord = getattr(V_sorted_idx, "_hq_block_order", None) if v_order_h is None else None

    def fresh(idx, ord_):   # the ranking that rides on a token list counts only while nobody has written into the list
        return (ord_ is not None and ord_[0].numel() == total_blocks
                and getattr(idx, "_hq_block_order_version", None) == idx._version)
    if k_order_h is not None:
        pass
    elif fresh(K_sorted_idx, k_ord) and fresh(V_sorted_idx, v_ord) and k_ord[0].device == v_ord[0].device:
        both = torch.stack((k_ord[0], v_ord[0])).to("cpu", torch.int64).numpy()
        k_order_h, v_order_h = both[0], both[1]
    elif fresh(V_sorted_idx, v_ord):
        v_order_h = v_ord[0].to("cpu", torch.int64).numpy()
    elif fresh(K_sorted_idx, k_ord):
        k_order_h = k_ord[0].to("cpu", torch.int64).numpy()
    if k_order_h is None:
        k_order_h = _host_blocks(K_sorted_idx)
    if v_order_h is None:
        v_order_h = _host_blocks(V_sorted_idx)
    k_plan = _plan_side_c(old["k"], hist_blocks, n_new_blocks, k_order_h, K_bit_num)
    v_plan = _plan_side_c(old["v"], hist_blocks, n_new_blocks, v_order_h, V_bit_num)
    if k_plan is None or v_plan is None:
        return None
    dev = new_V.device
    # one transfer for everything the device needs: both plans (int32 pairs riding as int64) and the positions of
    # the tokens that survive on the V side
    k_words, v_words, alive = k_plan[1], v_plan[1], v_plan[2]
    parts = [np.ascontiguousarray(k_words).view(np.int64), np.ascontiguousarray(v_words).view(np.int64)]
    if alive is not None:
        parts.append((alive[:, None] * BLOCK + np.arange(BLOCK, dtype=np.int64)).reshape(-1))
    sent = _to_dev(np.concatenate(parts), dev)
    n_kw, n_vw = parts[0].size, parts[1].size
    plan_dev = {"k": sent[:n_kw].view(torch.int32), "v": sent[n_kw:n_kw + n_vw].view(torch.int32)}
    sides = {}
    for name, is_k, side, new, (counts, words, _) in (("k", True, k_side, new_K, k_plan), ("v", False, v_side, new_V, v_plan)):
        sides[name] = _gather_side(is_k, side, new, counts, words, strategy, plan_dev[name])
    if alive is not None:   # evicted tokens leave the token ranges and the ring as well
        keep_t = sent[n_kw + n_vw:]
        V_norm = V_norm[keep_t]
        if last_weights is not None:
            last_weights.eviction(keep_t)
    t = list(pkv)
    _write_side(t, sides["k"], K_SLOT, dev)
    _write_side(t, sides["v"], V_SLOT, dev)
    t[38], t[39], t[40] = V_norm, res_K, res_V
    return tuple(t)


def compress(past_key_value: tuple, compress_length: int, history_length, K_sorted_idx: torch.Tensor,
             K_bit_num: torch.Tensor, V_bit_num: torch.Tensor, token_importance: torch.Tensor,
             quant_strategy: str, *, last_weights=None, block_size: int = 32, group_size: int = 32,
             times_range: bool = True, n_targets: int = 6, V_token_range: Optional[torch.Tensor] = None,
             engine: Optional[str] = None) -> tuple:
    """``engine``: None / "auto" = the one-launch-per-side gather when the selection is made of whole aligned blocks,
    else the step-by-step engine; "steps" forces the latter, "gather" raises when it does not apply (tests)."""
    if quant_strategy not in _STRATEGIES:
        raise ValueError('invalid quant_strategy')
    if block_size != BLOCK or group_size != BLOCK:
        raise ValueError("block_size and group_size must be 32")
    pkv = past_key_value
    new_K, new_V = pkv[39], pkv[40]
    if new_K is None or new_V is None:
        raise ValueError('invalid past_key_value')
    history = int(history_length)
    if compress_length % BLOCK or history % BLOCK:
        raise ValueError("compress_length and history_length must be multiples of 32")
    if K_bit_num.numel() != n_targets or V_bit_num.numel() != n_targets:
        raise ValueError(f"K_bit_num / V_bit_num must hold {n_targets} entries")
    whole = new_K.shape[2] == compress_length and new_V.shape[2] == compress_length   # nothing stays behind
    res_K = None if whole else _none_if_empty(new_K[:, :, compress_length:, :].clone())
    res_V = None if whole else _none_if_empty(new_V[:, :, compress_length:, :].clone())
    new_K, new_V = new_K[:, :, :compress_length, :], new_V[:, :, :compress_length, :]
    total = history + compress_length
    block_num = total // BLOCK

    V_norm = V_token_range if V_token_range is not None else calculate_token_range(new_V, pkv[38])
    # (the token list is spelt out only if the step engine runs)
    V_sorted_idx = rank_blocks_weighted(block_num, token_importance, V_norm if times_range else None)

    dev = new_V.device
    engine = engine or os.environ.get("HQEKV_POLICY_ENGINE", "auto")
    if engine not in ("auto", "gather", "steps"):
        raise ValueError("engine must be 'auto', 'gather' or 'steps'")
    if engine != "steps":
        done = _compress_gather(pkv, new_K, new_V, res_K, res_V, history, compress_length, K_sorted_idx, K_bit_num,
                                V_bit_num, V_norm, V_sorted_idx, last_weights, quant_strategy, n_targets)
        if done is not None:
            return done
        if engine == "gather":
            raise ValueError("the gather engine needs classes, rankings and counts made of whole aligned 32-token blocks")
    k_side, v_side = _read_side(pkv, K_SLOT, host=True), _read_side(pkv, V_SLOT, host=True)
    _migrate(k_side, new_K, _targets(K_sorted_idx, K_bit_num), history, True, quant_strategy)

    def after_v_eviction(side, new_idx):
        nonlocal V_norm
        keep = [side[b].idx_h for b in CLASS_BITS if side[b].idx_h is not None] + [new_idx]
        keep = _to_dev(np.sort(np.concatenate(keep)), dev)
        V_norm = V_norm[keep]
        if last_weights is not None:
            last_weights.eviction(keep)

    _migrate(v_side, new_V, _targets(V_sorted_idx, V_bit_num), history, False, quant_strategy,
             on_evict=after_v_eviction)

    t = list(pkv)
    _write_side(t, k_side, K_SLOT, dev)
    _write_side(t, v_side, V_SLOT, dev)
    t[38], t[39], t[40] = V_norm, res_K, res_V
    return tuple(t)


def reconstruct(past_key_value: tuple, quant_strategy: str, block_size: int = 32, group_size: int = 32):
    """Dequantise every class back into dense (B, H, kv_seq_len, D) fp16 K and V
    (quant/hybrid_quant.py:732-846, quant/hqe_2.py:967-1084).  Unlike the reference, the 4-bit V class
    is restored whether or not an 8-bit class exists, and the result is fp16 for any class mix."""
    if quant_strategy not in _STRATEGIES:
        raise ValueError('invalid quant_strategy')
    pkv = past_key_value
    k_side, v_side = _read_side(pkv, K_SLOT), _read_side(pkv, V_SLOT)
    new_K, new_V, T = pkv[39], pkv[40], int(pkv[41])
    some = next((x for x in (v_side[16].data, v_side[8].data, v_side[4].data, v_side[2].data, v_side[1].data, new_V) if x is not None), None)
    if some is None:
        raise ValueError('invalid past_key_value')
    B, H, dev = some.shape[0], some.shape[1], some.device
    if new_V is not None:
        D = new_V.shape[3]
    elif v_side[16].data is not None:
        D = v_side[16].data.shape[3]
    else:
        b = next(b for b in (8, 4, 2, 1) if v_side[b].data is not None)
        D = v_side[b].data.shape[3] * (32 // b)
    K = torch.zeros(B, H, T, D, dtype=torch.float16, device=dev)
    V = torch.zeros(B, H, T, D, dtype=torch.float16, device=dev)
    for b in CLASS_BITS:
        if b == 1 and (k_side[b].data is not None or v_side[b].data is not None):
            _check_low_bits(1, quant_strategy)
        if k_side[b].data is not None:
            K[:, :, k_side[b].idx, :] = _k_to_fp16(k_side[b], b, quant_strategy).transpose(2, 3)
        if v_side[b].data is not None:
            V[:, :, v_side[b].idx, :] = _v_to_fp16(v_side[b], b, quant_strategy)
    if new_K is not None:
        K[:, :, T - new_K.shape[2]:, :] = new_K
    if new_V is not None:
        V[:, :, T - new_V.shape[2]:, :] = new_V
    return K, V
