"""Host glue between the reference's 42-field cache tuple and the hybrid HIP launches.

The tuple layout is the reference's (quant/quant_matmul_hq.py:34-38):
  0 sixteen_K (B,Hkv,D,T16)  1 sixteen_K_idx  2 sixteen_V (B,Hkv,T16,D)  3 sixteen_V_idx
  K class b at base 4/12/20/28 (8/4/2/1 bit): code, idx, scale, zero;  V class at 8/16/24/32
  36 outliers  37 outliers_idx  38 V_token_norm  39 new_K (B,Hkv,Tn,D)  40 new_V  41 kv_seq_len
Each populated class becomes one ``hqekv_seg``; the kernels read the tensors where they lie.
"""
from __future__ import annotations

import ctypes as C
import os
import weakref
from typing import List, Optional, Tuple

import numpy as np
import torch

from . import _lib

BITS = (8, 4, 2, 1)   # 1: the uniform 1-bit class of the 'uniform_group' strategy (32 codes per word)
K_BASE = {8: 4, 4: 12, 2: 20, 1: 28}
V_BASE = {8: 8, 4: 16, 2: 24, 1: 32}
K16, K16_IDX, V16, V16_IDX = 0, 1, 2, 3
NEW_K, NEW_V, KV_SEQ_LEN = 39, 40, 41


def _idx(t: Optional[torch.Tensor], n: int, dev) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.dtype != torch.int64:
        t = t.to(torch.int64)
    if t.device != dev:
        t = t.to(dev)
    t = t.contiguous()
    if t.numel() != n:
        raise ValueError(f"index of length {t.numel()} for a class of {n} tokens")
    return t


def token_major_window(t: torch.Tensor):
    """An fp16 (B,H,n,D) tensor as the kernels read it: -> (tensor whose data_ptr is the first row, token rows between
    two (b, h) slabs or 0 when dense).  The head of a longer buffer -- ``buf[:, :, :n]`` of a capacity-sized residual
    buffer -- is read where it lies; anything else that is not dense is copied."""
    if t.is_contiguous():
        return t, 0
    B, H, n, D = t.shape
    sb, sh, st, sd = t.stride()
    if sd == 1 and st == D and sh % D == 0 and sh >= n * D and (B == 1 or sb == H * sh):
        return t, sh // D
    return t.contiguous(), 0


def ring_order(T: int, weights: torch.Tensor) -> int:
    """How torch's GPU reduction deals the 32 head rows of ``weights`` (B,32,1,T) to threads when it sums them: to two
    threads when rows are a multiple of 4 long, at least 256, and 8-byte aligned, else to one (measured on the
    device; ``hqekv_ring_row`` and the decode step reproduce either order bit for bit)."""
    return 2 if (T % 4 == 0 and T >= 256 and weights.data_ptr() % 8 == 0) else 1


def ring_row_on_device_applies(weights: torch.Tensor) -> bool:
    """Shapes for which the ring row's order is pinned against torch on the device."""
    return (weights.dtype == torch.float16 and weights.dim() == 4 and weights.shape[2] == 1 and weights.shape[1] == 32
            and weights.shape[0] <= 8 and weights.shape[3] >= 256 and weights.is_contiguous())


def _f16_k_item(k16: torch.Tensor, idx, keep: list) -> dict:
    """fp16 K class (B,Hkv,D,T): read channel-major, or token-major if it is a transposed view."""
    B, H, D, T = k16.shape
    if k16.is_contiguous():
        data, tm = k16, 0
    elif k16.stride(2) == 1 and k16.transpose(2, 3).is_contiguous():
        data, tm = k16, 1  # memory is (B,Hkv,T,D)
    else:
        data, tm = k16.contiguous(), 0
    keep.append(data)
    return dict(bits=16, n_tokens=T, data=data, idx=idx, token_major=tm)


def key_segments(pkv: tuple, dev, Tall: int, keep: list, low_uniform: bool = True,
                 residual: bool = True) -> Tuple[List[dict], int, int]:
    """K classes of the tuple in launch order; ``residual=False`` leaves out ``new_K`` (the only segment
    that changes between two compressions)."""
    items = []
    nh_kv = D = None
    if pkv[K16] is not None:
        k = pkv[K16]
        nh_kv, D = k.shape[1], k.shape[2]
        items.append(_f16_k_item(k, _idx(pkv[K16_IDX], k.shape[3], dev), keep))
    for b in BITS:
        base = K_BASE[b]
        if pkv[base] is not None:
            code = pkv[base].contiguous()
            sc, zr = pkv[base + 2].contiguous(), pkv[base + 3].contiguous()
            n = code.shape[3] * (32 // b)
            nh_kv, D = code.shape[1], code.shape[2]
            idx = _idx(pkv[base + 1], n, dev)
            keep += [code, sc, zr, idx]
            # the 1-bit class holds (std, mean) and normal-quantile codes unless the strategy is 'uniform_group'
            layout = _lib.LAYOUT_NORMAL1 if (b == 1 and not low_uniform) else 0
            items.append(dict(bits=b, n_tokens=n, data=code, scale=sc, zero=zr, idx=idx, layout=layout))
    new_K = pkv[NEW_K]
    if residual and new_K is not None and new_K.shape[2] > 0:
        nk, slab = token_major_window(new_K)
        keep.append(nk)
        nh_kv, D = nk.shape[1], nk.shape[3]
        n = nk.shape[2]
        items.append(dict(bits=16, n_tokens=n, data=nk, idx=None, pos_base=Tall - n, token_major=1, slab_tokens=slab))
    return items, nh_kv, D


def value_segments(pkv: tuple, dev, Tall: int, keep: list, low_uniform: bool = True,
                   residual: bool = True) -> Tuple[List[dict], int, int]:
    items = []
    nh_kv = D = None
    if pkv[V16] is not None:
        v = pkv[V16].contiguous()
        nh_kv, D = v.shape[1], v.shape[3]
        idx = _idx(pkv[V16_IDX], v.shape[2], dev)
        keep += [v, idx]
        items.append(dict(bits=16, n_tokens=v.shape[2], data=v, idx=idx))
    for b in BITS:
        base = V_BASE[b]
        if pkv[base] is not None:
            code = pkv[base].contiguous()
            sc, zr = pkv[base + 2].contiguous(), pkv[base + 3].contiguous()
            n = code.shape[2]
            nh_kv, D = code.shape[1], code.shape[3] * (32 // b)
            idx = _idx(pkv[base + 1], n, dev)
            keep += [code, sc, zr, idx]
            # the 1-bit class holds (std, mean) and normal-quantile codes unless the strategy is 'uniform_group'
            layout = _lib.LAYOUT_NORMAL1 if (b == 1 and not low_uniform) else 0
            items.append(dict(bits=b, n_tokens=n, data=code, scale=sc, zero=zr, idx=idx, layout=layout))
    new_V = pkv[NEW_V]
    if residual and new_V is not None and new_V.shape[2] > 0:
        nv, slab = token_major_window(new_V)
        keep.append(nv)
        nh_kv, D = nv.shape[1], nv.shape[3]
        n = nv.shape[2]
        items.append(dict(bits=16, n_tokens=n, data=nv, idx=None, pos_base=Tall - n, slab_tokens=slab))
    return items, nh_kv, D


def value_length(pkv: tuple) -> int:
    """Sum of the V class lengths plus the residual (quant/hqe_matmul.py:379-402)."""
    n = 0
    if pkv[V16] is not None:
        n += pkv[V16].shape[2]
    for b in (8, 4, 2, 1):
        if pkv[V_BASE[b]] is not None:
            n += pkv[V_BASE[b]].shape[2]
    if pkv[NEW_V] is not None:
        n += pkv[NEW_V].shape[2]
    return n


def idx_cover_once(idx_list, n: int) -> bool:
    """True when the class position arrays, taken together, hold every position in [0, n) exactly once -- what
    the softmax fused into the two GEMV launches relies on (a position nobody writes keeps whatever the score
    buffer held, one written twice is counted twice).  Arrays that carry a host copy (the cache policy's) are
    checked there; others on the device, which waits for it once: the verdict is remembered per set of tensors
    until one of them is written to."""
    idx_list = [t for t in idx_list if t is not None]
    if sum(int(t.numel()) for t in idx_list) != n:
        return False
    if not idx_list:
        return True
    # The verdict rides on the first array and names the others by weak reference: it holds while these very tensor
    # objects are alive, sit where they sat and have not been written through torch since.  (A kernel that writes an
    # array through its raw pointer does not show here: whoever launches one drops `_hq_cover` from the array.)
    key = tuple((t.data_ptr(), int(t.numel()), t._version) for t in idx_list) + (n,)
    hit = getattr(idx_list[0], "_hq_cover", None)
    if hit is not None and hit[0] == key and len(hit[2]) == len(idx_list) and all(r() is t for r, t in zip(hit[2], idx_list)):
        return hit[1]
    trusted = [getattr(t, "_hq_host_version", None) == t._version for t in idx_list]
    blocks = [getattr(t, "_hq_blocks", None) if ok_ else None for t, ok_ in zip(idx_list, trusted)]
    hosts = [getattr(t, "_hq_host", None) if ok_ else None for t, ok_ in zip(idx_list, trusted)]
    if n % 32 == 0 and all(b is not None and b.shape[0] * 32 == t.numel() for b, t in zip(blocks, idx_list)):
        c = np.concatenate(blocks)   # whole aligned 32-token blocks: check the block numbers
        nb = n // 32
        ok = bool(c.size == nb and (c >= 0).all() and (c < nb).all() and (np.bincount(c, minlength=nb) == 1).all())
    elif all(h is not None for h in hosts):
        c = np.concatenate(hosts)
        ok = bool(c.size == n and (c >= 0).all() and (c < n).all() and (np.bincount(c, minlength=n) == 1).all())
    else:
        c = torch.cat([t.reshape(-1).to(torch.int64) for t in idx_list])
        inside = (c >= 0) & (c < n)
        ok = bool(inside.all() & (torch.bincount(c.clamp(0, n - 1), minlength=n) == 1).all())
    idx_list[0]._hq_cover = (key, ok, [weakref.ref(t) for t in idx_list])
    return ok


def _class_idx(pkv: tuple, base0: int, bases) -> list:
    """Position arrays of the populated classes of one side."""
    out = [pkv[base0 + 1]] if pkv[base0] is not None else []
    return out + [pkv[bases[b] + 1] for b in BITS if pkv[bases[b]] is not None]


def classes_partition_positions(pkv: tuple) -> bool:
    """Both sides' classes cover [0, kept) exactly once each, kept = tokens held by the V classes."""
    v_idx = _class_idx(pkv, V16, V_BASE)
    n = sum(int(t.numel()) for t in v_idx if t is not None)
    if any(t is None for t in v_idx):
        return False
    k_idx = _class_idx(pkv, K16, K_BASE)
    if any(t is None for t in k_idx):
        return False
    return idx_cover_once(k_idx, n) and idx_cover_once(v_idx, n)


def _mask_arg(mask, B: int, Hq: int, Tall: int, dev, keep: list):
    """-> (pointer or None, row stride in elements) for an additive fp16 mask."""
    if mask is None:
        return None, 0
    if not torch.is_tensor(mask):
        if float(mask) == 0.0:
            return None, 0
        mask = torch.full((1, 1, 1, Tall), float(mask), dtype=torch.float16, device=dev)
    mask = mask.to(device=dev, dtype=torch.float16)
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    if mask.shape[-1] != Tall or mask.shape[-2] != 1:
        mask = mask.expand(*mask.shape[:-2], 1, Tall) if mask.shape[-1] in (1, Tall) else mask
        if mask.shape[-1] != Tall:
            raise ValueError(f"mask last dim {mask.shape[-1]} != {Tall}")
    if mask.shape[0] == 1 and mask.shape[1] == 1:
        m = mask.reshape(Tall).contiguous()
        keep.append(m)
        return m.data_ptr(), 0
    m = mask.expand(B, Hq, 1, Tall).contiguous()
    keep.append(m)
    return m.data_ptr(), Tall


def workspace_for(v_segs, n_v: int, B: int, Hq: int, Hkv: int, D: int, dev) -> torch.Tensor:
    """Split-K workspace of a stand-alone p.V launch."""
    need = _lib.load().hqekv_pv_workspace_bytes(v_segs, n_v, B, Hq, Hkv, D)
    if need < 0:
        raise ValueError("invalid segment table")
    return torch.empty(max(need, 16) // 4, dtype=torch.float32, device=dev)


def decode_workspace(k_segs, n_k: int, v_segs, n_v: int, B: int, Hq: int, Hkv: int, D: int, dev) -> torch.Tensor:
    """Workspace of a whole decode-attention call (split-K partials and per-tile softmax statistics)."""
    need = _lib.load().hqekv_decode_workspace_bytes(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D)
    if need < 0:
        raise ValueError("invalid segment table")
    return torch.empty(max(need, 256) // 4, dtype=torch.float32, device=dev)


_environ = os.environ   # (attribute lookups on the module are the slow part of this per-step call)


def default_flags() -> int:
    """Fuse the softmax into the two GEMV launches unless HQEKV_UNFUSED=1 asks for the general path."""
    return 0 if _environ.get("HQEKV_UNFUSED") == "1" else _lib.FUSE_SOFTMAX


class SegmentMemo:
    """One layer's segment tables between two compressions.  Fields 0..38 of the tuple (the classes) stay
    the same tensor objects from one decode step to the next -- the caller only replaces ``new_K``,
    ``new_V`` and the length -- so their table entries are built once and only the residual entry is
    rewritten per step.  The memo holds the class tensors it points into; it is valid for a tuple whose
    first 39 fields ARE the held objects, and rebuilt otherwise.  The workspace is kept as well (calls of
    one layer are ordered on one stream)."""

    def __init__(self):
        self.held: Optional[tuple] = None      # fields 0..38 of the tuple the tables were built from
        self.key = None                        # (device, low_uniform) they were built for
        self.ws: Optional[torch.Tensor] = None
        self.keep: list = []                   # converted / made-contiguous tensors the tables point into
        self.k_arr = self.v_arr = None         # ctypes arrays of hqekv_seg with one spare entry each
        self.n_k = self.n_v = 0
        self.Hkv = None
        self.dims = (None, None)
        self.partition = False                 # the classes' position arrays cover [0, kept) once per side
        self._step = None                      # what step_call keeps between steps
        self._spare = None                     # (attn_weights, attn_output) allocated ahead for the next step

    def lookup(self, pkv: tuple, dev, low_uniform: bool) -> bool:
        held = self.held
        if held is None or self.key != (dev, low_uniform):
            return False
        for a, b in zip(held, pkv):  # zip stops after the 39 held fields
            if a is not b:
                return False
        return True

    def build(self, pkv: tuple, dev, low_uniform: bool) -> None:
        self.keep = []
        k_items, hk, dk = key_segments(pkv, dev, 0, self.keep, low_uniform, residual=False)
        v_items, hv, dv = value_segments(pkv, dev, 0, self.keep, low_uniform, residual=False)
        if len(k_items) + 2 > _lib.MAX_SEGS or len(v_items) + 2 > _lib.MAX_SEGS:
            raise ValueError("too many segments")
        self.n_k, self.n_v = len(k_items), len(v_items)
        self.k_arr = (_lib.Seg * (self.n_k + 2))()   # two spare entries each: the residual and the step's new token
        self.v_arr = (_lib.Seg * (self.n_v + 2))()
        for dst, src in ((self.k_arr, _lib.make_segs(k_items)), (self.v_arr, _lib.make_segs(v_items))):
            for i in range(len(dst) - 2):
                C.memmove(C.byref(dst[i]), C.byref(src[i]), C.sizeof(_lib.Seg))
        self.need = {}                                # workspace bytes per (residual, tail, B, Hq) of this cache
        self.Hkv = hk if hk is not None else hv
        self.dims = (dk, dv)
        self.held = tuple(pkv[:NEW_K])
        self.key = (dev, low_uniform)
        self.partition = classes_partition_positions(pkv)
        self._step = None

    @staticmethod
    def _fill(s, t: torch.Tensor, end: int, layout: int, keep: list):
        """Table entry of an fp16 token-major block (B,Hkv,n,D) whose last token sits at position end - 1."""
        tc, slab = token_major_window(t)
        keep.append(tc)
        n = tc.shape[2]
        s.bits, s.layout, s.n_tokens, s.pos_base, s.data, s.slab_tokens = 16, layout, n, end - n, tc.data_ptr(), slab
        return tc.shape[1], tc.shape[3]

    def tables(self, pkv: tuple, Tall: int, keep: list, tail=None):
        """-> (k_segs, n_k, v_segs, n_v, Hkv, (dk, dv), (residual tokens, tail tokens)) with this step's residual
        -- and the tokens of ``tail`` = (k, v), which follow it -- filled in."""
        n_k, n_v, Hkv, (dk, dv) = self.n_k, self.n_v, self.Hkv, self.dims
        n_tail = tail[0].shape[2] if tail is not None else 0
        n_res = 0
        new_K, new_V = pkv[NEW_K], pkv[NEW_V]
        if new_K is not None and new_K.shape[2] > 0:
            n_res = new_K.shape[2]
            Hkv, dk = self._fill(self.k_arr[n_k], new_K, Tall - n_tail, _lib.LAYOUT_TOKEN_MAJOR, keep)
            n_k += 1
        if new_V is not None and new_V.shape[2] > 0:
            Hkv, dv = self._fill(self.v_arr[n_v], new_V, Tall - n_tail, 0, keep)
            n_v += 1
        if n_tail:
            Hkv, dk = self._fill(self.k_arr[n_k], tail[0], Tall, _lib.LAYOUT_TOKEN_MAJOR, keep)
            Hkv, dv = self._fill(self.v_arr[n_v], tail[1], Tall, 0, keep)
            n_k += 1
            n_v += 1
        return self.k_arr, n_k, self.v_arr, n_v, Hkv, (dk, dv), (n_res, n_tail)

    def workspace(self, need: int, dev) -> torch.Tensor:
        if self.ws is None or self.ws.numel() * 4 < need or self.ws.device != dev:
            self.ws = torch.empty(max(need + need // 8, 256) // 4, dtype=torch.float32, device=dev)
        return self.ws

    SPARE_MAX_BYTES = 4 << 20   # largest attn_weights tensor that is allocated one step ahead

    def step_call(self, q: torch.Tensor, pkv: tuple, Tall: int, k: torch.Tensor, v: torch.Tensor, res, n: int,
                  ring_store: Optional[torch.Tensor], ring_row: int, low_uniform: bool, known: bool = False):
        """One decode step of a layer as one C call (``hqekv_decode_step``) with as little host work as the call
        allows: the class entries of the tables are the memo's, the residual is the first ``n`` token rows of the
        capacity buffers ``res`` = (K, V), this step's ``k`` / ``v`` (B,Hkv,L,D, dense) are read as a segment of
        their own and copied to row ``n`` of the buffers, and -- when ``ring_store`` (rows x max_length, fp16) is
        given -- row ``ring_row`` of it receives the ring row.  ``known``: the caller vouches that ``pkv`` carries the
        class tensors the tables were built from (it is the tuple the previous step returned).
        -> (attn_weights, attn_output)."""
        dev = q.device
        if not (known and self.held is not None) and not self.lookup(pkv, dev, low_uniform):
            self.build(pkv, dev, low_uniform)
        B, Hq, _, D = q.shape
        Hkv, L = k.shape[1], k.shape[2]
        kbuf, vbuf = res
        st = self._step
        if st is None or st[0] is not kbuf:
            # entries that stay the same from step to step: the residual's (bits, layout, data, slab), the tail's
            # (bits, layout), and the appends' slab lengths
            for arr, base, buf, layout in ((self.k_arr, self.n_k, kbuf, _lib.LAYOUT_TOKEN_MAJOR), (self.v_arr, self.n_v, vbuf, 0)):
                for j in (0, 1):
                    e = arr[base + j]
                    e.bits, e.layout, e.scale, e.zero, e.idx, e.slab_tokens = 16, layout, None, None, None, 0
            x = _lib.StepExtra()
            x.k_dst_slab_tokens, x.v_dst_slab_tokens = kbuf.shape[2], vbuf.shape[2]
            st = self._step = (kbuf, x, kbuf.data_ptr(), vbuf.data_ptr(), kbuf.shape[2])
        _, x, kptr, vptr, cap = st
        n_k, n_v = self.n_k, self.n_v
        ka, va = self.k_arr, self.v_arr
        if n:
            e = ka[n_k]
            e.n_tokens, e.pos_base, e.data, e.slab_tokens = n, Tall - L - n, kptr, cap
            e = va[n_v]
            e.n_tokens, e.pos_base, e.data, e.slab_tokens = n, Tall - L - n, vptr, cap
            n_k += 1
            n_v += 1
        e = ka[n_k]
        e.n_tokens, e.pos_base, e.data, e.slab_tokens = L, Tall - L, k.data_ptr(), 0
        e = va[n_v]
        e.n_tokens, e.pos_base, e.data, e.slab_tokens = L, Tall - L, v.data_ptr(), 0
        n_k += 1
        n_v += 1
        # (positions nobody writes must read as zero when the classes do not cover every position)
        spare, self._spare = self._spare, None
        if spare is not None and self.partition and spare[0].shape == (B, Hq, 1, Tall) and spare[1].shape == (B, Hq, 1, D) \
                and spare[0].device == dev:
            weights, out = spare   # allocated while the previous step's kernels were running
        else:
            weights = (torch.empty if self.partition else torch.zeros)(B, Hq, 1, Tall, dtype=torch.float16, device=dev)
            out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=dev)
        if ring_store is not None:
            x.ring_line = ring_store.data_ptr() + 2 * ring_row * ring_store.shape[1]
            x.ring_order = 2 if (Tall % 4 == 0 and Tall >= 256 and weights.data_ptr() % 8 == 0) else 1
        else:
            x.ring_line = None
        row_bytes = 2 * D
        x.append_rows, x.new_k, x.new_v = L, k.data_ptr(), v.data_ptr()
        x.k_dst, x.v_dst = kptr + n * row_bytes, vptr + n * row_bytes
        flags = default_flags() if self.partition else 0
        lib = _lib.load()
        ws = self.ws
        with _lib.on_device(dev):
            for attempt in (0, 1):
                if ws is None or attempt:
                    need = lib.hqekv_decode_workspace_bytes(ka, n_k, va, n_v, B, Hq, Hkv, D)
                    if need < 0:
                        raise ValueError("invalid segment table")
                    ws = self.workspace(2 * need, dev)   # room for the residual to grow without asking again
                rc = lib.hqekv_decode_step(ka, n_k, va, n_v, q.data_ptr(), None, 0, weights.data_ptr(), out.data_ptr(),
                                           B, Hq, Hkv, D, Tall, ws.data_ptr(), ws.numel() * 4, flags,
                                           _lib.stream_ptr(dev), C.byref(x))
                if rc != -3:   # HQEKV_E_WORKSPACE: the cache has outgrown the workspace kept from earlier steps
                    break
        _lib.check(rc, "decode_step")
        # The next step's outputs, one position longer, allocated now: off that step's path to its first launch.  Only
        # while they are small (every layer of a model holds its own): a long step does not notice the allocation.
        if self.partition and B * Hq * (Tall + L) * 2 <= self.SPARE_MAX_BYTES:
            self._spare = (torch.empty(B, Hq, 1, Tall + L, dtype=torch.float16, device=dev),
                           torch.empty(B, Hq, 1, D, dtype=torch.float16, device=dev))
        return weights, out


def decode_attention(q: torch.Tensor, pkv: tuple, mask, Tall: int, zero_init: bool, flags: Optional[int] = None,
                     low_uniform: bool = True, memo: Optional[SegmentMemo] = None, tail=None, step=None):
    """q (B,Hq,1,D) fp16 -> (attn_weights (B,Hq,1,Tall) fp16 probabilities, attn_output (B,Hq,1,D) fp16).

    One q.K^T launch over all K classes and one p.V launch over all V classes with the softmax fused
    into them; or, with a mask / an incomplete cover of the positions / ``flags=0``, the general path
    (q.K^T, scale+mask+clamp+softmax, p.V, fixed-order combine).  Runs on torch's current stream.
    ``memo``: a ``SegmentMemo`` the caller keeps per layer, so that steps between two compressions rebuild
    only the residual's table entry.
    ``tail`` = (k, v), each (B,Hkv,L,D) fp16: tokens that follow the tuple's residual without being part of it yet
    (``Tall`` counts them).  The kernels read them as one more fp16 segment per side, so a caller can start the
    attention of a decode step before it appends the step's key and value to the residual.
    ``step``: what the caller's decode step does around the attention, folded into the call's last launch
    (``hqekv_decode_step``): ``step["ring_line"]`` = a (Tall,) fp16 view that receives ``attn_weights.sum(0).sum(0)``
    in torch's order (only for shapes ``ring_row_on_device_applies`` covers; the caller checks), ``step["append"]`` =
    (K buffer, V buffer, n): the rows of ``tail`` are copied to token row n of the (B,Hkv,cap,D) buffers.
    """
    _lib.require_gpu(q, "q")
    if q.dtype != torch.float16:
        raise TypeError("q must be float16 (the cache is fp16 by definition)")
    if q.dim() != 4 or q.shape[2] != 1:
        raise ValueError("q must be (B, Hq, 1, D): only single-token decode is computed")
    B, Hq, _, D = q.shape
    dev = q.device
    keep: list = []
    use_flags = default_flags() if flags is None else flags
    if memo is not None:
        if not memo.lookup(pkv, dev, low_uniform):
            memo.build(pkv, dev, low_uniform)
        k_segs, n_k, v_segs, n_v, Hkv, (dk, dv), res_tail = memo.tables(pkv, Tall, keep, tail)
        covered = memo.partition
    else:
        covered = not (use_flags & _lib.FUSE_SOFTMAX) or mask is not None or classes_partition_positions(pkv)
    if not covered:   # a position nobody writes must read as zero, and the fused softmax must not run
        use_flags &= ~_lib.FUSE_SOFTMAX
        zero_init = True
    if memo is None:
        n_tail = tail[0].shape[2] if tail is not None else 0
        k_items, hk, dk = key_segments(pkv, dev, Tall - n_tail, keep, low_uniform)
        v_items, hv, dv = value_segments(pkv, dev, Tall - n_tail, keep, low_uniform)
        if n_tail:
            tk, tv = tail[0].contiguous(), tail[1].contiguous()
            keep += [tk, tv]
            k_items.append(dict(bits=16, n_tokens=n_tail, data=tk, idx=None, pos_base=Tall - n_tail, token_major=1))
            v_items.append(dict(bits=16, n_tokens=n_tail, data=tv, idx=None, pos_base=Tall - n_tail))
            hk, dk, hv, dv = tk.shape[1], tk.shape[3], tv.shape[1], tv.shape[3]
        Hkv = hk if hk is not None else hv
        k_segs, v_segs, n_k, n_v = _lib.make_segs(k_items), _lib.make_segs(v_items), len(k_items), len(v_items)
    if Hkv is None:
        raise ValueError("invalid past_key_value")
    for d_ in (dk, dv):
        if d_ is not None and d_ != D:
            raise ValueError("head_dim of the cache does not match q")
    qc = q.contiguous()
    weights = (torch.zeros if zero_init else torch.empty)(B, Hq, 1, Tall, dtype=torch.float16, device=dev)
    out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=dev)
    mptr, mstride = _mask_arg(mask, B, Hq, Tall, dev, keep)
    lib = _lib.load()
    with _lib.on_device(dev):
        if memo is not None:
            need_key = (res_tail, B, Hq)
            need = memo.need.get(need_key)
            if need is None:
                need = memo.need[need_key] = lib.hqekv_decode_workspace_bytes(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D)
            if need < 0:
                raise ValueError("invalid segment table")
            ws = memo.workspace(need, dev)
        else:
            ws = decode_workspace(k_segs, n_k, v_segs, n_v, B, Hq, Hkv, D, dev)
        if step is None:
            rc = lib.hqekv_decode_attn(
                k_segs, n_k, v_segs, n_v, qc.data_ptr(), mptr, mstride,
                weights.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, Tall, ws.data_ptr(), ws.numel() * 4,
                use_flags, _lib.stream_ptr(dev))
        else:
            x = _lib.StepExtra()
            line = step.get("ring_line")
            if line is not None:
                x.ring_line, x.ring_order = line.data_ptr(), ring_order(Tall, weights)
            app = step.get("append")
            if app is not None:
                kbuf, vbuf, n = app
                tk, tv = tail[0].contiguous(), tail[1].contiguous()
                keep += [tk, tv]
                x.append_rows, x.new_k, x.new_v = tk.shape[2], tk.data_ptr(), tv.data_ptr()
                x.k_dst, x.v_dst = kbuf[0, 0, n].data_ptr(), vbuf[0, 0, n].data_ptr()
                x.k_dst_slab_tokens, x.v_dst_slab_tokens = kbuf.shape[2], vbuf.shape[2]
            rc = lib.hqekv_decode_step(
                k_segs, n_k, v_segs, n_v, qc.data_ptr(), mptr, mstride,
                weights.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, Tall, ws.data_ptr(), ws.numel() * 4,
                use_flags, _lib.stream_ptr(dev), C.byref(x))
    _lib.check(rc, "decode_attention")
    return weights, out


class DecodePlan:
    """Pre-validated launch plan for one layer's cache: segment tables, outputs and the split-K
    workspace are built once, so a decode step is a single C call (three kernel launches plus the
    combine) with no per-step Python work.  Holds references to every tensor it points into.
    """

    def __init__(self, q_like: torch.Tensor, pkv: tuple, mask=None, Tall: Optional[int] = None,
                 flags: Optional[int] = None, low_uniform: bool = True):
        _lib.require_gpu(q_like, "q")
        B, Hq, _, D = q_like.shape
        self.dev = q_like.device
        self.Tall = int(Tall) if Tall is not None else value_length(pkv)
        self._keep: list = []
        k_items, hk, _ = key_segments(pkv, self.dev, self.Tall, self._keep, low_uniform)
        v_items, hv, _ = value_segments(pkv, self.dev, self.Tall, self._keep, low_uniform)
        self.Hkv = hk if hk is not None else hv
        if self.Hkv is None:
            raise ValueError("invalid past_key_value")
        self.B, self.Hq, self.D = B, Hq, D
        self.n_k, self.n_v = len(k_items), len(v_items)
        self.k_segs, self.v_segs = _lib.make_segs(k_items), _lib.make_segs(v_items)
        self.weights = torch.zeros(B, Hq, 1, self.Tall, dtype=torch.float16, device=self.dev)
        self.out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=self.dev)
        self.mask_ptr, self.mask_stride = _mask_arg(mask, B, Hq, self.Tall, self.dev, self._keep)
        with _lib.on_device(self.dev):
            self.ws = decode_workspace(self.k_segs, self.n_k, self.v_segs, self.n_v, B, Hq, self.Hkv, D, self.dev)
        self.flags = default_flags() if flags is None else flags
        if (self.flags & _lib.FUSE_SOFTMAX) and mask is None and not classes_partition_positions(pkv):
            self.flags &= ~_lib.FUSE_SOFTMAX   # weights is zero-initialised above: uncovered positions stay 0
        self._lib = _lib.load()
        self.inv_sqrt_d = 1.0 / (D ** 0.5)

    def run(self, q: torch.Tensor, stream: Optional[int] = None, only: int = 0):
        """``only`` = _lib.ONLY_QK / ONLY_PV / ONLY_COMBINE runs one part of the step (per-kernel timing)."""
        st = _lib.stream_ptr(self.dev) if stream is None else stream
        rc = self._lib.hqekv_decode_attn(
            self.k_segs, self.n_k, self.v_segs, self.n_v, q.data_ptr(), self.mask_ptr, self.mask_stride,
            self.weights.data_ptr(), self.out.data_ptr(), self.B, self.Hq, self.Hkv, self.D, self.Tall,
            self.ws.data_ptr(), self.ws.numel() * 4, self.flags | only, st)
        if rc:
            _lib.check(rc, "DecodePlan.run")
        return self.weights, self.out

    # the three stages on their own, for per-kernel timing
    def run_qk(self, q: torch.Tensor, stream: Optional[int] = None):
        st = _lib.stream_ptr(self.dev) if stream is None else stream
        _lib.check(self._lib.hqekv_qk_hybrid(self.k_segs, self.n_k, q.data_ptr(), self.weights.data_ptr(), self.B,
                                             self.Hq, self.Hkv, self.D, self.Tall, st), "run_qk")

    def run_softmax(self, stream: Optional[int] = None):
        st = _lib.stream_ptr(self.dev) if stream is None else stream
        _lib.check(self._lib.hqekv_scale_softmax(self.weights.data_ptr(), self.mask_ptr, self.mask_stride,
                                                 self.B * self.Hq, self.Tall, self.inv_sqrt_d, st), "run_softmax")

    def run_pv(self, stream: Optional[int] = None):
        st = _lib.stream_ptr(self.dev) if stream is None else stream
        _lib.check(self._lib.hqekv_pv_hybrid(self.v_segs, self.n_v, self.weights.data_ptr(), self.out.data_ptr(),
                                             self.B, self.Hq, self.Hkv, self.D, self.Tall, self.ws.data_ptr(),
                                             self.ws.numel() * 4, st), "run_pv")
