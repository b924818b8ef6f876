"""The second caller of the path in the reference: its KIVI-style attention (``LlamaAttention.forward`` of
model/llama_kivi.py:96-266; model/qwen3_kivi.py has the same cache logic), without the projections, the
rotary embedding and ``o_proj``.  Every token is kept: K is quantised per channel in blocks of
``residual_length`` tokens, V per token one token at a time, both with an fp16 tail.

Cache tuple, as upstream (model/llama_kivi.py:266):
  0 K codes (B,Hkv,D,Tq/pf) int32   1 K fp16 tail (B,Hkv,r,D)   2 K scale (B,Hkv,D,Tq/32)   3 K zero
  4 V codes (B,Hkv,Tv,D/pf) int32   5 V fp16 tail (B,Hkv,r',D)  6 V scale (B,Hkv,Tv,D/32)   7 V zero
  8 kv_seq_len

Upstream attends with two per-class GEMVs plus two dense matmuls over the tails, a concatenation, the
softmax and an addition (:130-188).  Here a decode step is ONE hybrid launch sequence (q.K^T over the
quantised class and the tail, softmax fused, p.V over both, combine): the tuple's fields are handed to the
hybrid kernels as two segments per side, where they lie.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .attention import K_BASE, NEW_K, NEW_V, V_BASE, SegmentMemo, decode_attention, default_flags
from .decode_layer import gqa_prompt_attention
from .pack_unpack import uniform_group_quantize_pack_last_dim


class _Buffers:
    """What a ``KiviAttentionLayer`` keeps between decode steps: the K class tensors, the K tail in a buffer of
    ``residual_length`` rows, the V tail as a window [v0, v0 + nv) of a longer buffer, the V class in capacity buffers,
    and the tuple (views of all this) it handed out last."""
    __slots__ = ("kq", "ks", "kz", "kt", "nk", "vt", "cap_vt", "v0", "nv", "vcode", "vscale", "vzero", "n_vq", "returned",
                 "extra")

    def __init__(self):
        self.returned = None
        self.extra = _lib.StepExtra()


class KiviAttentionLayer:
    """``k_bits``/``v_bits`` in {1, 2, 4, 8}; ``group_size`` 32; ``residual_length`` a multiple of 32
    (upstream: 2, 2, 32, 128 -- model/llama_kivi.py:72-76)."""

    MIN_V_ROWS = 1024   # least capacity (token rows) of the V class buffers of the in-place decode step

    def __init__(self, head_dim: int, k_bits: int = 2, v_bits: int = 2, group_size: int = 32,
                 residual_length: int = 128):
        if group_size != 32:
            raise ValueError("group_size must be 32")
        if residual_length <= 0 or residual_length % group_size:
            raise ValueError("residual_length must be a positive multiple of the group size")
        if k_bits not in K_BASE or v_bits not in V_BASE:
            raise ValueError("k_bits and v_bits must be 1, 2, 4 or 8")
        self.head_dim, self.k_bits, self.v_bits = head_dim, k_bits, v_bits
        self.group_size, self.residual_length = group_size, residual_length
        self.scaling = head_dim ** -0.5
        self._memo = SegmentMemo()
        self._k_segs = (_lib.Seg * 3)()   # (quantised class, fp16 tail, this step's token) of each side, rewritten every step
        self._v_segs = (_lib.Seg * 3)()
        self._ws: Optional[torch.Tensor] = None
        self._st = None                   # buffers behind the tuple this layer handed out last (see _Buffers)
        self.in_place = True              # decode steps append in capacity buffers (False: upstream's cat / slice sequence)

    # ------------------------------------------------------------------ prompt
    def _prefill(self, q, k, v, attention_mask):
        n_rep = q.shape[1] // k.shape[1]
        T, R = k.shape[-2], self.residual_length
        out = gqa_prompt_attention(q, k, v, attention_mask, self.scaling)   # grouped heads: no repeat_kv copies
        tail = T % R
        k_quant = k if tail == 0 else (k[:, :, :T - tail, :] if T >= R else None)
        k_full = None if tail == 0 else k[:, :, T - tail:, :].contiguous()
        kq = ks = kz = None
        if k_quant is not None:
            # (B,Hkv,D,T) view of token-major memory: the quantiser reads it in place
            kq, ks, kz = uniform_group_quantize_pack_last_dim(k_quant.transpose(2, 3), self.group_size, self.k_bits)
        if T <= R:
            vq, v_full, vs, vz = None, v, None, None
        else:
            v_full = v[:, :, T - R:, :].contiguous()
            vq, vs, vz = uniform_group_quantize_pack_last_dim(v[:, :, :T - R, :].contiguous(), self.group_size,
                                                              self.v_bits)
        return out, (kq, k_full, ks, kz, vq, v_full, vs, vz)

    # ------------------------------------------------------------------ decode attention
    def _attend(self, q, kq, ks, kz, k_full, vq, vs, vz, v_full, T: int):
        """The step's attention straight from the tuple's fields: per side the quantised class at positions
        [0, n) and the fp16 tail behind it -- two table entries whose pointers and lengths are rewritten in place
        (the class tensors are new objects after every step here, so a memo keyed on them would be rebuilt every
        time).  Both sides cover every position once by construction, so the softmax rides in the two launches."""
        B, Hq, _, D = q.shape
        dev = q.device
        keep = []

        def fill(segs, code, scale, zero, bits, n_class, tail, layout_tail):
            n = 0
            if code is not None:
                code, scale, zero = code.contiguous(), scale.contiguous(), zero.contiguous()
                keep.extend((code, scale, zero))
                e = segs[0]
                e.bits, e.layout, e.n_tokens, e.pos_base = bits, 0, n_class, 0
                e.data, e.scale, e.zero, e.idx = code.data_ptr(), scale.data_ptr(), zero.data_ptr(), None
                n = 1
            if tail is not None and tail.shape[2] > 0:
                tail = tail.contiguous()
                keep.append(tail)
                e = segs[n]
                e.bits, e.layout, e.n_tokens, e.pos_base = 16, layout_tail, tail.shape[2], n_class
                e.data, e.scale, e.zero, e.idx = tail.data_ptr(), None, None, None
                n += 1
            return n

        Hkv = (k_full if k_full is not None else kq).shape[1]
        n_kq = 0 if kq is None else kq.shape[3] * (32 // self.k_bits)
        n_vq = 0 if vq is None else vq.shape[2]
        n_k = fill(self._k_segs, kq, ks, kz, self.k_bits, n_kq, k_full, _lib.LAYOUT_TOKEN_MAJOR)
        n_v = fill(self._v_segs, vq, vs, vz, self.v_bits, n_vq, v_full, 0)
        qc = q.contiguous()
        weights = torch.empty(B, Hq, 1, T, dtype=torch.float16, device=dev)
        out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=dev)
        lib = _lib.load()
        with _lib.on_device(dev):
            need = lib.hqekv_decode_workspace_bytes(self._k_segs, n_k, self._v_segs, n_v, B, Hq, Hkv, D)
            if need < 0:
                raise ValueError("invalid segment table")
            if self._ws is None or self._ws.numel() * 4 < need or self._ws.device != dev:
                self._ws = torch.empty(max(need + need // 4, 256) // 4, dtype=torch.float32, device=dev)
            rc = lib.hqekv_decode_attn(self._k_segs, n_k, self._v_segs, n_v, qc.data_ptr(), None, 0,
                                       weights.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, T, self._ws.data_ptr(),
                                       self._ws.numel() * 4, default_flags(), _lib.stream_ptr(dev))
        _lib.check(rc, "KiviAttentionLayer")
        return weights, out

    # ------------------------------------------------------------------ a decode step in place
    def _adopt(self, pkv: tuple, like: torch.Tensor) -> "_Buffers":
        """Capacity buffers holding what ``pkv`` holds: the K tail, the V tail (a window that slides one row per step)
        and the V class (which grows one row per step).  The K class stays as it is: it changes every
        ``residual_length`` steps only."""
        kq, k_full, ks, kz, vq, v_full, vs, vz, _ = pkv
        B, H, _, D = like.shape
        dev, R = like.device, self.residual_length
        st = _Buffers()
        st.kq, st.ks, st.kz = kq, ks, kz
        st.kt = torch.empty(B, H, R, D, dtype=torch.float16, device=dev)
        st.nk = 0 if k_full is None else k_full.shape[2]
        if st.nk:
            st.kt[:, :, :st.nk].copy_(k_full)
        st.cap_vt = 2 * R + 32
        st.vt = torch.empty(B, H, st.cap_vt, D, dtype=torch.float16, device=dev)
        st.v0, st.nv = 0, (0 if v_full is None else v_full.shape[2])
        if st.nv:
            st.vt[:, :, :st.nv].copy_(v_full)
        st.n_vq = 0 if vq is None else vq.shape[2]
        st.vcode = st.vscale = st.vzero = None
        self._grow_v_class(st, B, H, D, dev, st.n_vq + 1, (vq, vs, vz))
        return st

    def _grow_v_class(self, st: "_Buffers", B: int, H: int, D: int, dev, need: int, old=None) -> None:
        """Room for ``need`` rows in the V class buffers (doubling); ``old`` = (codes, scale, zero) to take over."""
        if st.vcode is not None and need <= st.vcode.shape[2]:
            return
        cap = max(self.MIN_V_ROWS, 2 * need)
        code = torch.empty(B, H, cap, D * self.v_bits // 32, dtype=torch.int32, device=dev)
        scale = torch.empty(B, H, cap, D // 32, dtype=torch.float16, device=dev)
        zero = torch.empty_like(scale)
        src = old if old is not None else (st.vcode, st.vscale, st.vzero)
        if st.n_vq and src[0] is not None:
            code[:, :, :st.n_vq].copy_(src[0][:, :, :st.n_vq])
            scale[:, :, :st.n_vq].copy_(src[1][:, :, :st.n_vq])
            zero[:, :, :st.n_vq].copy_(src[2][:, :, :st.n_vq])
        st.vcode, st.vscale, st.vzero = code, scale, zero

    def _step_in_buffers(self, q, k, v, pkv: tuple, T: int):
        """One decode step with everything appended in place: ONE call for the attention over (K class, K tail, this
        step's key) and (V class, V tail, this step's value) with the two rows copied behind their tails in the
        call's last launch, one quantiser launch when the oldest value row leaves the tail (written straight into the
        class buffers), one concatenation every ``residual_length`` steps when a block of keys is quantised.  The
        tuple handed back holds views of the buffers, with upstream's shapes and contents [117-266]."""
        q, k, v = (x if x.is_contiguous() else x.contiguous() for x in (q, k, v))
        st = self._st
        if st is None or st.returned is not pkv:
            st = self._st = self._adopt(pkv, k)
        B, Hq, _, D = q.shape
        Hkv, R, dev = k.shape[1], self.residual_length, q.device
        n_kq = 0 if st.kq is None else st.kq.shape[3] * (32 // self.k_bits)
        row = 2 * D   # bytes per token row

        def seg(e, bits, layout, n, pos, data, scale=None, zero=None, slab=0):
            e.bits, e.layout, e.n_tokens, e.pos_base, e.slab_tokens = bits, layout, n, pos, slab
            e.data, e.scale, e.zero, e.idx = data, scale, zero, None

        ka, n_k = self._k_segs, 0
        if n_kq:
            seg(ka[n_k], self.k_bits, 0, n_kq, 0, st.kq.data_ptr(), st.ks.data_ptr(), st.kz.data_ptr())
            n_k += 1
        if st.nk:
            seg(ka[n_k], 16, _lib.LAYOUT_TOKEN_MAJOR, st.nk, n_kq, st.kt.data_ptr(), slab=R)
            n_k += 1
        seg(ka[n_k], 16, _lib.LAYOUT_TOKEN_MAJOR, 1, T - 1, k.data_ptr())
        n_k += 1
        va, n_v = self._v_segs, 0
        if st.n_vq:
            seg(va[n_v], self.v_bits, 0, st.n_vq, 0, st.vcode.data_ptr(), st.vscale.data_ptr(), st.vzero.data_ptr(),
                slab=st.vcode.shape[2])
            n_v += 1
        if st.nv:
            seg(va[n_v], 16, 0, st.nv, st.n_vq, st.vt.data_ptr() + st.v0 * row, slab=st.cap_vt)
            n_v += 1
        seg(va[n_v], 16, 0, 1, T - 1, v.data_ptr())
        n_v += 1
        x = st.extra
        x.ring_line, x.append_rows, x.new_k, x.new_v = None, 1, k.data_ptr(), v.data_ptr()
        x.k_dst, x.v_dst = st.kt.data_ptr() + st.nk * row, st.vt.data_ptr() + (st.v0 + st.nv) * row
        x.k_dst_slab_tokens, x.v_dst_slab_tokens = R, st.cap_vt
        weights = torch.empty(B, Hq, 1, T, dtype=torch.float16, device=dev)
        out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=dev)
        lib = _lib.load()
        import ctypes as C
        with _lib.on_device(dev):
            for attempt in (0, 1):
                if self._ws is None or self._ws.device != dev or attempt:
                    need = lib.hqekv_decode_workspace_bytes(ka, n_k, va, n_v, B, Hq, Hkv, D)
                    if need < 0:
                        raise ValueError("invalid segment table")
                    self._ws = torch.empty(max(2 * need, 256) // 4, dtype=torch.float32, device=dev)
                rc = lib.hqekv_decode_step(ka, n_k, va, n_v, q.data_ptr(), None, 0, weights.data_ptr(), out.data_ptr(),
                                           B, Hq, Hkv, D, T, self._ws.data_ptr(), self._ws.numel() * 4, default_flags(),
                                           _lib.stream_ptr(dev), C.byref(x))
                if rc != -3:   # HQEKV_E_WORKSPACE: the cache has outgrown the workspace kept from earlier steps
                    break
            _lib.check(rc, "KiviAttentionLayer")
            st.nk += 1
            st.nv += 1
            if st.nk == R:   # a full block of fp16 keys: quantise it per channel, straight from its rows [236-252]
                c, s_, z = uniform_group_quantize_pack_last_dim(st.kt.transpose(2, 3), self.group_size, self.k_bits)
                st.kq = c if st.kq is None else torch.cat((st.kq, c), dim=3)
                st.ks = s_ if st.ks is None else torch.cat((st.ks, s_), dim=3)
                st.kz = z if st.kz is None else torch.cat((st.kz, z), dim=3)
                st.nk = 0
            if st.nv > R:    # the oldest fp16 value row leaves the tail for the class [254-264]
                self._grow_v_class(st, B, Hkv, D, dev, st.n_vq + 1)
                code, scale, zero = st.vcode, st.vscale, st.vzero
                n = st.n_vq
                _lib.check(lib.hqekv_quant_pack_rows(
                    st.vt.data_ptr() + st.v0 * row, st.cap_vt * D, D,
                    code.data_ptr() + n * code.stride(2) * 4, code.stride(1), code.stride(2),
                    scale.data_ptr() + n * scale.stride(2) * 2, zero.data_ptr() + n * zero.stride(2) * 2,
                    scale.stride(1), scale.stride(2), B * Hkv, 1, D, self.v_bits, _lib.stream_ptr(dev)),
                    "uniform_group_quantize_pack_last_dim")
                st.n_vq += 1
                st.v0 += 1
                st.nv -= 1
                if st.v0 + st.nv == st.cap_vt:   # the window has reached the end of its buffer: back to the start
                    st.vt[:, :, :st.nv].copy_(st.vt[:, :, st.v0:st.v0 + st.nv].clone())
                    st.v0 = 0
        nq = st.n_vq
        fields = (st.kq, st.kt[:, :, :st.nk] if st.nk else None, st.ks, st.kz,
                  st.vcode[:, :, :nq] if nq else None, st.vt[:, :, st.v0:st.v0 + st.nv],
                  st.vscale[:, :, :nq] if nq else None, st.vzero[:, :, :nq] if nq else None, T)
        st.returned = fields
        return out, weights, fields

    # ------------------------------------------------------------------ one call
    def forward(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                attention_mask: Optional[torch.Tensor] = None, past_key_value: Optional[tuple] = None):
        """query (B,Hq,L,D), key/value (B,Hkv,L,D) fp16, rotary applied.
        -> (attn_output (B,Hq,L,D), attn_weights (B,Hq,1,T) for a decode step, None for a prompt -- upstream's
        fused prompt attention returns none either -- , the 9-field tuple)."""
        L = key_states.shape[-2]
        kv_seq_len = L + (past_key_value[-1] if past_key_value is not None else 0)
        if past_key_value is None:
            out, fields = self._prefill(query_states, key_states, value_states, attention_mask)
            return out, None, fields + (kv_seq_len,)
        if L != 1:
            raise ValueError("a decode step appends one token")
        if (self.in_place and attention_mask is None and query_states.is_cuda and query_states.dtype == torch.float16
                and self.head_dim == query_states.shape[-1] == 128):
            return self._step_in_buffers(query_states, key_states, value_states, past_key_value, kv_seq_len)
        self._st = None
        kq, k_full, ks, kz, vq, v_full, vs, vz, _ = past_key_value
        R = self.residual_length
        k_full = key_states if k_full is None else torch.cat((k_full, key_states), dim=2)
        v_full = value_states if v_full is None else torch.cat((v_full, value_states), dim=2)

        if attention_mask is None and query_states.is_cuda and self.head_dim == query_states.shape[-1]:
            attn_weights, attn_output = self._attend(query_states, kq, ks, kz, k_full, vq, vs, vz, v_full, kv_seq_len)
        else:
            # with a mask: the quantised class and the fp16 tail of each side as fields of the hybrid tuple
            # (positions [0, Tq) are the class -- no index list: it sits at the head of the row --, the tail follows)
            t = [None] * 42
            if kq is not None:
                kb = K_BASE[self.k_bits]
                t[kb], t[kb + 2], t[kb + 3] = kq, ks, kz
            if vq is not None:
                vb = V_BASE[self.v_bits]
                t[vb], t[vb + 2], t[vb + 3] = vq, vs, vz
            t[NEW_K], t[NEW_V], t[41] = k_full, v_full, kv_seq_len
            attn_weights, attn_output = decode_attention(query_states, tuple(t), attention_mask, kv_seq_len,
                                                         zero_init=False, memo=self._memo)

        if k_full.shape[-2] == R:   # a full block of fp16 keys: quantise it per channel, straight from its rows
            c, s, z = uniform_group_quantize_pack_last_dim(k_full.transpose(2, 3), self.group_size, self.k_bits)
            k_full = None
            kq = c if kq is None else torch.cat((kq, c), dim=3)
            ks = s if ks is None else torch.cat((ks, s), dim=3)
            kz = z if kz is None else torch.cat((kz, z), dim=3)
        if v_full.shape[-2] > R:    # the oldest fp16 value row leaves the tail
            c, s, z = uniform_group_quantize_pack_last_dim(v_full[:, :, :1, :].contiguous(), self.group_size,
                                                           self.v_bits)
            v_full = v_full[:, :, 1:, :].contiguous()
            vq = c if vq is None else torch.cat((vq, c), dim=2)
            vs = s if vs is None else torch.cat((vs, s), dim=2)
            vz = z if vz is None else torch.cat((vz, z), dim=2)
        return attn_output, attn_weights, (kq, k_full, ks, kz, vq, v_full, vs, vz, kv_seq_len)

    __call__ = forward
