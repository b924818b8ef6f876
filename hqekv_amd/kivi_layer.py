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


class KiviAttentionLayer:
    """``k_bits``/``v_bits`` in {1, 2, 4, 8}; ``group_size`` 32; ``residual_length`` a multiple of 32
    (upstream: 2, 2, 32, 128 -- model/llama_kivi.py:72-76)."""

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
        self._k_segs = (_lib.Seg * 2)()   # (quantised class, fp16 tail) of each side, rewritten every step
        self._v_segs = (_lib.Seg * 2)()
        self._ws: Optional[torch.Tensor] = None

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
