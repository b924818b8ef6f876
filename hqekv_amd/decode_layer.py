"""The caller of the decode path: the cache-side state machine of the reference's attention layer
(``LlamaAttention_hqe.forward``, model/llama_hqe.py:55-251; ``Qwen3Attention_hqe`` has the same cache
logic) without what surrounds it -- projections, rotary embedding, ``o_proj``.

Per call (model/llama_hqe.py, line numbers in brackets):
  prefill   attention over the prompt; cache = ``(None,)*39 + (K, V, len)`` [186]
  decode    ``new_K/new_V = cat(residual, k/v)`` [131-133] -> hybrid attention over the 42-field tuple [136]
  always    the probabilities feed the ring of the last 20 rows [199]; with >= 32 un-quantised tokens:
            class sizes from the ratios [216-224] (or layer 0's, handed down as ``auxiliary_parameters``
            [211-214]), block ranking [228], ``KV_cache_hqe_2`` [230-231], bookkeeping and the ratio
            update for the next 32-token increment [233-239].

Decode attention, quantisation, demotion and eviction run on the HIP kernels of this package, and so does the
prompt for fp16 tensors of head_dim 128: one matrix-core kernel for the causal attention over the whole prompt
(flash-attention in the reference [146-154]) and one for the probabilities of the last 20 rows, the only rows the
ring keeps [156-170].  A prompt with an explicit additive mask, another head size or element type goes through
torch's fused attention for the output.  Neither path materialises ``repeat_kv`` copies of K or V.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from . import prompt_attention
from .attention import SegmentMemo, value_length
from .hqe_2 import KV_cache_hqe_2
from .hqe_matmul import qkv_matmul_hqe_2
from .public_func import last_attn_weights

LAST_TOKEN_NUM = 20
BLOCK = 32


def _repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    if n_rep == 1:
        return x
    B, H, T, D = x.shape
    return x[:, :, None, :, :].expand(B, H, n_rep, T, D).reshape(B, H * n_rep, T, D)


_GQA_SDPA = [True]   # torch's fused attention takes grouped query heads directly (no repeat_kv copies) until it says no


def gqa_prompt_attention(q, k, v, attention_mask, scaling):
    """softmax(q k^T * scaling + mask) v over a whole prompt with grouped query heads (the reference calls
    flash-attention here, model/llama_hqe.py:146-154).  Without a mask -- the causal rule -- fp16 tensors of head_dim
    128 go to the library's matrix-core kernel (``prompt_attention``); a prompt with an explicit additive mask, another
    head size or element type goes through torch's fused attention.  K and V are handed over as they are, (B,Hkv,T,D);
    only when torch's kernel refuses grouped heads are they expanded."""
    if attention_mask is None and prompt_attention.supported(q, k, v):
        return prompt_attention.prompt_attention(q, k, v, scaling, causal=True)
    n_rep = q.shape[1] // k.shape[1]
    causal = attention_mask is None and k.shape[-2] > 1
    if n_rep > 1 and _GQA_SDPA[0]:
        try:
            return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=attention_mask, is_causal=causal,
                                                                    scale=scaling, enable_gqa=True)
        except (TypeError, RuntimeError):
            _GQA_SDPA[0] = False
    return torch.nn.functional.scaled_dot_product_attention(q, _repeat_kv(k, n_rep), _repeat_kv(v, n_rep),
                                                            attn_mask=attention_mask, is_causal=causal, scale=scaling)


def last_rows_probabilities(q, k, attention_mask, scaling, rows):
    """Probabilities of the last ``rows`` query rows of a prompt over all keys, (B,Hq,rows,T), as the reference
    computes them for the importance ring (model/llama_hqe.py:156-168): the library's kernel for fp16 tensors of
    head_dim 128 (same roundings; without a mask the causal rule), torch otherwise.  The query heads that share a KV
    head are folded into the row dimension of one batched product instead of materialising ``repeat_kv`` copies."""
    mask_fits = attention_mask is None or (attention_mask.dim() == 4 and attention_mask.shape[1] == 1
                                           and attention_mask.shape[0] in (1, q.shape[0]) and attention_mask.shape[3] == q.shape[2])
    if rows <= prompt_attention.MAX_LAST_ROWS and mask_fits and prompt_attention.supported(q, k):
        return prompt_attention.prompt_last_rows(q, k, scaling, rows, attention_mask)
    B, Hq, T, D = q.shape
    Hkv = k.shape[1]
    q_last = q[:, :, T - rows:, :].reshape(B, Hkv, (Hq // Hkv) * rows, D)          # (b, kv head, [rep, row], d)
    w = (torch.matmul(q_last, k.transpose(2, 3)) * scaling).view(B, Hq, rows, T)
    if attention_mask is not None:
        w = w + attention_mask[:, :, -rows:, :]
        w = torch.max(w, torch.tensor(torch.finfo(w.dtype).min, dtype=w.dtype, device=w.device))
    elif rows > 1 or T > 1:
        keep = torch.arange(T, device=q.device)[None, :] <= (T - rows + torch.arange(rows, device=q.device))[:, None]
        w = w.masked_fill(~keep, torch.finfo(w.dtype).min)
    return torch.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)


_F32 = np.float32


def class_token_counts(total_length: int, ratio_q: torch.Tensor, ratio_e: torch.Tensor):
    """Tokens per target -- fp16, 8, 4, 2, 1 bit, evicted -- for a history of ``total_length`` tokens
    (model/llama_hqe.py:216-224).  64 tokens' worth of blocks stay fp16 and nothing goes to 8 bit; the rest is
    split by ``ratio_q`` (4, 2, 1 bit) and ``ratio_e`` (evicted), in float32 like the reference, rounded to
    whole blocks and repaired to add up (model/public_func.py:259-268).  -> (shares (6,) float32, token counts (6,)
    int32).  The arithmetic runs on numpy float32 scalars and 6-element arrays -- the same IEEE operations in the
    same order as the reference's CPU tensor ops, at a fraction of their dispatch cost."""
    blocks = total_length // BLOCK
    shares = np.zeros(6, dtype=np.float32)
    shares[0] = 64 / total_length
    rest = _F32(1) - shares[0]
    shares[2:5] = rest * ratio_q.numpy()
    shares[5] = rest * ratio_e.numpy()[0]
    counts = [int(c) for c in np.rint(_F32(blocks) * shares)]   # half to even, like torch.round
    excess = sum(counts) - blocks
    if excess < 0:
        counts[4] -= excess
    else:   # taken from the 1-bit entry, then from the entries below it, each down to zero at most
        i = 4
        while excess > 0 and i >= 0:
            take = min(excess, counts[i])
            counts[i] -= take
            excess -= take
            i -= 1
    return torch.from_numpy(shares), torch.tensor([c * BLOCK for c in counts], dtype=torch.int32)


def ratios_for_next_increment(history: int, ratio_e_0: torch.Tensor, ratio_q: torch.Tensor):
    """The eviction share applies to the tokens the next compression adds, not to the history it re-ranks:
    scale it by added / (history + added) and give the quantised classes the rest, in their old proportions
    (model/llama_hqe.py:235-239).  -> (ratio_e, ratio_q), float32 as in the reference (numpy scalars, see above)."""
    added = (history + BLOCK) // BLOCK * BLOCK - history
    ratio_e = (_F32(added) * ratio_e_0.numpy()) / _F32(history + added)
    rq = ratio_q.numpy()
    total = rq[0]
    for x in rq[1:]:
        total = total + x
    return torch.from_numpy(ratio_e), torch.from_numpy((_F32(1) - ratio_e) * rq / total)


class HqeAttentionLayer:
    """State of one layer: un-quantised length, kept history length, eviction / quantisation ratios and the
    importance ring.  ``bit_0`` is the evicted share, ``bit_4``/``bit_2``/``bit_1`` the 4-, 2- and 1-bit
    shares of what is kept (config.bit_* of the reference); two blocks always stay fp16 and the 8-bit
    share is 0 [216]."""

    def __init__(self, head_dim: int, bit_0: float, bit_4: float, bit_2: float, bit_1: float = 0.0,
                 quant_strategy: str = "uniform_group", times_range: bool = True,
                 last_length: int = LAST_TOKEN_NUM):
        self.head_dim = head_dim
        self.scaling = head_dim ** -0.5
        self.quant_strategy = quant_strategy
        self.times_range = times_range
        self.ratio_e_0 = torch.tensor([bit_0], dtype=torch.float32)
        self.ratio_e = self.ratio_e_0.clone()
        self.ratio_q = torch.tensor([bit_4, bit_2, bit_1], dtype=torch.float32)
        self.current_length = 0
        self.history_reserve_length = 0
        self.token_num = 0
        self.last_weights = last_attn_weights(last_length=last_length)
        self._memo = SegmentMemo()   # segment tables of the classes, rebuilt after each compression
        self._res = None             # (K buffer, V buffer): the fp16 residual in capacity-sized storage
        self.fused_step = True       # ring row and residual appends inside the attention call (False: separate launches)
        self._own_tuple = False      # the tuple handed in carries the class tensors this layer built its tables from
        self._returned = None        # (the tuple the last plain decode step returned, tokens in its residual)

    def reset(self) -> None:
        """What the reference's ``generate`` does per layer before a new prompt [555-557]."""
        self.current_length = 0
        self.history_reserve_length = 0
        self.token_num = 0
        self.ratio_e = self.ratio_e_0.clone()
        self.last_weights.reset()
        self._memo = SegmentMemo()
        self._res = None
        self._returned = None

    def set_max_length(self, max_length: int) -> None:
        """Prompt length + new tokens: the width of the importance ring [691-695]."""
        self.last_weights.set_max_length(max_length)

    # ------------------------------------------------------------------ prompt
    def _prefill(self, q, k, v, attention_mask):
        """Prompt attention [141-188]: the output over all rows, and the probabilities of the last 20 rows only (what
        the ring keeps).  K and V are read once per KV head, without ``repeat_kv`` copies."""
        rows = min(q.shape[2], LAST_TOKEN_NUM)
        attn_weights = last_rows_probabilities(q, k, attention_mask, self.scaling, rows)
        attn_output = gqa_prompt_attention(q, k, v, attention_mask, self.scaling)
        return attn_weights, attn_output

    # ------------------------------------------------------------------ residual storage
    def _residual_in_buffers(self, pkv: tuple, key_states: torch.Tensor) -> tuple:
        """The tuple with its fp16 residual held as the head of this layer's capacity-sized buffers (B,Hkv,cap,D), so
        that a decode step appends a row in place instead of re-allocating ``cat(residual, k)`` [131-133].  A residual
        that is not there yet -- after the prompt, after a compression, or a tuple from elsewhere -- is copied in
        once; the fields of the tuple are views of the same shape and content as the reference's tensors."""
        res_K, res_V = pkv[-3], pkv[-2]
        B, H, L, D = key_states.shape
        n = res_K.shape[2] if res_K is not None else 0
        buf = self._res
        held = self._memo.held
        self._own_tuple = held is not None and all(a is b for a, b in zip(held, pkv))
        fits = (buf is not None and buf[0].shape[0] == B and buf[0].shape[1] == H and buf[0].shape[3] == D
                and buf[0].device == key_states.device and buf[0].dtype == key_states.dtype and n + L <= buf[0].shape[2])
        if fits and (n == 0 or (res_K.data_ptr() == buf[0].data_ptr() and res_V.data_ptr() == buf[1].data_ptr()
                                and res_K.stride() == buf[0].stride() and res_V.stride() == buf[1].stride())):
            return pkv
        cap = max(2 * BLOCK, (n + L + BLOCK - 1) // BLOCK * BLOCK + BLOCK)
        kb = torch.empty(B, H, cap, D, dtype=key_states.dtype, device=key_states.device)
        vb = torch.empty_like(kb)
        if n:
            kb[:, :, :n].copy_(res_K)
            vb[:, :, :n].copy_(res_V)
        self._res = (kb, vb)
        if n == 0:
            return pkv
        return pkv[:-3] + (kb[:, :, :n], vb[:, :, :n], pkv[-1])

    # ------------------------------------------------------------------ one call
    def forward(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                attention_mask: Optional[torch.Tensor] = None, past_key_value: Optional[tuple] = None,
                auxiliary_parameters: Optional[Tuple[torch.Tensor, ...]] = None):
        """query (B,Hq,L,D), key/value (B,Hkv,L,D), rotary already applied.
        -> (attn_output (B,Hq,L,D), attn_weights (the last <= 20 rows for a prompt), tuple, auxiliary_parameters)."""
        L = key_states.shape[-2]
        self.current_length += L
        kv_seq_len = L + (past_key_value[-1] if past_key_value is not None else 0)
        if past_key_value is not None:
            # The attention reads this step's key and value where they are, as a segment behind the residual, and
            # is queued first; the copies that append them to the residual [131-133] follow it on the stream, off
            # the step's critical path.
            back = self._returned
            known = (back is not None and back[0] is past_key_value and self._res is not None
                     and back[1] + L <= self._res[0].shape[2])
            if known:   # the very tuple the previous step handed out: its residual is the head of the buffers
                n, self._own_tuple = back[1], True
            else:
                past_key_value = self._residual_in_buffers(past_key_value, key_states)
                n = past_key_value[-3].shape[2] if past_key_value[-3] is not None else 0
            self._returned = None
            # tokens the classes hold = the history this layer has kept; a tuple from elsewhere is counted
            Tall = (self.history_reserve_length if self._own_tuple else value_length(past_key_value) - n) + n + L
            lw = self.last_weights
            # shapes for which the ring row's summation order is pinned against torch's on the device
            on_device = (self.fused_step and L == 1 and Tall >= 256 and query_states.shape[1] == 32
                         and query_states.shape[0] <= 8 and query_states.dtype == torch.float16
                         and (lw.weights is None or lw.weights.dtype == torch.float16) and lw.max_length >= Tall)
            if self.fused_step and attention_mask is None and L == 1 and query_states.is_cuda:
                # slices of a fused projection's output arrive with a batch stride of their own: one small copy each
                # buys the one-call step
                query_states, key_states, value_states = (x if x.is_contiguous() else x.contiguous()
                                                          for x in (query_states, key_states, value_states))
            plain_inputs = (self.fused_step and attention_mask is None and query_states.shape[2] == 1
                            and query_states.is_contiguous() and key_states.is_contiguous() and value_states.is_contiguous()
                            and query_states.dtype == torch.float16 and query_states.is_cuda
                            and self.quant_strategy in ("uniform_group", "high_uniform_group_low_normal_group"))
            if plain_inputs:
                # One call: attention, the ring row (in torch's own summation order) and the two residual appends
                # [131-133, 200]; the kernels read this step's key and value where they are, as a segment behind the
                # residual, and copy them into the residual buffers in the call's last launch.
                if on_device and lw.weights is None:
                    lw.decode_row(query_states, Tall)   # creates the store
                attn_weights, attn_output = self._memo.step_call(
                    query_states, past_key_value, Tall, key_states, value_states, self._res, n,
                    lw.weights if on_device else None, lw.next_line, self.quant_strategy == "uniform_group", known)
            else:
                attn_weights, attn_output = qkv_matmul_hqe_2(query_states, past_key_value, attention_mask,
                                                             self.head_dim, self.quant_strategy, memo=self._memo,
                                                             tail=(key_states, value_states))
            if plain_inputs and on_device:
                lw.advance(Tall)
            else:
                lw.update(attn_weights)
            if not plain_inputs:   # the plain sequence of the reference: two copies after the attention
                self._res[0][:, :, n:n + L].copy_(key_states)
                self._res[1][:, :, n:n + L].copy_(value_states)
            new_K, new_V = self._res[0][:, :, :n + L], self._res[1][:, :, :n + L]
            past_key_value = past_key_value[:-3] + (new_K, new_V, kv_seq_len)
            if plain_inputs:
                self._returned = (past_key_value, n + L)
        else:
            attn_weights, attn_output = self._prefill(query_states, key_states, value_states, attention_mask)
            past_key_value = (None,) * 39 + (key_states, value_states, kv_seq_len)
            self.last_weights.update(attn_weights)

        if self.current_length < BLOCK:
            self.token_num += 1
            return attn_output, attn_weights, past_key_value, None

        self._returned = None   # what follows builds another tuple
        # whole blocks of the un-quantised tokens join the history; the rest stays the fp16 residual
        compress_length = self.current_length // BLOCK * BLOCK
        total_length = self.history_reserve_length + compress_length
        shared = auxiliary_parameters is not None          # layer 0 of this step already sized the classes
        if shared:
            shares, K_bit_num, V_bit_num = auxiliary_parameters
        else:
            shares, K_bit_num = class_token_counts(total_length, self.ratio_q, self.ratio_e)
            V_bit_num = K_bit_num.clone()
        # the importance of every token and the ranking of the blocks; like the reference's ranking helper, which
        # divides its argument by the block length in place, this leaves the policy the divided values [226-231]
        importance, K_token_idx = self.last_weights.ranked_importance(total_length)
        past_key_value = KV_cache_hqe_2(past_key_value, compress_length, self.history_reserve_length,
                                        K_token_idx, K_bit_num, V_bit_num, importance,
                                        self.quant_strategy, self.last_weights, BLOCK, BLOCK, self.times_range)
        self.history_reserve_length += compress_length - int(K_bit_num[-1])
        self.current_length -= compress_length
        if not shared:
            self.ratio_e, self.ratio_q = ratios_for_next_increment(self.history_reserve_length, self.ratio_e_0,
                                                                   self.ratio_q)
        self.token_num += 1
        return attn_output, attn_weights, past_key_value, (shares, K_bit_num, V_bit_num)

    __call__ = forward
