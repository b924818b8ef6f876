"""Drop-in for ``qkv_matmul_hqe_2`` of the reference's ``quant/hqe_matmul.py`` (:354-451), the decode
attention the model files call (model/llama_hqe.py:136).  It differs from ``qkv_matmul`` in two
ways, both kept: the sequence length is the sum of the V class lengths plus the residual, not the
tuple's ``kv_seq_len`` (:379-406), and the attention mask is ignored (:431).
"""
from __future__ import annotations

from typing import Tuple

import torch

from .attention import decode_attention, value_length


def qkv_matmul_hqe_2(q: torch.Tensor, past_key_value: Tuple, attention_mask, head_dim: int,
                     quant_strategy: str, block_size: int = 32, group_size: int = 32, memo=None, tail=None, step=None):
    """-> (attn_weights (B,Hq,1,real_len) fp16, attn_output (B,Hq,1,D) fp16).
    Not in the reference's signature, both optional: ``memo``, an ``attention.SegmentMemo`` kept per layer, and
    ``tail`` = (k, v), the step's new key and value rows (B,Hkv,L,D) when the caller has not appended them to the
    tuple's residual yet; they count into ``real_len``; ``step``: the ring row and the residual appends of the
    caller's decode step, folded into the call (``attention.decode_attention``)."""
    if quant_strategy not in ("uniform_group", "high_uniform_group_low_normal_group"):
        # upstream accepts only these two here (quant/hqe_matmul.py:370-377)
        raise ValueError('invalid quant_strategy')
    if block_size != 32 or group_size != 32:
        raise ValueError("block_size and group_size must be 32")
    real_len = value_length(past_key_value) + (tail[1].shape[2] if tail is not None else 0)
    if real_len == 0:
        raise ValueError('invalid past_key_value')
    return decode_attention(q, past_key_value, None, real_len, zero_init=False,
                            low_uniform=quant_strategy == "uniform_group", memo=memo, tail=tail, step=step)


def qkv_matmul_hqe(q: torch.Tensor, past_key_value: Tuple, attention_mask, head_dim: int,
                   quant_strategy: str, block_size: int = 32, group_size: int = 32):
    """Signature of quant/hqe_matmul.py:27-35: attention over a cache whose K is quantised per token
    (the generation written by ``quant/hqe.py``).  The model files import the name
    (model/llama_hqe.py:25) and call ``qkv_matmul_hqe_2`` only; it resolves here and is not built."""
    raise NotImplementedError(
        "qkv_matmul_hqe (per-token K, quant/hqe_matmul.py:27) belongs to the superseded cache generation; "
        "use qkv_matmul_hqe_2")
