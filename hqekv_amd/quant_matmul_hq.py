"""Drop-in for the reference's ``quant/quant_matmul_hq.py``: decode attention over the 42-field cache.

``qkv_matmul`` (quant/quant_matmul_hq.py:23-120, one GEMV per class plus torch scatter/softmax) and
``qkv_matmul_hq`` (:122-174, the fused launches) compute the same thing; both run here as one
q.K^T launch over every class, one scale/mask/clamp/softmax pass and one p.V launch.
The scores buffer spans ``kv_seq_len`` positions and starts at zero, as upstream (:58).
"""
from __future__ import annotations

from typing import Tuple

import torch

from .attention import KV_SEQ_LEN, decode_attention

_STRATEGIES = ("uniform_group", "high_uniform_group_low_normal_group")
_KNOWN = ("uniform", "normal", "uniform_group", "normal_group", "high_uniform_group_low_normal_group")


def _check_strategy(quant_strategy: str) -> None:
    if quant_strategy not in _KNOWN:
        raise ValueError('invalid quant_strategy')
    if quant_strategy not in _STRATEGIES:
        raise NotImplementedError(
            f"quant_strategy '{quant_strategy}' uses the per-row / normal-quantile kernels, which are not built")


def qkv_matmul(q: torch.Tensor, past_key_value: Tuple, attention_mask, head_dim: int, quant_strategy: str,
               block_size: int = 32, group_size: int = 32):
    """-> (attn_weights (B,Hq,1,kv_seq_len) fp16, attn_output (B,Hq,1,D) fp16)."""
    _check_strategy(quant_strategy)
    if block_size != 32 or group_size != 32:
        raise ValueError("block_size and group_size must be 32")
    if all(x is None for x in past_key_value[:36]) and past_key_value[39] is None:
        raise ValueError('invalid past_key_value')
    if head_dim != q.shape[-1]:
        raise ValueError("head_dim does not match q")
    Tall = int(past_key_value[KV_SEQ_LEN])
    return decode_attention(q, past_key_value, attention_mask, Tall, zero_init=True,
                            low_uniform=quant_strategy == "uniform_group")


qkv_matmul_hq = qkv_matmul
