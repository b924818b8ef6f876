"""Drop-in for ``KV_cache_hqe_2`` / ``KV_cache_reconstruct_hqe`` of the reference's ``quant/hqe_2.py``
(:456-843, :967-1084): quantise, demote and evict the cache, K per channel and V per token.
Same positional order and the same 42-field tuple in and out; the work is done by
:mod:`hqekv_amd.cache_policy` on HIP kernels."""
from __future__ import annotations

import torch

from . import cache_policy
from .public_func import last_attn_weights  # noqa: F401  (re-exported like the reference module does)


def KV_cache_hqe_2(past_key_value: tuple, compress_length: int, history_length: int, K_sorted_idx: torch.Tensor,
                   K_bit_num: torch.Tensor, V_bit_num: torch.Tensor, token_importance: torch.Tensor,
                   quant_strategy: str, last_weights=None, block_size: int = 32, group_size: int = 32,
                   times_range: bool = True) -> tuple:
    """K_bit_num / V_bit_num hold six token counts: fp16, 8, 4, 2, 1 bit and evicted (multiples of 32)."""
    return cache_policy.compress(past_key_value, compress_length, history_length, K_sorted_idx, K_bit_num,
                                 V_bit_num, token_importance, quant_strategy, last_weights=last_weights,
                                 block_size=block_size, group_size=group_size, times_range=times_range,
                                 n_targets=6)


def KV_cache_reconstruct_hqe(past_key_value: tuple, quant_strategy: str, block_size: int = 32,
                             group_size: int = 32):
    """-> dense fp16 (K, V) of shape (B, Hkv, kv_seq_len, D)."""
    return cache_policy.reconstruct(past_key_value, quant_strategy, block_size, group_size)
