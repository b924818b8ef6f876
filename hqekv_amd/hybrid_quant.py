"""Drop-in for the reference's ``quant/hybrid_quant.py``: ``KV_cache_compress`` (:318-612),
``KV_cache_compress_1`` (:614-730) and ``KV_cache_reconstruct`` (:732-846) -- the generation of the cache
policy without eviction (five token counts: fp16, 8, 4, 2, 1 bit).  Same positional order and the same
42-field tuple; the work is done by :mod:`hqekv_amd.cache_policy` on HIP kernels."""
from __future__ import annotations

import torch

from . import cache_policy


def KV_cache_compress(past_key_value: tuple, compress_length: int, history_length: int,
                      K_sorted_idx: torch.Tensor, K_bit_num: torch.Tensor, V_bit_num: torch.Tensor,
                      token_importance: torch.Tensor, quant_strategy: str, block_size: int = 32,
                      group_size: int = 32) -> tuple:
    return cache_policy.compress(past_key_value, compress_length, history_length, K_sorted_idx, K_bit_num,
                                 V_bit_num, token_importance, quant_strategy, block_size=block_size,
                                 group_size=group_size, times_range=True, n_targets=5)


def KV_cache_compress_1(past_key_value: tuple, compress_length: int, history_length: int,
                        K_sorted_idx: torch.Tensor, K_bit_num: torch.Tensor, V_bit_num: torch.Tensor,
                        token_importance: torch.Tensor, V_token_range: torch.Tensor, quant_strategy: str,
                        block_size: int = 32, group_size: int = 32) -> tuple:
    """As ``KV_cache_compress`` with the per-token V range supplied by the caller (None = compute it)."""
    return cache_policy.compress(past_key_value, compress_length, history_length, K_sorted_idx, K_bit_num,
                                 V_bit_num, token_importance, quant_strategy, block_size=block_size,
                                 group_size=group_size, times_range=True, n_targets=5, V_token_range=V_token_range)


def KV_cache_reconstruct(past_key_value: tuple, quant_strategy: str, block_size: int = 32, group_size: int = 32):
    """-> dense fp16 (K, V) of shape (B, Hkv, kv_seq_len, D)."""
    return cache_policy.reconstruct(past_key_value, quant_strategy, block_size, group_size)
