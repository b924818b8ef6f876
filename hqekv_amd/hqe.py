"""Import name of the reference's first cache generation (``quant/hqe.py``), where K is quantised per
token like V.  ``model/llama_hqe.py:23`` and ``model/qwen3_hqe.py:23`` import ``KV_cache_hqe`` from it
but only ever call ``KV_cache_hqe_2`` (model/llama_hqe.py:230), so the name has to resolve for the
model files to load; the per-token-K generation itself is not built and says so when called.
"""
from __future__ import annotations


def KV_cache_hqe(past_key_value, compress_length, history_reserve_length, K_sorted_idx, K_bit_num, V_bit_num,
                 token_importance, quant_strategy, last_weights=None, block_size: int = 32, group_size: int = 32):
    """Signature of quant/hqe.py:143-155."""
    raise NotImplementedError(
        "KV_cache_hqe (K quantised per token, quant/hqe.py:143) is the superseded cache generation; "
        "the decode path of the model files uses KV_cache_hqe_2")
