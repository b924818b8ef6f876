"""Importance tracking and block selection helpers the cache policy needs -- the counterpart of the
in-scope part of the reference's ``model/public_func.py`` (token range :58-90, block ranking :92-106,
the ring of recent attention rows :208-257, count repair :259-268).  Plain torch tensor ops on the
caller's device; nothing here is a hot loop.
"""
from __future__ import annotations

from typing import Optional

import torch


def calculate_token_norm(new_cache: Optional[torch.Tensor], token_norm: Optional[torch.Tensor]):
    """Per-token squared norm summed over batch, heads and channels, appended to the running vector."""
    if new_cache is None:
        return None
    n = new_cache.mul(new_cache).sum(0).sum(0).sum(-1)
    return n if token_norm is None else torch.cat((token_norm, n), dim=-1)


def calculate_new_token_range(new_cache: Optional[torch.Tensor]):
    """Per-token (max_d - min_d) summed over batch and heads."""
    if new_cache is None:
        return None
    return (torch.max(new_cache, dim=-1)[0] - torch.min(new_cache, dim=-1)[0]).sum(0).sum(0)


def calculate_token_range(new_cache: Optional[torch.Tensor], token_range: Optional[torch.Tensor]):
    """``calculate_new_token_range`` appended to the running per-token vector."""
    if new_cache is None:
        return None
    r = calculate_new_token_range(new_cache)
    return r if token_range is None else torch.cat((token_range, r), dim=-1)


def get_block_importance(block_size: int, block_num: int, importance: torch.Tensor) -> torch.Tensor:
    """Mean importance of each block.  Like the reference (model/public_func.py:85-90) this divides
    ``importance`` by the block length IN PLACE when it is contiguous (the reshape is then a view): the
    decode layer relies on that side effect -- the importance it hands to the cache policy afterwards is
    the divided one (model/llama_hqe.py:226-231)."""
    b = importance.reshape(block_num, -1)
    b /= b.shape[1]
    return torch.sum(b, dim=-1)


def get_block_token_idx(block_size: int, block_num: int, importance: torch.Tensor) -> torch.Tensor:
    """Token indices of the blocks ordered by descending mean importance, tokens inside a block in order
    (model/public_func.py:92-106, including the in-place divide of ``importance``).  The sort is stable --
    equal block scores keep their original order -- where the reference leaves the order of ties to the
    device sort."""
    _, order = torch.sort(get_block_importance(block_size, block_num, importance), descending=True, stable=True)
    ar = torch.arange(block_size, dtype=order.dtype, device=order.device)
    idx = (order.reshape(-1, 1) * block_size + ar.reshape(1, -1)).flatten()
    # the block order rides along: the cache policy needs the ranking on the host and fetches these
    # block_num entries instead of block_num * block_size
    idx._hq_block_order = (order, block_size)
    return idx


def make_sum_equal(array: torch.Tensor, array_sum: int, start_idx: int = 4) -> torch.Tensor:
    """Repair rounded block counts so they sum to ``array_sum``: a surplus is taken from index
    ``start_idx`` walking down to 0, a deficit is added to ``start_idx``; later entries (the evicted
    share) are never touched.  Works in place and returns the array, like the reference."""
    sub = array.sum() - array_sum
    for i in range(start_idx, -1, -1):
        if array[i] - sub < 0:
            sub -= array[i]
            array[i] = 0
        else:
            array[i] -= sub
            break
    return array


class last_attn_weights:
    """Ring of the last ``last_length`` attention rows (summed over batch and heads); the column mean of
    the ring is the token importance the policy ranks blocks by."""

    def __init__(self, last_length: int = 20):
        self.last_length = last_length
        self.max_length = 0
        self.kv_seq_len = 0
        self.next_line = 0
        self.weights = None

    def calculate_token_importance(self) -> torch.Tensor:
        count = torch.arange(self.kv_seq_len, 0, -1, dtype=self.weights.dtype, device=self.weights.device)
        count[:-self.last_length] = self.last_length
        return self.weights[:, :self.kv_seq_len].sum(0) / count

    def clear(self) -> None:
        self.next_line = 0
        self.weights.zero_()

    def eviction(self, reserve_idx: torch.Tensor) -> None:
        if self.weights is not None:
            kept = self.weights[:, reserve_idx]
            self.weights[:, :kept.shape[1]] = kept

    def reset(self) -> None:
        self.max_length = 0
        self.kv_seq_len = 0
        self.next_line = 0
        self.weights = None

    def set_max_length(self, max_length: int) -> None:
        self.max_length = max_length

    def update(self, attn_weights: torch.Tensor) -> None:
        if self.weights is None:
            self.weights = torch.zeros(self.last_length, self.max_length, dtype=attn_weights.dtype,
                                       device=attn_weights.device)
        if attn_weights.shape[2] > 1:   # prefill: keep the last rows
            rows = attn_weights if attn_weights.shape[2] < self.last_length else attn_weights[:, :, -self.last_length:, :]
            new_line = rows.sum(0).sum(0)
            self.weights[:new_line.shape[0], :new_line.shape[1]] = new_line
        else:                           # decode: one row into the ring
            # sum over the batch, then over the heads, each rounded to the ring's dtype like the reference's
            # ``.sum(0).sum(0)``; with one batch row the first sum is the identity, and the second one
            # writes its row of the ring directly
            per_head = attn_weights[0] if attn_weights.shape[0] == 1 else attn_weights.sum(0)
            new_line = self.weights[self.next_line:self.next_line + 1, :per_head.shape[-1]]
            if new_line.dtype == per_head.dtype:
                torch.sum(per_head, dim=0, out=new_line)
            else:
                new_line.copy_(per_head.sum(0))
        self.kv_seq_len = new_line.shape[1]
        self.next_line = (self.next_line + new_line.shape[0]) % self.last_length
