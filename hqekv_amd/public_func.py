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


def _token_major_slabs(x: torch.Tensor):
    """Tokens between two (b, h) slabs of a (B, H, T, D) tensor whose rows are dense and whose slabs are equally
    spaced (a dense tensor, or the head of a capacity buffer), else None."""
    B, H, T, D = x.shape
    sb, sh, st, sd = x.stride()
    if sd != 1 or st != D or sh % D or sh < T * D or (B > 1 and sb != H * sh):
        return None
    return sh // D


def calculate_new_token_range(new_cache: Optional[torch.Tensor]):
    """Per-token (max_d - min_d) summed over batch and heads (model/public_func.py:58-66): on the device one launch of
    ``hqekv_token_range``, which adds in torch's own order."""
    if new_cache is None:
        return None
    if new_cache.is_cuda and new_cache.dtype == torch.float16 and new_cache.dim() == 4 and new_cache.numel() \
            and new_cache.shape[0] * new_cache.shape[1] <= 1024:
        slab = _token_major_slabs(new_cache)
        if slab is not None:
            from . import _lib
            B, H, T, D = new_cache.shape
            out = torch.empty(T, dtype=torch.float16, device=new_cache.device)
            with _lib.on_device(new_cache.device):
                rc = _lib.load().hqekv_token_range(new_cache.data_ptr(), B, H, T, D, slab, out.data_ptr(),
                                                   _lib.stream_ptr(new_cache.device))
            _lib.check(rc, "token_range")
            return out
    lo, hi = torch.aminmax(new_cache, dim=-1)
    return (hi - lo).sum(0).sum(0)


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


class RankedBlocks:
    """A block ranking that has not been spelt out yet: ``scores`` holds the mean importance of every block,
    ``order`` (made on first use) the block numbers, most important first -- a stable descending sort, so the
    order is a function of the scores alone and whoever holds two rankings may sort them in one call.  The cache
    policy plans from the block order; ``tokens()`` builds the token list the reference's helper returns (and
    remembers it).  Reads like a tensor where the policy looks: ``numel()``, and the block order riding along under
    the names it rides along with on a token list."""
    __slots__ = ("scores", "block_size", "_order", "_tokens")
    _version = 0                    # nobody can have written into positions that do not exist yet
    _hq_block_order_version = 0

    def __init__(self, scores: torch.Tensor, block_size: int):
        self.scores, self.block_size, self._order, self._tokens = scores, block_size, None, None

    @property
    def order(self) -> torch.Tensor:
        if self._order is None:
            self._order = torch.sort(self.scores, descending=True, stable=True)[1]
        return self._order

    @staticmethod
    def sort_together(a: "RankedBlocks", b: "RankedBlocks") -> torch.Tensor:
        """Both orders from one sort call, as a (2, blocks) tensor; rows are what each would get alone."""
        if a._order is None and b._order is None and a.scores.shape == b.scores.shape \
                and a.scores.device == b.scores.device and a.scores.dtype == b.scores.dtype:
            both = torch.sort(torch.stack((a.scores, b.scores)), dim=1, descending=True, stable=True)[1]
            a._order, b._order = both[0], both[1]
            return both
        return torch.stack((a.order, b.order))

    @property
    def _hq_block_order(self):
        return self.order, self.block_size

    def numel(self) -> int:
        return self.scores.numel() * self.block_size

    def tokens(self) -> torch.Tensor:
        if self._tokens is None:
            order, bs = self.order, self.block_size
            ar = torch.arange(bs, dtype=order.dtype, device=order.device)
            idx = (order.reshape(-1, 1) * bs + ar.reshape(1, -1)).flatten()
            # the block order rides along: the cache policy needs the ranking on the host and fetches these
            # block_num entries instead of block_num * block_size
            idx._hq_block_order = (order, bs)
            idx._hq_block_order_version = idx._version   # ignored once somebody writes into idx
            self._tokens = idx
        return self._tokens


def rank_blocks(block_size: int, block_num: int, importance: torch.Tensor) -> RankedBlocks:
    """The ranking of ``get_block_token_idx`` without the token list (same in-place divide of ``importance``)."""
    return RankedBlocks(get_block_importance(block_size, block_num, importance), block_size)


def rank_blocks_weighted(block_num: int, importance: torch.Tensor, weights: Optional[torch.Tensor]) -> RankedBlocks:
    """The ranking of ``importance * weights`` (``importance`` alone without weights) in blocks of 32, the V side's
    (quant/hqe_2.py:510-518); neither argument is modified.  On the device one launch of
    ``hqekv_weighted_block_scores`` in place of the product, the divide and the block sums."""
    total = block_num * 32
    if importance.is_cuda and importance.dtype == torch.float16 and importance.is_contiguous() \
            and importance.numel() == total and total > 0 \
            and (weights is None or (weights.is_cuda and weights.dtype == torch.float16 and weights.is_contiguous()
                                     and weights.numel() == total)):
        from . import _lib
        scores = torch.empty(block_num, dtype=torch.float16, device=importance.device)
        with _lib.on_device(importance.device):
            rc = _lib.load().hqekv_weighted_block_scores(importance.data_ptr(), None if weights is None else weights.data_ptr(),
                                                         total, scores.data_ptr(), _lib.stream_ptr(importance.device))
        _lib.check(rc, "weighted_block_scores")
        return RankedBlocks(scores, 32)
    return rank_blocks(32, block_num, importance * weights if weights is not None else importance.clone())


def get_block_token_idx(block_size: int, block_num: int, importance: torch.Tensor) -> torch.Tensor:
    """Token indices of the blocks ordered by descending mean importance, tokens inside a block in order
    (model/public_func.py:92-106, including the in-place divide of ``importance``).  The sort is stable --
    equal block scores keep their original order -- where the reference leaves the order of ties to the
    device sort."""
    return rank_blocks(block_size, block_num, importance).tokens()


def make_sum_equal(array: torch.Tensor, array_sum: int, start_idx: int = 4) -> torch.Tensor:
    """Repair rounded block counts so that they add up to ``array_sum`` (the rule of the reference's
    model/public_func.py:259-268): what is too much is taken away from entry ``start_idx``, then from the
    entries below it, each down to zero at most; what is missing is added to entry ``start_idx``.  Entries
    above ``start_idx`` (the evicted share) are never touched.  Works in place and returns ``array``."""
    excess = int(array.sum()) - int(array_sum)
    if excess < 0:
        array[start_idx] -= excess
        return array
    i = start_idx
    while excess > 0 and i >= 0:
        take = min(excess, int(array[i]))
        array[i] -= take
        excess -= take
        i -= 1
    return array


class last_attn_weights:
    """The last ``last_length`` attention rows, each summed over batch and heads (model/public_func.py:208-257;
    same attribute and method names: the model code and the cache policy reach into them).  ``weights`` is the
    (last_length, max_length) store: the rows of a prompt fill it from the top, decode rows go round in a ring
    from ``next_line``.  A token's importance is the mean of its column over the rows that have seen it."""

    def __init__(self, last_length: int = 20):
        self.last_length = last_length
        self.reset()

    def reset(self) -> None:
        self.max_length = 0
        self.kv_seq_len = 0
        self.next_line = 0
        self.weights = None
        self._seen = None

    def set_max_length(self, max_length: int) -> None:
        self.max_length = max_length

    def clear(self) -> None:
        self.next_line = 0
        self.weights.zero_()

    def calculate_token_importance(self) -> torch.Tensor:
        n, w = self.kv_seq_len, self.weights
        # column j has been seen by min(last_length, n - j) rows: the newest tokens by fewer than all of them.
        # One vector made once serves every n: r[i] = min(last_length, len(r) - i), and the counts for n columns are
        # its last n entries.
        r = self._seen
        if r is None or r.shape[0] < n or r.device != w.device or r.dtype != w.dtype:
            m = max(n, w.shape[1])
            r = self._seen = torch.clamp(m - torch.arange(m, device=w.device), max=self.last_length).to(w.dtype)
        return w[:, :n].sum(0) / r[r.shape[0] - n:]

    def ranked_importance(self, total: int):
        """What a compression needs from the ring for the first ``total`` tokens (a multiple of 32):
        ``calculate_token_importance()[:total]`` divided by 32 -- the values ``get_block_token_idx`` leaves behind in
        its argument, which the policy is handed (model/llama_hqe.py:226-231) -- and the ranking of the blocks by their
        mean importance.  On the device one launch (``hqekv_importance_scores``) in place of the sum over the rows,
        the divide by the counts, the copy, the in-place divide and the block sums.  -> (importance / 32, RankedBlocks)."""
        n, w = self.kv_seq_len, self.weights
        if w.is_cuda and w.dtype == torch.float16 and w.is_contiguous() and 0 < total <= n and total % 32 == 0:
            from . import _lib
            imp = torch.empty(total, dtype=torch.float16, device=w.device)
            scores = torch.empty(total // 32, dtype=torch.float16, device=w.device)
            with _lib.on_device(w.device):
                rc = _lib.load().hqekv_importance_scores(w.data_ptr(), w.shape[0], w.shape[1], n, total, imp.data_ptr(),
                                                         scores.data_ptr(), _lib.stream_ptr(w.device))
            _lib.check(rc, "importance_scores")
            return imp, RankedBlocks(scores, 32)
        imp = self.calculate_token_importance()[:total].clone()
        return imp, rank_blocks(32, total // 32, imp)

    def eviction(self, reserve_idx: torch.Tensor) -> None:
        """Keep the columns ``reserve_idx`` (ascending positions of the survivors), packed to the left."""
        if self.weights is None:
            return
        kept = torch.index_select(self.weights, 1, reserve_idx)
        self.weights.narrow(1, 0, kept.shape[1]).copy_(kept)

    def decode_row(self, like: torch.Tensor, T: int) -> torch.Tensor:
        """The (T,) slot the next decode row belongs in, for a caller that has the row written by the kernels
        (``hqekv_decode_step`` / ``hqekv_ring_row``) instead of calling ``update``; follow it with ``advance(T)``."""
        if self.weights is None:
            self.weights = like.new_zeros(self.last_length, self.max_length)
        return self.weights[self.next_line, :T]

    def advance(self, T: int) -> None:
        """Bookkeeping of ``update`` for one decode row that has been written in place."""
        self.kv_seq_len = T
        self.next_line = (self.next_line + 1) % self.last_length

    def update(self, attn_weights: torch.Tensor) -> None:
        """attn_weights (B, H, L, T): a prompt (L > 1) stores its last rows, a decode step (L == 1) one ring row.
        The sums run over the batch first and over the heads second, each rounded to the store's dtype."""
        if self.weights is None:
            self.weights = attn_weights.new_zeros(self.last_length, self.max_length)
        L, T = attn_weights.shape[2], attn_weights.shape[3]
        if L > 1:
            rows = min(L, self.last_length)
            self.weights[:rows, :T] = attn_weights[:, :, L - rows:, :].sum(0).sum(0)
        else:
            rows = 1
            if attn_weights.is_cuda and self.weights.dtype == attn_weights.dtype:
                from .attention import ring_order, ring_row_on_device_applies
                if ring_row_on_device_applies(attn_weights):
                    # one launch for any batch size, in the order torch's own reduction adds the rows
                    from . import _lib
                    line = self.weights[self.next_line, :T]
                    with _lib.on_device(attn_weights.device):
                        rc = _lib.load().hqekv_ring_row(attn_weights.data_ptr(), attn_weights.shape[0], attn_weights.shape[1], T,
                                                        line.data_ptr(), ring_order(T, attn_weights),
                                                        _lib.stream_ptr(attn_weights.device))
                    _lib.check(rc, "ring_row")
                    self.advance(T)
                    return
            per_head = attn_weights[0] if attn_weights.shape[0] == 1 else attn_weights.sum(0)
            line = self.weights[self.next_line:self.next_line + 1, :T]
            if line.dtype == per_head.dtype:
                torch.sum(per_head, dim=0, out=line)   # one reduction, written in place
            else:
                line.copy_(per_head.sum(0))
        self.kv_seq_len = T
        self.next_line = (self.next_line + rows) % self.last_length
