"""Prompt-side attention on the library's matrix-core kernels (``csrc/prompt_attn.hip``): the whole-prompt causal
attention the reference takes from flash-attention, and the probabilities of the last query rows it computes with a
dense matmul over ``repeat_kv`` copies [model/llama_hqe.py:141-188].  fp16, head_dim 128; K and V keep their own head
count, and every tensor is read through its strides (slices of a fused QKV projection are not copied)."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib

HEAD_DIM = 128
MAX_LAST_ROWS = 32


def supported(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor] = None) -> bool:
    """fp16 CUDA tensors (B, H, T, 128) whose rows the kernels can read in place or after one copy."""
    ts = [t for t in (q, k, v) if t is not None]
    return all(t.is_cuda and t.dtype == torch.float16 and t.dim() == 4 and t.shape[-1] == HEAD_DIM for t in ts)


def _rows(t: torch.Tensor) -> torch.Tensor:
    """``t`` with unit channel stride and 16-byte aligned rows (a copy only when it has neither)."""
    if t.stride(3) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:3]):
        return t
    return t.contiguous()


def _strides(t: torch.Tensor):
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def prompt_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scaling: float, causal: bool = True) -> torch.Tensor:
    """softmax(q k^T * scaling [causal]) v -> (B, Hq, T, 128) fp16, contiguous."""
    if not supported(q, k, v):
        raise NotImplementedError("prompt_attention: fp16 CUDA tensors of head_dim 128 only")
    B, Hq, T, D = q.shape
    Hkv = k.shape[1]
    q, k, v = _rows(q), _rows(k), _rows(v)
    out = torch.empty((B, Hq, T, D), dtype=q.dtype, device=q.device)
    with _lib.on_device(q.device):
        rc = _lib.load().hqekv_prompt_attn(q.data_ptr(), _strides(q), k.data_ptr(), _strides(k), v.data_ptr(), _strides(v),
                                           out.data_ptr(), _strides(out), B, Hq, Hkv, T, D, float(scaling), 1 if causal else 0,
                                           _lib.stream_ptr(q.device))
    _lib.check(rc, "prompt_attn")
    return out


def prompt_last_rows(q: torch.Tensor, k: torch.Tensor, scaling: float, rows: int,
                     attention_mask: Optional[torch.Tensor] = None, sliced: bool = True) -> torch.Tensor:
    """Probabilities of the last ``rows`` query rows over all keys -> (B, Hq, rows, T) fp16, with the reference's
    roundings.  ``attention_mask``: additive (B or 1, 1, >= rows, T), its last ``rows`` rows are used; None: causal.
    ``sliced``: let the library cut the keys into slices over more workgroups (two launches) when there are few heads."""
    if not supported(q, k):
        raise NotImplementedError("prompt_last_rows: fp16 CUDA tensors of head_dim 128 only")
    B, Hq, T, D = q.shape
    Hkv = k.shape[1]
    if not 0 < rows <= min(MAX_LAST_ROWS, T):
        raise ValueError(f"prompt_last_rows: rows={rows} outside 1..min({MAX_LAST_ROWS}, T={T})")
    q, k = _rows(q), _rows(k)
    m_ptr, m_str = None, None
    if attention_mask is not None:
        if attention_mask.dim() != 4 or attention_mask.shape[1] != 1 or attention_mask.shape[3] != T \
                or attention_mask.shape[0] not in (1, B) or attention_mask.shape[2] < rows:
            raise ValueError(f"prompt_last_rows: mask of shape {tuple(attention_mask.shape)} (expected (B or 1, 1, >= rows, T))")
        m = attention_mask[:, :, -rows:, :]
        if m.dtype != q.dtype or m.stride(3) != 1:
            m = m.to(q.dtype).contiguous()
        m_ptr = m.data_ptr()
        m_str = (C.c_int64 * 2)(m.stride(0) if m.shape[0] > 1 else 0, m.stride(2))
    probs = torch.empty((B, Hq, rows, T), dtype=q.dtype, device=q.device)
    lib = _lib.load()
    ws_bytes = lib.hqekv_prompt_last_rows_workspace_bytes(B, Hq, T) if sliced else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes > 0 else None
    with _lib.on_device(q.device):
        rc = lib.hqekv_prompt_last_rows(q.data_ptr(), _strides(q), k.data_ptr(), _strides(k), m_ptr, m_str,
                                        probs.data_ptr(), B, Hq, Hkv, T, D, rows, float(scaling),
                                        ws.data_ptr() if ws is not None else None, ws_bytes, _lib.stream_ptr(q.device))
    _lib.check(rc, "prompt_last_rows")
    return probs
