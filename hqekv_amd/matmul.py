"""Drop-in for the in-scope wrappers of the reference's ``quant/matmul.py``.

Same names and positional orders as quant/matmul.py:263-299 (``cuda_bmm_fA_qB_uniform_group``),
:736-760 (``cuda_bmm_fA_qB_wv_uniform_group``), :72-95 / :147-170 (``cuda_bmm_fA_qB_normal_group`` and its
p.V twin), :351-434 (``cuda_bmm_forward_qk_group_hq``) and
:507-579 (``cuda_bmm_forward_wv_group_hq``).  The reference flattens and transposes every operand
into a kernel-side layout before each launch; these wrappers hand the stored layouts to the
kernels unchanged.  Only the first row of ``fA`` / ``in_vector`` is computed upstream
(quant/csrc/gemv_cuda_uniform.cu:420), so M must be 1 here.
"""
from __future__ import annotations

import torch

from . import _lib
from . import attention as _att


def _need_f16(t: torch.Tensor, name: str) -> torch.Tensor:
    _lib.require_gpu(t, name)
    if t.dtype != torch.float16:
        raise TypeError(f"{name} must be float16")
    return t.contiguous()


def _gemv_group(entry: str, who: str, group_size: int, fA: torch.Tensor, qB: torch.Tensor, scales: torch.Tensor,
                zeros: torch.Tensor, bits: int, allowed_bits) -> torch.Tensor:
    if group_size != 32:
        raise ValueError("group_size must be 32")
    if bits not in allowed_bits:
        raise ValueError("bits must be " + ", ".join(map(str, allowed_bits)))
    fA = _need_f16(fA, "fA")
    B, nh_q, M, K = fA.shape
    if M != 1:
        raise ValueError("only M == 1 (single-token decode) is computed")
    _lib.require_gpu(qB, "qB")
    if qB.dtype != torch.int32:
        raise TypeError("qB must be int32")
    qB = qB.contiguous()
    scales, zeros = _need_f16(scales, "scales"), _need_f16(zeros, "zeros")
    nh_kv = qB.shape[1]
    N = qB.shape[-1] * (32 // bits)
    if qB.shape[0] != B or qB.shape[2] != K or nh_q % nh_kv:
        raise ValueError("qB shape does not match fA")
    if tuple(scales.shape) != (B, nh_kv, K, N // 32) or tuple(zeros.shape) != tuple(scales.shape):
        raise ValueError("scales/zeros shape does not match qB")
    lib = _lib.load()
    out = torch.empty(B, nh_q, 1, N, dtype=torch.float16, device=fA.device)
    with _lib.on_device(fA.device):
        need = lib.hqekv_gemv_workspace_bytes(B, nh_q, nh_kv, K, N, bits)
        ws = torch.empty(max(need, 16) // 4, dtype=torch.float32, device=fA.device)
        rc = getattr(lib, entry)(fA.data_ptr(), qB.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                                 out.data_ptr(), B, nh_q, nh_kv, K, N, bits, ws.data_ptr(),
                                 ws.numel() * 4, _lib.stream_ptr(fA.device))
    _lib.check(rc, who)
    return out


def cuda_bmm_fA_qB_uniform_group(group_size: int, fA: torch.Tensor, qB: torch.Tensor,
                                 scales: torch.Tensor, zeros: torch.Tensor, bits: int) -> torch.Tensor:
    """C[b,hq,0,n] = sum_k fA[b,hq,0,k] * (scales[b,hkv,k,n/32] * code[b,hkv,k,n] + zeros[b,hkv,k,n/32]).

    fA (B,nh_q,1,K) fp16; qB (B,nh_kv,K,N/pf) int32; scales/zeros (B,nh_kv,K,N/32) fp16 -> (B,nh_q,1,N) fp16.
    q.K^T passes K = head_dim, N = tokens; p.V passes K = tokens, N = head_dim.
    """
    return _gemv_group("hqekv_gemv_uniform_group", "cuda_bmm_fA_qB_uniform_group", group_size, fA, qB, scales,
                       zeros, bits, (1, 2, 4, 8))


# the reference keeps a second entry point for the split-K p.V kernel; the dispatch is internal here
cuda_bmm_fA_qB_wv_uniform_group = cuda_bmm_fA_qB_uniform_group


def cuda_bmm_fA_qB_normal_group(group_size: int, fA: torch.Tensor, qB: torch.Tensor,
                                stds: torch.Tensor, means: torch.Tensor, bits: int) -> torch.Tensor:
    """The same GEMV over normal-quantile codes (quant/matmul.py:72-95; what the attention glue calls for the
    1-bit class under 'high_uniform_group_low_normal_group', quant/hqe_matmul.py:372,424):
    C[b,hq,0,n] = sum_k fA[b,hq,0,k] * dequant(code[b,hkv,k,n]; stds[b,hkv,k,n/32], means[b,hkv,k,n/32]).
    Only ``bits == 1`` (2-entry table -+0.6745) is built; the wider normal-quantile tables are not on the path."""
    if bits in (2, 4, 8):
        raise NotImplementedError("normal-quantile GEMV is built for the 1-bit class only")
    return _gemv_group("hqekv_gemv_normal_group", "cuda_bmm_fA_qB_normal_group", group_size, fA, qB, stds, means,
                       bits, (1,))


# quant/matmul.py:147-170: the split-K p.V twin; one entry serves both shapes here
cuda_bmm_fA_qB_wv_normal_group = cuda_bmm_fA_qB_normal_group


def _hq_tuple(m16, m16_idx, m8, m8_idx, s8, z8, m4, m4_idx, s4, z4, m2, m2_idx, s2, z2,
              m1, m1_idx, s1, z1, new, is_k: bool) -> tuple:
    """Lay the positional arguments of the *_group_hq wrappers into the slots of a 42-tuple."""
    # m1/s1/z1: upstream's fused wrappers take the 1-bit class as (codes, std_1, means_1), the normal-quantile
    # coding (quant/matmul.py:351-373); the segments are built with that layout by the callers below
    t = [None] * 42
    kb, vb = _att.K_BASE, _att.V_BASE
    base = kb if is_k else vb
    t[_att.K16 if is_k else _att.V16] = m16
    t[_att.K16_IDX if is_k else _att.V16_IDX] = m16_idx
    for b, (m, i, s, z) in zip((8, 4, 2, 1), ((m8, m8_idx, s8, z8), (m4, m4_idx, s4, z4), (m2, m2_idx, s2, z2),
                                              (m1, m1_idx, s1, z1))):
        t[base[b]], t[base[b] + 1], t[base[b] + 2], t[base[b] + 3] = m, i, s, z
    t[_att.NEW_K if is_k else _att.NEW_V] = new
    return tuple(t)


def cuda_bmm_forward_qk_group_hq(group_size, nh_kv, in_vector, matrix_16, matrix_16_idx,
                                 matrix_8, matrix_8_idx, scales_8, zeros_8,
                                 matrix_4, matrix_4_idx, scales_4, zeros_4,
                                 matrix_2, matrix_2_idx, scales_2, zeros_2,
                                 matrix_1, matrix_1_idx, std_1, means_1, new_K) -> torch.Tensor:
    """Fused hybrid q.K^T: raw fp16 scores (B,nh_q,1,Tall) scattered through each class's idx, the
    residual ``new_K`` (B,nh_kv,Tn,D) at the tail.  matrix_16 is (B,nh_kv,D,T16)."""
    if group_size != 32:
        raise ValueError("group_size must be 32")
    in_vector = _need_f16(in_vector, "in_vector")
    B, nh_q, M, D = in_vector.shape
    if M != 1:
        raise ValueError("only M == 1 (single-token decode) is computed")
    Tall = 0
    if matrix_16_idx is not None:
        Tall += matrix_16.shape[-1]
    for m, i, b in ((matrix_8, matrix_8_idx, 8), (matrix_4, matrix_4_idx, 4), (matrix_2, matrix_2_idx, 2)):
        if i is not None:
            Tall += m.shape[-1] * (32 // b)
    if matrix_1_idx is not None:
        Tall += matrix_1.shape[-1] * 32
    if new_K is not None:
        Tall += new_K.shape[-2]
    if Tall == 0:
        raise ValueError('invalid matrix.')
    pkv = _hq_tuple(matrix_16, matrix_16_idx, matrix_8, matrix_8_idx, scales_8, zeros_8,
                    matrix_4, matrix_4_idx, scales_4, zeros_4, matrix_2, matrix_2_idx, scales_2, zeros_2,
                    matrix_1, matrix_1_idx, std_1, means_1, new_K, True)
    dev = in_vector.device
    keep: list = []
    items, hk, dk = _att.key_segments(pkv, dev, Tall, keep, low_uniform=False)  # (std_1, means_1): normal-quantile class
    if hk != nh_kv or dk != D:
        raise ValueError("cache shape does not match nh_kv / head_dim")
    out = torch.zeros(B, nh_q, 1, Tall, dtype=torch.float16, device=dev)
    segs = _lib.make_segs(items)
    with _lib.on_device(dev):
        rc = _lib.load().hqekv_qk_hybrid(segs, len(items), in_vector.data_ptr(), out.data_ptr(), B, nh_q,
                                         nh_kv, D, Tall, _lib.stream_ptr(dev))
    _lib.check(rc, "cuda_bmm_forward_qk_group_hq")
    return out


def cuda_bmm_forward_wv_group_hq(group_size, nh_kv, in_vector, matrix_16, matrix_16_idx,
                                 matrix_8, matrix_8_idx, scales_8, zeros_8,
                                 matrix_4, matrix_4_idx, scales_4, zeros_4,
                                 matrix_2, matrix_2_idx, scales_2, zeros_2,
                                 matrix_1, matrix_1_idx, std_1, means_1, new_V) -> torch.Tensor:
    """Fused hybrid p.V: in_vector (B,nh_q,1,Tall) probabilities gathered through each class's idx,
    the residual ``new_V`` (B,nh_kv,Tn,D) weighted by the tail.  Returns (B,nh_q,1,D) fp16."""
    if group_size != 32:
        raise ValueError("group_size must be 32")
    in_vector = _need_f16(in_vector, "in_vector")
    B, nh_q, M, Tall = in_vector.shape
    if M != 1:
        raise ValueError("only M == 1 (single-token decode) is computed")
    pkv = _hq_tuple(matrix_16, matrix_16_idx, matrix_8, matrix_8_idx, scales_8, zeros_8,
                    matrix_4, matrix_4_idx, scales_4, zeros_4, matrix_2, matrix_2_idx, scales_2, zeros_2,
                    matrix_1, matrix_1_idx, std_1, means_1, new_V, False)
    dev = in_vector.device
    keep: list = []
    items, hv, D = _att.value_segments(pkv, dev, Tall, keep, low_uniform=False)
    if not items:
        raise ValueError('invalid matrix.')
    if hv != nh_kv:
        raise ValueError("cache shape does not match nh_kv")
    out = torch.empty(B, nh_q, 1, D, dtype=torch.float16, device=dev)
    segs = _lib.make_segs(items)
    with _lib.on_device(dev):
        ws = _att.workspace_for(segs, len(items), B, nh_q, nh_kv, D, dev)
        rc = _lib.load().hqekv_pv_hybrid(segs, len(items), in_vector.data_ptr(), out.data_ptr(), B, nh_q,
                                         nh_kv, D, Tall, ws.data_ptr(), ws.numel() * 4, _lib.stream_ptr(dev))
    _lib.check(rc, "cuda_bmm_forward_wv_group_hq")
    return out
