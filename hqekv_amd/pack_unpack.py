"""Drop-in for the reference's ``quant/pack_unpack.py`` (uniform-group family) on HIP kernels.

Same names, argument order and return shapes/dtypes as quant/pack_unpack.py:53-70 (pack),
:134-154 (fake quant), :156-193 (quantise+pack), :281-295 (unpack), :316-333 (dequantise).
Every function launches hand-written gfx950 kernels through libhqekv.so; there is no torch
or CPU fallback.  Differences from the reference that callers can observe:
  * the input tensor is never modified (the reference's ``sub_``/``div_`` write through a view),
  * a group whose elements are all equal quantises to code 0 (the reference reaches the same
    codes through NaN -> int conversion),
  * ``group_size`` must be 32.
"""
from __future__ import annotations

from typing import Tuple

import torch

from . import _lib

GROUP = 32
n_bits_range = [8, 4, 2, 1]

_QUANTILES = {}


def _normal_tables():
    # quant/pack_unpack.py:6-14 -- kept for importers; the kernels hold the 1-bit entries as constants
    if not _QUANTILES:
        from scipy.stats import norm
        ub = {n: torch.tensor(norm.ppf(torch.arange(0, 1, 1 / (2 ** n)) + 1 / (2 ** n)), dtype=torch.float32)
              for n in n_bits_range}
        ct = {n: torch.tensor(norm.ppf(torch.arange(0, 1, 1 / (2 ** n)) + 0.5 / (2 ** n)), dtype=torch.float32)
              for n in n_bits_range}
        _QUANTILES["ub"], _QUANTILES["ct"] = ub, ct
    return _QUANTILES["ub"], _QUANTILES["ct"]


def __getattr__(name):
    if name == "normal_quantiles_upper_bound":
        return _normal_tables()[0]
    if name == "normal_quantiles_center":
        return _normal_tables()[1]
    raise AttributeError(name)


def _check_bits(bit: int) -> int:
    if bit not in (1, 2, 4, 8):
        raise ValueError(f"bit must be 1, 2, 4 or 8 (got {bit})")
    return 32 // bit


def _check_group(group_size: int) -> None:
    if group_size != GROUP:
        raise ValueError(f"group_size must be {GROUP} (got {group_size})")


def pack_along_last_dim(data: torch.Tensor, bit: int) -> torch.Tensor:
    """(B, nh, D, T) int32 codes -> (B, nh, D, T // (32 // bit)) int32 words, LSB first."""
    pf = _check_bits(bit)
    _lib.require_gpu(data, "data")
    if data.dtype != torch.int32:
        raise TypeError("data must be int32")
    B, nh, D, T = data.shape
    if T % pf:
        raise ValueError("last dim must be a multiple of 32 // bit")
    data = data.contiguous()
    code = torch.empty(B, nh, D, T // pf, dtype=torch.int32, device=data.device)
    with _lib.on_device(data.device):
        _lib.check(_lib.load().hqekv_pack_i32(data.data_ptr(), code.data_ptr(), B * nh * D, T, bit,
                                              _lib.stream_ptr(data.device)), "pack_along_last_dim")
    return code


def unpack_along_last_dim(code: torch.Tensor, bit: int) -> torch.Tensor:
    """(B, nh, D, T/pf) int32 -> (B, nh, D, T) fp16 holding the integer codes."""
    pf = _check_bits(bit)
    _lib.require_gpu(code, "code")
    if code.dtype != torch.int32:
        raise TypeError("code must be int32")
    B, nh, D, Td = code.shape
    code = code.contiguous()
    T = Td * pf
    out = torch.empty(B, nh, D, T, dtype=torch.float16, device=code.device)
    with _lib.on_device(code.device):
        _lib.check(_lib.load().hqekv_dequant_unpack_rows(
            code.data_ptr(), 0, Td, None, None, 0, 0, out.data_ptr(), 0, T, 1, B * nh * D, T, bit,
            _lib.stream_ptr(code.device)), "unpack_along_last_dim")
    return out


def quantize_pack_into(
    data: torch.Tensor, bit: int, code: torch.Tensor, scale: torch.Tensor, mn: torch.Tensor
) -> None:
    """Quantise ``data`` (B, nh, R, L) along L into caller-provided (possibly strided) outputs.

    ``code`` (B, nh, R, L/pf) int32 and ``scale``/``mn`` (B, nh, R, L/32) fp16 may be windows of
    larger capacity-sized buffers (unit stride on the last axis); this is the append path.
    ``data`` may be contiguous or the ``.transpose(2, 3)`` view of a token-major tensor (how the
    reference hands K to its quantiser, quant/hqe_2.py:32-35), which is read in place.
    """
    pf = _check_bits(bit)
    _lib.require_gpu(data, "data")
    if data.dtype != torch.float16:
        raise TypeError("data must be float16")
    B, nh, R, L = data.shape
    if L % GROUP:
        raise ValueError("last dim must be a multiple of 32")
    if tuple(code.shape) != (B, nh, R, L // pf) or tuple(scale.shape) != (B, nh, R, L // GROUP) \
            or tuple(mn.shape) != tuple(scale.shape):
        raise ValueError("output shapes do not match the input")
    if code.dtype != torch.int32 or scale.dtype != torch.float16 or mn.dtype != torch.float16:
        raise TypeError("outputs must be int32 / float16 / float16")
    if data.numel() == 0:
        return
    for t in (code, scale, mn):
        if t.numel() and (t.stride(-1) != 1 or t.stride(0) != nh * t.stride(1)):
            raise ValueError("outputs need a unit last stride and a flattenable (B, nh) prefix")
    if scale.stride() != mn.stride():
        raise ValueError("scale and mn must share strides")
    lib = _lib.load()
    st = _lib.stream_ptr(data.device)
    with _lib.on_device(data.device):
        tm = (data.stride(2) == 1 and data.stride(3) == R and data.stride(1) == R * L
              and data.stride(0) == nh * R * L and R % 2 == 0 and R > 1)
        if tm:
            # token-major memory (B, nh, L, R): groups of 32 tokens per channel, read in place
            _lib.check(lib.hqekv_quant_pack_k_tokenmajor(
                data.data_ptr(), R * L, R, code.data_ptr(), code.stride(1), code.stride(2),
                scale.data_ptr(), mn.data_ptr(), scale.stride(1), scale.stride(2),
                B * nh, L, R, bit, st), "uniform_group_quantize_pack_last_dim")
        else:
            if not data.is_contiguous():
                data = data.contiguous()
            _lib.check(lib.hqekv_quant_pack_rows(
                data.data_ptr(), R * L, L, code.data_ptr(), code.stride(1), code.stride(2),
                scale.data_ptr(), mn.data_ptr(), scale.stride(1), scale.stride(2),
                B * nh, R, L, bit, st), "uniform_group_quantize_pack_last_dim")


def uniform_group_quantize_pack_last_dim(
    data: torch.Tensor, group_size: int, bit: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Asymmetric min/max quantiser over groups of 32 along the last dim, packed LSB first.

    Returns ``(code (B,nh,D,T/pf) int32, scale (B,nh,D,T/32) fp16, mn (B,nh,D,T/32) fp16)``.
    """
    _check_group(group_size)
    pf = _check_bits(bit)
    B, nh, D, T = data.shape
    dev = data.device
    code = torch.empty(B, nh, D, T // pf, dtype=torch.int32, device=dev)
    scale = torch.empty(B, nh, D, T // GROUP, dtype=torch.float16, device=dev)
    mn = torch.empty_like(scale)
    quantize_pack_into(data, bit, code, scale, mn)
    return code, scale, mn


def uniform_group_dequantize_unpack_last_dim(
    code: torch.Tensor, scale: torch.Tensor, mn: torch.Tensor, group_size: int, bit: int
) -> torch.Tensor:
    """fp16 ``rnd16(rnd16(code * scale) + mn)`` of shape (B, nh, D, T)."""
    _check_group(group_size)
    pf = _check_bits(bit)
    _lib.require_gpu(code, "code")
    B, nh, D, Td = code.shape
    T = Td * pf
    if code.dtype != torch.int32 or scale.dtype != torch.float16 or mn.dtype != torch.float16:
        raise TypeError("code must be int32, scale/mn float16")
    if T % GROUP or tuple(scale.shape) != (B, nh, D, T // GROUP) or tuple(mn.shape) != tuple(scale.shape):
        raise ValueError("scale/mn shapes do not match the codes")
    code, scale, mn = code.contiguous(), scale.contiguous(), mn.contiguous()
    out = torch.empty(B, nh, D, T, dtype=torch.float16, device=code.device)
    with _lib.on_device(code.device):
        _lib.check(_lib.load().hqekv_dequant_unpack_rows(
            code.data_ptr(), 0, Td, scale.data_ptr(), mn.data_ptr(), 0, T // GROUP,
            out.data_ptr(), 0, T, 1, B * nh * D, T, bit, _lib.stream_ptr(code.device)),
            "uniform_group_dequantize_unpack_last_dim")
    return out


def uniform_group_fake_quant(data: torch.Tensor, group_size: int, bit: int):
    """Quantise then dequantise (quant/pack_unpack.py:134-154); ``bit == 0`` returns 0."""
    if bit == 0:
        return 0
    code, scale, mn = uniform_group_quantize_pack_last_dim(data, group_size, bit)
    return uniform_group_dequantize_unpack_last_dim(code, scale, mn, group_size, bit)


def normal_group_quantize_pack_last_dim(data: torch.Tensor, group_size: int, bit: int):
    """The 1-bit normal-quantile quantiser (quant/pack_unpack.py:218-253 with bit == 1):
    -> ``(code (B,nh,D,T/32) int32, std (B,nh,D,T/32) fp16, mean (B,nh,D,T/32) fp16)``, code = [x > mean] after
    the reference's fp16 steps.  Other bit widths of the normal family are not built."""
    _check_group(group_size)
    if bit != 1:
        raise NotImplementedError("only the 1-bit table of the normal-quantile family is on the decode path")
    _lib.require_gpu(data, "data")
    if data.dtype != torch.float16:
        raise TypeError("data must be float16")
    B, nh, R, L = data.shape
    if L % GROUP:
        raise ValueError("last dim must be a multiple of 32")
    dev = data.device
    code = torch.empty(B, nh, R, L // 32, dtype=torch.int32, device=dev)
    std = torch.empty(B, nh, R, L // GROUP, dtype=torch.float16, device=dev)
    mean = torch.empty_like(std)
    if data.numel() == 0:
        return code, std, mean
    lib = _lib.load()
    st = _lib.stream_ptr(dev)
    with _lib.on_device(dev):
        tm = (data.stride(2) == 1 and data.stride(3) == R and data.stride(1) == R * L
              and data.stride(0) == nh * R * L and R % 2 == 0 and R > 1)
        if tm:   # the transposed view of token-major K, read in place
            _lib.check(lib.hqekv_normal1_quant_pack_k_tokenmajor(
                data.data_ptr(), R * L, R, code.data_ptr(), code.stride(1), code.stride(2),
                std.data_ptr(), mean.data_ptr(), std.stride(1), std.stride(2), B * nh, L, R, st),
                "normal_group_quantize_pack_last_dim")
        else:
            if not data.is_contiguous():
                data = data.contiguous()
            _lib.check(lib.hqekv_normal1_quant_pack_rows(
                data.data_ptr(), R * L, L, code.data_ptr(), code.stride(1), code.stride(2),
                std.data_ptr(), mean.data_ptr(), std.stride(1), std.stride(2), B * nh, R, L, st),
                "normal_group_quantize_pack_last_dim")
    return code, std, mean


def normal_group_dequantize_unpack_last_dim(code: torch.Tensor, std: torch.Tensor, mean: torch.Tensor,
                                            group_size: int, bit: int) -> torch.Tensor:
    """fp16 ``rnd16(rnd16(+-fp16(0.6745) * std) + mean)`` of shape (B, nh, D, T) (quant/pack_unpack.py:356-376,
    bit == 1)."""
    _check_group(group_size)
    if bit != 1:
        raise NotImplementedError("only the 1-bit table of the normal-quantile family is on the decode path")
    _lib.require_gpu(code, "code")
    B, nh, D, Td = code.shape
    T = Td * 32
    if code.dtype != torch.int32 or std.dtype != torch.float16 or mean.dtype != torch.float16:
        raise TypeError("code must be int32, std/mean float16")
    if tuple(std.shape) != (B, nh, D, T // GROUP) or tuple(mean.shape) != tuple(std.shape):
        raise ValueError("std/mean shapes do not match the codes")
    code, std, mean = code.contiguous(), std.contiguous(), mean.contiguous()
    out = torch.empty(B, nh, D, T, dtype=torch.float16, device=code.device)
    with _lib.on_device(code.device):
        _lib.check(_lib.load().hqekv_normal1_dequant_unpack_rows(
            code.data_ptr(), 0, Td, std.data_ptr(), mean.data_ptr(), 0, T // GROUP,
            out.data_ptr(), 0, T, 1, B * nh * D, T, _lib.stream_ptr(code.device)),
            "normal_group_dequantize_unpack_last_dim")
    return out


def normal_group_fake_quant(data: torch.Tensor, group_size: int, bit: int):
    """quant/pack_unpack.py:195-216 for bit == 1 (``bit == 0`` returns 0)."""
    if bit == 0:
        return 0
    code, std, mean = normal_group_quantize_pack_last_dim(data, group_size, bit)
    return normal_group_dequantize_unpack_last_dim(code, std, mean, group_size, bit)


def _not_built(name):
    def f(*a, **k):
        raise NotImplementedError(
            f"{name} belongs to the per-row / normal-quantile families, which are not part of the "
            "uniform-group decode path this library implements")
    f.__name__ = name
    return f


uniform_quantize_pack_last_dim = _not_built("uniform_quantize_pack_last_dim")
uniform_dequantize_unpack_last_dim = _not_built("uniform_dequantize_unpack_last_dim")
normal_quantize_pack_last_dim = _not_built("normal_quantize_pack_last_dim")
normal_dequantize_unpack_last_dim = _not_built("normal_dequantize_unpack_last_dim")
