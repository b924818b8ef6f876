"""ctypes binding of libhqekv.so (the C ABI declared in include/hqekv.h).

The product path has no CPU fallback: if the shared library is missing, or a call fails,
an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path
from typing import Optional

import torch

_PKG = Path(__file__).resolve().parent
_LIB_PATH = Path(os.environ.get("HQEKV_LIB", _PKG / "libhqekv.so"))

MAX_SEGS = 8
FUSE_SOFTMAX = 1
SEPARATE_COMBINE = 2
FOLD_COMBINE = 4
TWO_STEP_DEQUANT = 8
ONLY_QK = 0x100
ONLY_PV = 0x200
ONLY_COMBINE = 0x400
DOT_MFMA = 0x800    # inner products on the matrix cores (Hq/Hkv == 4, or a slice of four of a ratio above 8)
DOT_VALU = 0x1000   # inner products on the vector ALU
ONLY_RAW_QK = 0x2000   # the q.K^T launch alone, raw fp16 scores
QK_TILINGS = {"8waves": 1, "4waves": 2, "wave512": 3, "wave256": 4}   # HQEKV_QK_TILING_*: tilings a call may force


def qk_tiling(n: int) -> int:
    """Flag bits of HQEKV_QK_TILING(n)."""
    return (int(n) & 0xF) << 4


LAYOUT_TOKEN_MAJOR = 1   # fp16 K segment stored (B,Hkv,T,D)
LAYOUT_NORMAL1 = 2       # 1-bit segment in normal-quantile coding (scale = std, zero = mean)

# every symbol include/hqekv.h declares
EXPORTS = (
    "hqekv_version", "hqekv_last_error",
    "hqekv_quant_pack_rows", "hqekv_quant_pack_k_tokenmajor", "hqekv_dequant_unpack_rows", "hqekv_pack_i32",
    "hqekv_selftest_quant_division", "hqekv_selftest_wave_reduce", "hqekv_selftest_stream_read",
    "hqekv_normal1_quant_pack_rows", "hqekv_normal1_quant_pack_k_tokenmajor", "hqekv_normal1_dequant_unpack_rows",
    "hqekv_gemv_workspace_bytes", "hqekv_gemv_uniform_group", "hqekv_gemv_normal_group",
    "hqekv_qk_hybrid", "hqekv_scale_softmax", "hqekv_pv_workspace_bytes", "hqekv_pv_hybrid",
    "hqekv_decode_workspace_bytes", "hqekv_decode_attn", "hqekv_decode_attn_static", "hqekv_decode_step", "hqekv_ring_row",
    "hqekv_importance_scores", "hqekv_weighted_block_scores", "hqekv_token_range",
    "hqekv_prompt_attn", "hqekv_prompt_last_rows", "hqekv_prompt_last_rows_workspace_bytes",
    "hqekv_cache_migrate", "hqekv_plan_side",
)


class Seg(C.Structure):
    """Mirror of ``struct hqekv_seg``."""
    _fields_ = [
        ("bits", C.c_int32),
        ("layout", C.c_int32),
        ("n_tokens", C.c_int64),
        ("pos_base", C.c_int64),
        ("data", C.c_void_p),
        ("scale", C.c_void_p),
        ("zero", C.c_void_p),
        ("idx", C.c_void_p),
        ("slab_tokens", C.c_int64),
    ]


class StepExtra(C.Structure):
    """Mirror of ``struct hqekv_step_extra``."""
    _fields_ = [
        ("ring_line", C.c_void_p),
        ("ring_order", C.c_int32),
        ("append_rows", C.c_int32),
        ("new_k", C.c_void_p),
        ("new_v", C.c_void_p),
        ("k_dst", C.c_void_p),
        ("v_dst", C.c_void_p),
        ("k_dst_slab_tokens", C.c_int64),
        ("v_dst_slab_tokens", C.c_int64),
    ]


class CacheClass(C.Structure):
    """Mirror of ``struct hqekv_cache_class``."""
    _fields_ = [
        ("bits", C.c_int32),
        ("layout", C.c_int32),
        ("n_tokens", C.c_int64),
        ("slab_tokens", C.c_int64),
        ("data", C.c_void_p),
        ("scale", C.c_void_p),
        ("zero", C.c_void_p),
        ("idx", C.c_void_p),
    ]


_lib: Optional[C.CDLL] = None

_i64, _int, _vp = C.c_int64, C.c_int, C.c_void_p
_SEGP = C.POINTER(Seg)
_CCP = C.POINTER(CacheClass)

_PROTOS = {
    "hqekv_version": (C.c_int, []),
    "hqekv_last_error": (C.c_char_p, []),
    "hqekv_quant_pack_rows": (C.c_int, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "hqekv_quant_pack_k_tokenmajor": (C.c_int, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "hqekv_dequant_unpack_rows": (C.c_int, [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "hqekv_pack_i32": (C.c_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "hqekv_selftest_quant_division": (C.c_int, [_vp, _vp]),
    "hqekv_selftest_wave_reduce": (C.c_int, [_vp, _vp, _i64, _vp]),
    "hqekv_selftest_stream_read": (C.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hqekv_normal1_quant_pack_rows": (C.c_int, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "hqekv_normal1_quant_pack_k_tokenmajor": (C.c_int, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "hqekv_normal1_dequant_unpack_rows": (C.c_int, [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "hqekv_gemv_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64, _i64, _int]),
    "hqekv_gemv_uniform_group": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _vp]),
    "hqekv_gemv_normal_group": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _vp]),
    "hqekv_qk_hybrid": (C.c_int, [_SEGP, _int, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "hqekv_scale_softmax": (C.c_int, [_vp, _vp, _i64, _i64, _i64, C.c_float, _vp]),
    "hqekv_pv_workspace_bytes": (_i64, [_SEGP, _int, _i64, _i64, _i64, _i64]),
    "hqekv_pv_hybrid": (C.c_int, [_SEGP, _int, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "hqekv_decode_workspace_bytes": (_i64, [_SEGP, _int, _SEGP, _int, _i64, _i64, _i64, _i64]),
    "hqekv_decode_attn": (C.c_int, [_SEGP, _int, _SEGP, _int, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _int, _vp]),
    "hqekv_decode_step": (C.c_int, [_SEGP, _int, _SEGP, _int, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _int, _vp, C.POINTER(StepExtra)]),
    "hqekv_ring_row": (C.c_int, [_vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "hqekv_importance_scores": (C.c_int, [_vp, C.c_int32, _i64, _i64, _i64, _vp, _vp, _vp]),
    "hqekv_weighted_block_scores": (C.c_int, [_vp, _vp, _i64, _vp, _vp]),
    "hqekv_token_range": (C.c_int, [_vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp]),
    "hqekv_prompt_attn": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float, _int, _vp]),
    "hqekv_prompt_last_rows": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, C.c_float, _vp, _i64, _vp]),
    "hqekv_prompt_last_rows_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "hqekv_decode_attn_static": (C.c_int, [_SEGP, _int, _SEGP, _int, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "hqekv_plan_side": (C.c_int, [C.POINTER(_vp), _vp, C.c_int32, C.c_int32, _vp, _vp, C.c_int32, _vp, _vp, _vp, _vp]),
    "hqekv_cache_migrate": (C.c_int, [_int, _CCP, _int, _CCP, _int, _vp, _i64, _i64, _vp, _vp]),
}
STATIC_SCRATCH_BYTES = 8 << 20   # HQEKV_STATIC_SCRATCH_BYTES


def lib_path() -> Path:
    return _LIB_PATH


def load() -> C.CDLL:
    """Load libhqekv.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m hqekv_amd.build` "
                "(there is no CPU fallback for the HIP path)")
        lib = C.CDLL(str(_LIB_PATH))
        for name, (res, args) in _PROTOS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code into the exception the reference's callers expect."""
    if rc == 0:
        return
    msg = load().hqekv_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise RuntimeError(f"{what}: HIP error {rc}: {msg}")


def stream_ptr(device: torch.device) -> int:
    """Raw handle of torch's current stream on ``device`` (the cheap lookup: this runs once per launch)."""
    idx = device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx)


class on_device:
    """``with on_device(dev):`` -- make ``dev`` the current HIP device for a launch.  Does nothing when it already
    is (one integer comparison instead of torch's two device switches), which is every call of a one-GPU process."""
    __slots__ = ("ctx",)

    def __init__(self, device: torch.device):
        idx = device.index
        self.ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: the HIP path has no CPU fallback")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def make_segs(items) -> "C.Array[Seg]":
    """items: iterable of dicts with keys bits, n_tokens, data, scale, zero, idx, pos_base, token_major."""
    items = list(items)
    if len(items) > MAX_SEGS:
        raise ValueError("too many segments")
    arr = (Seg * max(1, len(items)))()
    for s, it in zip(arr, items):
        s.bits = it["bits"]
        s.layout = LAYOUT_TOKEN_MAJOR if it.get("token_major") else int(it.get("layout", 0))
        s.n_tokens = it["n_tokens"]
        s.pos_base = int(it.get("pos_base", 0))
        s.data = ptr(it["data"])
        s.scale = ptr(it.get("scale"))
        s.zero = ptr(it.get("zero"))
        s.idx = ptr(it.get("idx"))
        s.slab_tokens = int(it.get("slab_tokens", 0))
    return arr
