"""The C-ABI library loads on a machine without a GPU and exports every symbol include/hqekv.h declares."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def _declared():
    text = (ROOT / "include" / "hqekv.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hqekv_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from hqekv_amd import _lib
    assert sorted(_lib.EXPORTS) == _declared()
    assert sorted(_lib._PROTOS) == _declared()


def test_library_exports_every_declared_symbol():
    from hqekv_amd import _lib
    if not _lib.lib_path().exists():
        pytest.fail(f"{_lib.lib_path()} not built: run `python -m hqekv_amd.build`")
    lib = ctypes.CDLL(str(_lib.lib_path()))
    for name in _declared():
        assert hasattr(lib, name), name
    assert _lib.load().hqekv_version() >= 1


def test_argument_validation_without_a_gpu():
    """Invalid arguments are rejected before anything touches a device."""
    from hqekv_amd import _lib
    lib = _lib.load()
    rc = lib.hqekv_quant_pack_rows(None, 0, 0, None, 0, 0, None, None, 0, 0, 1, 1, 64, 3, None)
    assert rc == -1 and b"bits" in lib.hqekv_last_error()
    rc = lib.hqekv_quant_pack_rows(None, 0, 0, None, 0, 0, None, None, 0, 0, 1, 1, 48, 2, None)
    assert rc == -1
    rc = lib.hqekv_gemv_uniform_group(None, None, None, None, None, 1, 4, 1, 128, 48, 2, None, 0, None)
    assert rc == -1
    rc = lib.hqekv_qk_hybrid(None, 0, None, None, 1, 6, 4, 128, 10, None)
    assert rc == -1  # Hq % Hkv
    rc = lib.hqekv_qk_hybrid(None, 0, None, None, 1, 12, 4, 128, 10, None)
    assert rc == -4  # GQA group of 3 unsupported
    with pytest.raises(ValueError):
        _lib.check(-1, "x")
    with pytest.raises(RuntimeError):
        _lib.check(700, "x")
