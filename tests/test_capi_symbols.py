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
    assert rc == -1  # a group of 3 query heads per KV head is served: only the null pointers are wrong
    rc = lib.hqekv_qk_hybrid(None, 0, None, None, 1, 130, 2, 128, 10, None)
    assert rc == -4 and b"up to 64" in lib.hqekv_last_error()
    rc = lib.hqekv_normal1_quant_pack_rows(None, 0, 0, None, 0, 0, None, None, 0, 0, 1, 1, 48, None)
    assert rc == -1 and b"multiple of 32" in lib.hqekv_last_error()
    rc = lib.hqekv_normal1_quant_pack_k_tokenmajor(None, 0, 0, None, 0, 0, None, None, 0, 0, 1, 64, 127, None)
    assert rc == -1
    rc = lib.hqekv_normal1_dequant_unpack_rows(None, 0, 0, None, None, 0, 0, None, 0, 0, 1, 1, 64, None)
    assert rc == -1 and b"null" in lib.hqekv_last_error()
    assert lib.hqekv_selftest_wave_reduce(None, None, 4, None) == -1
    assert lib.hqekv_selftest_quant_division(None, None) == -1
    assert lib.hqekv_selftest_stream_read(None, 16, None, 1, None) == -1
    assert lib.hqekv_selftest_stream_read(16, 16, 16, 0, None) == -1
    assert lib.hqekv_selftest_stream_read(16, 24, 16, 1, None) == -2
    # cache migration: class tables are checked before anything is launched
    cc = (_lib.CacheClass * 2)()
    cc[0].bits, cc[0].n_tokens, cc[0].data = 16, 48, 256
    assert lib.hqekv_cache_migrate(1, cc, 1, cc, 1, None, 4, 128, None, None) == -1 and b"whole blocks" in lib.hqekv_last_error()
    cc[0].n_tokens = 64
    assert lib.hqekv_cache_migrate(1, cc, 1, cc, 1, None, 4, 128, None, None) == -1 and b"null plan" in lib.hqekv_last_error()
    cc[0].bits = 3
    assert lib.hqekv_cache_migrate(0, cc, 1, cc, 1, None, 4, 128, None, None) == -1
    assert lib.hqekv_cache_migrate(0, cc, 9, cc, 1, None, 4, 128, None, None) == -1
    # a segment table with an unknown bit width
    segs = _lib.make_segs([dict(bits=3, n_tokens=32, data=None)])
    segs[0].data = 16
    assert lib.hqekv_qk_hybrid(segs, 1, None, None, 1, 4, 4, 128, 32, None) == -1
    with pytest.raises(ValueError):
        _lib.check(-1, "x")
    with pytest.raises(RuntimeError):
        _lib.check(700, "x")


def test_reference_import_names_resolve():
    """`from pack_unpack import ...`, `from quant.hqe_matmul import ...`, `from model.public_func import ...`"""
    import importlib
    import sys
    from hqekv_amd import compat
    saved = {k: sys.modules.get(k) for k in list(sys.modules) if k.split(".")[0] in ("quant", "model") or k in compat._MODULES}
    try:
        compat.install(force=True)
        from pack_unpack import uniform_group_quantize_pack_last_dim  # noqa: F401
        from matmul import cuda_bmm_fA_qB_uniform_group, cuda_bmm_forward_qk_group_hq  # noqa: F401
        # the three import lines of the model files (model/llama_hqe.py:23-25), verbatim
        from quant.hqe import KV_cache_hqe
        from quant.hqe_2 import KV_cache_hqe_2  # noqa: F401
        from quant.hqe_matmul import qkv_matmul_hqe, qkv_matmul_hqe_2  # noqa: F401
        with pytest.raises(NotImplementedError):  # imported there, never called: the per-token-K generation
            KV_cache_hqe((None,) * 42, 32, 0, None, None, None, None, "uniform_group")
        with pytest.raises(NotImplementedError):
            qkv_matmul_hqe(None, (None,) * 42, None, 128, "high_uniform_group_low_normal_group")
        from quant.quant_matmul_hq import qkv_matmul, qkv_matmul_hq  # noqa: F401
        from quant.hybrid_quant import KV_cache_compress, KV_cache_reconstruct  # noqa: F401
        from model.public_func import get_block_token_idx, last_attn_weights, make_sum_equal  # noqa: F401
        assert importlib.import_module("quant.pack_unpack") is importlib.import_module("hqekv_amd.pack_unpack")
    finally:
        for k in list(sys.modules):
            if (k.split(".")[0] in ("quant", "model") or k in compat._MODULES) and k not in saved:
                del sys.modules[k]
        for k, v in saved.items():
            if v is not None:
                sys.modules[k] = v


def test_host_helpers_match_oracle():
    import torch
    from hqekv_amd import public_func as P
    from oracle import hqe_oracle as O
    g = torch.Generator().manual_seed(0)
    imp = torch.rand(256, generator=g)
    assert torch.equal(P.get_block_token_idx(32, 8, imp.clone()), O.get_block_token_idx(32, 8, imp))
    v = torch.randn(2, 3, 16, 32, generator=g).half()
    assert torch.equal(P.calculate_token_range(v, None), O.calculate_token_range(v, None))
    a = torch.tensor([2, 0, 10, 10, 10, 5])
    for target in (35, 40, 25):
        assert P.make_sum_equal(a.clone(), target).tolist() == O.make_sum_equal(a, target).tolist()
    lw = P.last_attn_weights(4)
    lw.set_max_length(8)
    for step in range(6):
        lw.update(torch.full((1, 2, 1, 5 + (step > 2)), float(step + 1)))
    # ring of the last 4 decode rows, each summed over 2 heads; columns seen by fewer rows divide by fewer
    imp2 = lw.calculate_token_importance()
    assert imp2.shape == (6,) and abs(float(imp2[0]) - 2 * (3 + 4 + 5 + 6) / 4) < 1e-6


@pytest.mark.parametrize("batch", [1, 3])
def test_importance_ring_matches_oracle(batch):
    """Decode rows written straight into the ring (one reduction, no temporary) against the oracle's
    ``.sum(0).sum(0)`` + slice assignment, fp16, growing length, more steps than the ring has rows."""
    import torch
    from hqekv_amd import public_func as P
    from oracle import hqe_oracle as O
    g = torch.Generator().manual_seed(5)
    a, b = P.last_attn_weights(20), O.ImportanceRing(20, 300)
    a.set_max_length(300)
    prompt = torch.rand(batch, 8, 20, 200, generator=g).half()
    a.update(prompt)
    b.update(prompt)
    for step in range(45):
        w = torch.rand(batch, 8, 1, 201 + step, generator=g).half()
        a.update(w)
        b.update(w)
        assert a.next_line == b.next_line and a.kv_seq_len == b.kv_seq_len
    assert torch.equal(a.weights, b.weights)
    assert torch.equal(a.calculate_token_importance(), b.importance())
