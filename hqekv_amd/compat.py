"""Make the reference's import names resolve to this package.

The reference's modules import each other as top-level names (``from pack_unpack import ...``,
quant/hqe_2.py:6; ``from matmul import ...``, quant/hqe_matmul.py:10; ``from model.public_func import
...``, quant/hqe_2.py:1) and as ``quant.<name>`` (model/llama_hqe.py:23-25).  ``install()`` registers
both spellings in ``sys.modules`` so model code written against the reference runs unchanged.
"""
from __future__ import annotations

import importlib
import sys
import types

_MODULES = ("pack_unpack", "matmul", "quant_matmul_hq", "hqe_matmul", "hybrid_quant", "hqe_2", "hqe")


def install(force: bool = False) -> None:
    quant = sys.modules.get("quant")
    if quant is None or force:
        quant = types.ModuleType("quant")
        quant.__path__ = []  # a namespace for the aliases below
        sys.modules["quant"] = quant
    for name in _MODULES:
        mod = importlib.import_module(f"hqekv_amd.{name}")
        for alias in (name, f"quant.{name}"):
            if force or alias not in sys.modules:
                sys.modules[alias] = mod
        setattr(quant, name, mod)
    pf = importlib.import_module("hqekv_amd.public_func")
    model = sys.modules.get("model")
    if model is None or force:
        model = types.ModuleType("model")
        model.__path__ = []
        sys.modules["model"] = model
    if force or "model.public_func" not in sys.modules:
        sys.modules["model.public_func"] = pf
    setattr(model, "public_func", pf)
