"""Build libhqekv.so (hand-written HIP for gfx950) in-tree with hipcc.

``python -m hqekv_amd.build`` compiles every source under ``hqekv_amd/csrc`` and links
``hqekv_amd/libhqekv.so``.  hipcc cross-compiles for gfx950 without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB = PKG / "libhqekv.so"
SOURCES = ["capi.hip", "quant_pack.hip", "attn.hip", "decode_static.hip", "migrate.hip", "planner.hip", "importance.hip", "prompt_attn.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # packed-FP32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + out)
    return out


def build(verbose: bool = False) -> Path:
    hipcc = _hipcc()
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)
    objs = [objdir / (Path(s).stem + ".o") for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        logs = list(ex.map(compile_one, zip(SOURCES, objs)))
    tmp = LIB.with_suffix(".so.tmp")
    logs.append(_run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *map(str, objs), "-o", str(tmp)]))
    os.replace(tmp, LIB)
    if verbose:
        for l in logs:
            if l.strip():
                print(l)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
