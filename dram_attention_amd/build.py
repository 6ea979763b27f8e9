"""Compile libdramattn.so (gfx950) from csrc/ with hipcc.

Run as ``python -m dram_attention_amd.build``; ``__graft_entry__.build()`` calls
:func:`build_library`.  The library is built in-tree next to this file.
"""

from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB_PATH = HERE / "libdramattn.so"
SOURCES = (
    "api.hip",
    "page_minmax.hip",
    "pages_build.hip",
    "page_score.hip",
    "topk_pages.hip",
    "lru_update.hip",
    "decode_attention.hip",
    "stream_attention.hip",
)
# packed fp32 VALU ops are switched off for every device compile of this library
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libdramattn.so cannot be built")
    return exe


def build_library(verbose: bool = False) -> Path:
    """Compile every kernel source and link the shared library; returns its path."""
    hipcc = _hipcc()
    objdir = HERE / "build"
    objdir.mkdir(exist_ok=True)

    def compile_one(src: str) -> Path:
        obj = objdir / (src + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
