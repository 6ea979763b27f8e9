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


def check_hand_placed_registers(verbose: bool = False) -> None:
    """The tile scorer (csrc/page_score_tile.hpp) places a few vector instructions by
    inline asm, which the compiler's tracking of matrix-core hazards does not see.
    Its safety rule is that those instructions write only registers no MFMA of the
    kernel ever names as an operand or destination.  This reads the compiler's own
    listing of page_score.hip and fails the build if any variant breaks the rule."""
    import re

    hipcc = _hipcc()
    listing = HERE / "build" / "page_score.s"
    cmd = [hipcc, *[f for f in HIPCC_FLAGS if f != "-fPIC"], "-S", "--cuda-device-only",
           str(CSRC / "page_score.hip"), "-o", str(listing)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc -S failed on page_score.hip:\n{proc.stderr}")
    text = listing.read_text()
    names = re.findall(r"^(_ZN2da22page_score_tile_kernel[^\s:]*):", text, re.M)
    if not names:
        raise RuntimeError("no page_score_tile_kernel in the listing of page_score.hip")
    for name in names:
        start = text.index("\n" + name + ":")
        lines = text[start:text.index("s_endpgm", start)].splitlines()
        placed, matrix, labels, loops = {}, {}, {}, []
        for n, line in enumerate(lines):
            m = re.match(r"\s+(v_dot2_f32_bf16|v_bfi_b32|v_mov_b32) v(\d+),", line)
            if m:
                placed.setdefault(int(m.group(2)), []).append(n)
            m = re.match(r"\s+v_mfma\S+ (.*)", line)
            if m:
                for lo, hi in re.findall(r"v\[(\d+):(\d+)\]", m.group(1)):
                    for r in range(int(lo), int(hi) + 1):
                        matrix.setdefault(r, []).append(n)
            m = re.match(r"(\.LBB\w+):", line)
            if m:
                labels[m.group(1)] = n
            m = re.match(r"\s+s_cbranch\w*\s+(\.LBB\w+)|\s+s_branch\s+(\.LBB\w+)", line)
            if m:
                target = labels.get(m.group(1) or m.group(2))
                if target is not None:          # a label already seen: a backward branch, i.e. a loop
                    loops.append((target, n))
        if len(placed) != 8 or not matrix:
            raise RuntimeError(f"{name}: expected 8 hand-placed destinations and some MFMAs, "
                               f"found {len(placed)} and {len(matrix)} registers")
        # A register may serve both only when every MFMA that names it comes after
        # the last hand-placed write to it (the variable behind it is dead by then),
        # in straight-line code: never inside a loop that also holds such a write.
        for r in sorted(set(placed) & set(matrix)):
            last_write, first_use = max(placed[r]), min(matrix[r])
            in_one_loop = any(lo <= w <= hi and lo <= u <= hi for lo, hi in loops
                              for w in placed[r] for u in matrix[r])
            if first_use < last_write or in_one_loop:
                raise RuntimeError(f"{name}: register v{r} is written by a hand-placed "
                                   "instruction while an MFMA may still use it")
    if verbose:
        print(f"hand-placed registers of {len(names)} tile scorer variants are clear of MFMA operands")


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
    check_hand_placed_registers(verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
