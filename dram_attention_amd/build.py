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
    "prefill_attention.hip",
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


def check_tile_scorer_listing(text: str) -> int:
    """The rule the hand-placed instructions of the tile scorer (csrc/page_score_tile.hpp)
    must keep, checked on the compiler's own listing ``text`` of page_score.hip; returns
    the number of kernel variants checked and raises RuntimeError naming the kernel and
    the offending line otherwise.

    The scorer places its dot products by inline asm in blocks of eight, which the
    compiler's tracking of matrix-core hazards does not see.  Per variant:
      - the kernel starts by claiming eight registers (eight ``v_mov_b32 vN, 0``: the
        first eight of the kernel) and has at least one MFMA;
      - every ``v_dot2_f32_bf16`` sits in a run of exactly eight, each writing a
        different one of the claimed registers, and the run is closed by ``s_nop 2``
        (the wait a dot product's consumer needs);
      - no claimed register is an operand or destination of an MFMA, unless every such
        MFMA comes after the last hand-placed write to it, in straight-line code
        (never inside a loop that also holds such a write)."""
    import re

    heads = list(re.finditer(r"^(_ZN2da22page_score_tile_kernel[^\s:]*):", text, re.M))
    if not heads:
        raise RuntimeError("no page_score_tile_kernel in the listing of page_score.hip")
    names = [m.group(1) for m in heads]
    for head in heads:
        name, start = head.group(1), head.start()
        lines = text[start:text.index("s_endpgm", start)].splitlines()

        def bad(n, why):
            return RuntimeError(f"{name}: {why} (line {n} of the kernel: {lines[n].strip()!r})")

        claimed, claim_line = [], {}
        writes, matrix, labels, loops, dots = {}, {}, {}, [], []
        for n, line in enumerate(lines):
            m = re.match(r"\s+v_mov_b32 v(\d+), 0\s*$", line)
            if m and len(claimed) < 8 and not dots:
                claimed.append(int(m.group(1)))
                claim_line[int(m.group(1))] = n
            m = re.match(r"\s+v_dot2_f32_bf16 v(\d+),", line)
            if m:
                dots.append((n, int(m.group(1))))
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
        if len(set(claimed)) != 8:
            raise RuntimeError(f"{name}: expected eight registers claimed by v_mov_b32 vN, 0 ahead of "
                               f"the first dot product, found {sorted(set(claimed))}")
        if not matrix:
            raise RuntimeError(f"{name}: no MFMA in the kernel")
        if not dots or len(dots) % 8:
            raise RuntimeError(f"{name}: {len(dots)} hand-placed dot products, not blocks of eight")
        for b in range(0, len(dots), 8):
            block = dots[b:b + 8]
            first = block[0][0]
            for i, (n, reg) in enumerate(block):
                if n != first + i:
                    raise bad(n, "a hand-placed dot product outside a run of eight")
                if reg not in claimed:
                    raise bad(n, f"a hand-placed dot product writes v{reg}, which the kernel never claimed")
            if len({reg for _, reg in block}) != 8:
                raise bad(first, "a block of dot products writes a register twice")
            closing = first + 8
            if closing >= len(lines) or not re.match(r"\s+s_nop 2\s*$", lines[closing]):
                raise bad(min(closing, len(lines) - 1), "a block of dot products is not closed by s_nop 2")
            for n, reg in block:
                writes.setdefault(reg, []).append(n)
        for reg in claimed:
            writes.setdefault(reg, []).append(claim_line[reg])
        # A register may serve both only when every MFMA that names it comes after
        # the last hand-placed write to it (the variable behind it is dead by then),
        # in straight-line code: never inside a loop that also holds such a write.
        for r in sorted(set(writes) & set(matrix)):
            last_write, first_use = max(writes[r]), min(matrix[r])
            in_one_loop = any(lo <= w <= hi and lo <= u <= hi for lo, hi in loops
                              for w in writes[r] for u in matrix[r])
            if first_use < last_write or in_one_loop:
                raise bad(first_use, f"register v{r} is written by a hand-placed instruction while "
                                     "an MFMA may still use it")
    return len(names)


def check_hand_placed_registers(verbose: bool = False) -> None:
    """Compile page_score.hip to a listing and hold it against check_tile_scorer_listing;
    fails the build if any variant of the tile scorer breaks the rule."""
    hipcc = _hipcc()
    (HERE / "build").mkdir(exist_ok=True)
    listing = HERE / "build" / "page_score.s"
    cmd = [hipcc, *[f for f in HIPCC_FLAGS if f != "-fPIC"], "-S", "--cuda-device-only",
           str(CSRC / "page_score.hip"), "-o", str(listing)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc -S failed on page_score.hip:\n{proc.stderr}")
    n = check_tile_scorer_listing(listing.read_text())
    if verbose:
        print(f"hand-placed registers of {n} tile scorer variants are clear of MFMA operands")


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
