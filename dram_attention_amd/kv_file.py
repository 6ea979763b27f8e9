"""Per-layer KV cache files, in the format of the reference's chat example:
``<cache_dir>/NN_cache.pth`` is ``torch.save({"cache_k": k, "cache_v": v})`` with
k, v the prompt's keys and values (1, S, Hkv, D) as CPU tensors
(writer: examples/long-qa-chat/model.py:205-217, reader: examples/long-qa-chat/chat.py:214-233
of the reference).
"""

from __future__ import annotations

import os
from typing import Tuple

import torch


def layer_cache_path(cache_dir: str, index: int) -> str:
    return os.path.join(cache_dir, f"{index:02d}_cache.pth")


def save_layer_cache(cache_dir: str, index: int, xk: torch.Tensor, xv: torch.Tensor) -> str:
    """Write the prompt's keys / values of layer ``index`` ((1, S, Hkv, D) each)."""
    if xk.shape != xv.shape or xk.dim() != 4 or xk.shape[0] != 1:
        raise ValueError(f"expected (1, S, Hkv, D) keys and values, got {tuple(xk.shape)} and "
                         f"{tuple(xv.shape)}")
    os.makedirs(cache_dir, exist_ok=True)
    path = layer_cache_path(cache_dir, index)
    torch.save({"cache_k": xk.to(device="cpu"), "cache_v": xv.to(device="cpu")}, path)
    return path


def load_layer_cache(cache_dir: str, index: int, device="cuda") -> Tuple[torch.Tensor, torch.Tensor]:
    """Read layer ``index``'s file and return (cache_k, cache_v) on ``device``.  The file
    is memory-mapped and loaded with ``weights_only=True`` (nothing in it is executed),
    so a 1M-token layer (4.3 GB) is never held twice in host memory."""
    path = layer_cache_path(cache_dir, index)
    cache = torch.load(path, map_location="cpu", mmap=True, weights_only=True)
    missing = {"cache_k", "cache_v"} - set(cache)
    if missing:
        raise KeyError(f"{path}: missing {sorted(missing)}")
    k, v = cache["cache_k"], cache["cache_v"]
    if k.shape != v.shape or k.dim() != 4 or k.shape[0] != 1:
        raise ValueError(f"{path}: expected (1, S, Hkv, D) tensors, got {tuple(k.shape)} and "
                         f"{tuple(v.shape)}")
    return k.to(device), v.to(device)
