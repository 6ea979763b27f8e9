"""ctypes binding of libdramattn.so (declared in include/dram_attention_amd.h).

The library is the only compute backend of this package: every wrapper below
raises if it cannot be loaded; nothing falls back to torch or to the CPU.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "libdramattn.so"

DA_F32, DA_F16, DA_BF16 = 0, 1, 2
DA_I32, DA_I64 = 0, 1
DA_TIME_F32, DA_TIME_I32 = 0, 1

_DTYPES = {torch.float32: DA_F32, torch.float16: DA_F16, torch.bfloat16: DA_BF16}
_ITYPES = {torch.int32: DA_I32, torch.int64: DA_I64}
_TIME_TYPES = {torch.float32: DA_TIME_F32, torch.int32: DA_TIME_I32}

# name -> (restype, argtypes); one line per symbol of the header
SIGNATURES = {
    "da_version": (c_int, []),
    "da_last_error_string": (c_char_p, []),
    "da_host_device_pointer": (c_int, [c_void_p, ctypes.POINTER(c_void_p)]),
    "da_prefill_attention": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
         c_int64, c_int, c_int, c_int, c_int, c_float, c_void_p, c_int64, c_int64, c_void_p,
         c_void_p],
    ),
    "da_page_minmax": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_void_p],
    ),
    "da_pages_build": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int64, c_int, c_int, c_int, c_void_p,
         c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "da_page_score": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int64,
         c_int, c_int, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p],
    ),
    "da_topk_pages_workspace_bytes": (c_size_t, [c_int, c_int, c_int64, c_int]),
    "da_topk_pages": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_int64, c_int, c_void_p, c_int64,
         c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "da_lru_update_workspace_bytes": (c_size_t, [c_int, c_int, c_int64, c_int]),
    "da_lru_update": (
        c_int,
        [c_void_p, c_int64, c_int, c_int, c_int, c_int64, c_int, c_void_p, c_int, c_void_p,
         c_int64, c_int, c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "da_topk_pages_lru": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_int64, c_int, c_void_p, c_int64,
         c_int64, c_int64, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p,
         c_void_p, c_size_t, c_void_p],
    ),
    "da_pages_gather": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_int, c_int, c_int, c_void_p],
    ),
    "da_decode_attention_workspace_bytes": (
        c_size_t, [c_int, c_int, c_int, c_int, c_int64, c_int64, c_int64]),
    "da_decode_attention": (
        c_int,
        [c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int64, c_int64,
         c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_int64, c_float, c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "da_decode_attention_static_capacity": (c_size_t, []),
    "da_decode_attention_static": (
        c_int,
        [c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int64, c_int64,
         c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_int64, c_float, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "da_decode_attention_paged": (
        c_int,
        [c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int64, c_int64,
         c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_int64, c_float, c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p,
         c_void_p],
    ),
    "da_pages_gather_attend": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p,
         c_void_p, c_int, c_int, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_float, c_int64,
         c_int64, c_void_p, c_size_t, c_void_p],
    ),
}


class PagedOverlap(ctypes.Structure):
    """struct da_paged_overlap of the header."""

    _fields_ = [
        ("page_size", ctypes.c_int32),
        ("phase", ctypes.c_int32),
        ("slot_epoch", c_void_p),
        ("slot_epoch_head_stride", c_int64),
        ("epoch", c_void_p),
        ("miss_slot", c_void_p),
        ("miss_count", c_void_p),
        ("miss_capacity", ctypes.c_int32),
        ("gather_blocks", ctypes.c_int32),
        ("dram", c_void_p),
        ("dram_head_stride_bytes", c_int64),
        ("dram_page_stride_bytes", c_int64),
        ("hbm", c_void_p),
        ("hbm_head_stride_bytes", c_int64),
        ("hbm_slot_stride_bytes", c_int64),
        ("miss_page", c_void_p),
        ("link_gbps", c_float),
        ("block_gbps", c_float),
    ]

_lib = None


def load() -> ctypes.CDLL:
    """Load libdramattn.so and bind every symbol; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m dram_attention_amd.build` "
            "(there is no fallback path)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().da_last_error_string().decode(errors="replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"unsupported element type {dtype}") from None


def itype_code(dtype: torch.dtype) -> int:
    try:
        return _ITYPES[dtype]
    except KeyError:
        raise TypeError(f"index tensors must be int32 or int64, got {dtype}") from None


def time_code(dtype: torch.dtype) -> int:
    try:
        return _TIME_TYPES[dtype]
    except KeyError:
        raise TypeError(f"page_access_time must be float32 or int32, got {dtype}") from None


def stream_ptr(device: torch.device) -> int:
    """The raw hipStream_t of torch's current stream on `device`."""
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} must live on a GPU: the HIP kernels are the only implementation "
            f"(got device {t.device})"
        )


def device_visible_ptr(t: torch.Tensor) -> int:
    """Address a kernel can dereference: data_ptr() for GPU tensors, the mapped
    device address for pinned host tensors."""
    if t.is_cuda:
        return t.data_ptr()
    if not t.is_pinned():
        raise RuntimeError("host tensors handed to the kernels must be pinned")
    out = c_void_p()
    check(load().da_host_device_pointer(t.data_ptr(), ctypes.byref(out)), "da_host_device_pointer")
    return out.value
