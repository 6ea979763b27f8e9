"""LRU lookup / evict / slot-assign and page streaming on HIP kernels.

Mirrors dram_attention/lru_triton_kernel.py of the reference:
``load_lru_cache_`` (:140-194) keeps its signature and in-place semantics.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import _lib


class LruScratch(NamedTuple):
    """Per-cache device buffers the two kernels exchange (allocated once)."""

    miss_page: torch.Tensor   # (H, K) int32: i-th distinct missed page of a head
    miss_slot: torch.Tensor   # (H, K) int32: the slot it was given
    miss_count: torch.Tensor  # (H,) int32
    hit_mask: torch.Tensor    # (H, K) uint8: 1 = resident when visited
    workspace: torch.Tensor   # zeroed once; holds the step-bump ticket
    slot_epoch: torch.Tensor  # (H, N_hbm) int32: step at which a slot was last re-assigned
    # (H, k_cand) int32: least recent slots, when a selector fills it; a view made by
    # candidate_list(), whose buffer carries one stamp word per head behind the lists
    candidates: torch.Tensor = None

    @staticmethod
    def allocate(num_heads: int, k: int, device, num_hbm_pages: int = 0) -> "LruScratch":
        lib = _lib.load()
        ws = lib.da_lru_update_workspace_bytes(num_heads, k, 0, 0)
        return LruScratch(
            slot_epoch=torch.zeros(num_heads, max(num_hbm_pages, 1), dtype=torch.int32,
                                   device=device),
            miss_page=torch.empty(num_heads, max(k, 1), dtype=torch.int32, device=device),
            miss_slot=torch.empty(num_heads, max(k, 1), dtype=torch.int32, device=device),
            miss_count=torch.zeros(num_heads, dtype=torch.int32, device=device),
            hit_mask=torch.empty(num_heads, max(k, 1), dtype=torch.uint8, device=device),
            workspace=torch.zeros(ws, dtype=torch.uint8, device=device),
            candidates=candidate_list(num_heads, max(lru_candidate_count(k, num_hbm_pages), 1),
                                      device),
        )


def candidate_list(num_heads: int, k_cand: int, device) -> torch.Tensor:
    """Room for the lists of least recently used slots as da_topk_pages_lru writes them:
    an (H, k_cand) int32 view of a buffer that holds one stamp word per head behind the
    lists (the step counter's value when a list was made; da_lru_update ignores a list
    whose stamp is not the step it reads).  Starts out with stamps no counter has."""
    buf = torch.full((num_heads * k_cand + num_heads,), -1, dtype=torch.int32, device=device)
    return buf[: num_heads * k_cand].view(num_heads, k_cand)


def check_candidate_list(candidates: torch.Tensor) -> None:
    H, k_cand = candidates.shape
    room = candidates.untyped_storage().nbytes() // 4 - candidates.storage_offset()
    if (candidates.dtype != torch.int32 or not candidates.is_contiguous()
            or room < H * k_cand + H):
        raise ValueError("the candidate list must come from candidate_list(): contiguous int32 "
                         "lists with one stamp word per head behind them")


MIN_LRU_CANDIDATES = 256   # one sort block's fast path
MAX_LRU_CANDIDATES = 8192  # what one workgroup orders in LDS


def lru_candidate_count(k: int, num_hbm_pages: int) -> int:
    """Least recent slots to list ahead of an update with ``k`` requests per head.  Up
    to 1024 requests: what the sort's short path handles, so that the list does not
    lengthen the top-k launch; it covers the misses of a typical step there (an eighth
    of the requests at the 128K workload), and a step that misses more falls back to
    ordering all slots inside the update.  Beyond that (the 1M workload: as many
    requests as slots, two thirds of the slots touched and a third replaced in every
    step) only the complete order is sure to hold enough untouched slots, and the
    longer top-k launch hides its cost."""
    want = MIN_LRU_CANDIDATES if k <= 1024 else num_hbm_pages
    return min(num_hbm_pages, MAX_LRU_CANDIDATES, want)


def lru_update(
    dram_kv_cache: torch.Tensor,
    page_access_time: torch.Tensor,
    dram_page_to_hbm_page_mapping: torch.Tensor,
    hbm_page_to_dram_page_mapping: torch.Tensor,
    topk_dram_page_index: torch.Tensor,
    current_step: torch.Tensor,
    hbm_kv_cache: torch.Tensor,
    scratch: LruScratch,
    bump_step: bool,
    serial_walk: bool = False,
    use_candidates: bool = False,
) -> None:
    """The metadata half of a step: touch, evict, assign; leaves the miss list in
    ``scratch`` (one launch on the current stream).  ``serial_walk`` forces the
    literal one-request-at-a-time walk (same result, for checks and baselines).
    ``use_candidates``: ``scratch.candidates`` holds the least recently used slots
    in eviction order (filled by ``topk_pages(..., lru=...)``); the kernel uses the
    list only if its stamp is the step it reads, i.e. if no update came in between."""
    num_heads, num_dram_pages, page_dim = dram_kv_cache.shape
    _, k = topk_dram_page_index.shape
    assert (
        dram_kv_cache.shape[0] == hbm_kv_cache.shape[0]
        and dram_kv_cache.shape[2] == hbm_kv_cache.shape[2]
    )
    num_hbm_pages = hbm_kv_cache.shape[1]
    if scratch.miss_page.shape != (num_heads, max(k, 1)):
        raise ValueError("scratch was allocated for another (heads, k)")
    for name, t in (("page_access_time", page_access_time),
                    ("dram_page_to_hbm_page_mapping", dram_page_to_hbm_page_mapping),
                    ("hbm_page_to_dram_page_mapping", hbm_page_to_dram_page_mapping),
                    ("topk_dram_page_index", topk_dram_page_index),
                    ("current_step", current_step), ("hbm_kv_cache", hbm_kv_cache)):
        _lib.require_gpu(t, name)
        if t.dim() > 1 and t.shape[-1] > 1 and t.stride(-1) != 1:
            raise ValueError(f"{name} must be dense along its last axis")
    # the kernel indexes these by slot and by page: their extents must be the stores'
    for name, t, want in (("page_access_time", page_access_time, (num_heads, num_hbm_pages)),
                          ("hbm_page_to_dram_page_mapping", hbm_page_to_dram_page_mapping,
                           (num_heads, num_hbm_pages)),
                          ("dram_page_to_hbm_page_mapping", dram_page_to_hbm_page_mapping,
                           (num_heads, num_dram_pages))):
        if tuple(t.shape) != want:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, the page stores need {want}")
    if topk_dram_page_index.shape[0] != num_heads:
        raise ValueError("topk_dram_page_index must have one row per head")
    if dram_page_to_hbm_page_mapping.dtype != hbm_page_to_dram_page_mapping.dtype:
        raise TypeError("the two page mappings must share one integer type")
    if current_step.dtype != torch.int32:
        raise TypeError("current_step must be int32")
    if dram_kv_cache.dtype != hbm_kv_cache.dtype:
        raise TypeError("DRAM and HBM page stores must share one element type")
    if dram_kv_cache.stride(2) != 1 or hbm_kv_cache.stride(2) != 1:
        raise ValueError("pages must be dense")
    epoch = scratch.slot_epoch if scratch.slot_epoch.shape == (num_heads, num_hbm_pages) else None
    if use_candidates:
        check_candidate_list(scratch.candidates)
    lib = _lib.load()
    _lib.check(
        lib.da_lru_update(
            topk_dram_page_index.data_ptr(), topk_dram_page_index.stride(0),
            _lib.itype_code(topk_dram_page_index.dtype), num_heads, k, num_dram_pages,
            num_hbm_pages, current_step.data_ptr(), int(bump_step) | (2 if serial_walk else 0),
            page_access_time.data_ptr(), page_access_time.stride(0),
            _lib.time_code(page_access_time.dtype),
            dram_page_to_hbm_page_mapping.data_ptr(), dram_page_to_hbm_page_mapping.stride(0),
            hbm_page_to_dram_page_mapping.data_ptr(), hbm_page_to_dram_page_mapping.stride(0),
            _lib.itype_code(dram_page_to_hbm_page_mapping.dtype),
            scratch.hit_mask.data_ptr(), scratch.miss_page.data_ptr(),
            scratch.miss_slot.data_ptr(), scratch.miss_count.data_ptr(),
            epoch.data_ptr() if epoch is not None else None,
            scratch.candidates.data_ptr() if use_candidates else None,
            scratch.candidates.shape[1] if use_candidates else 0,
            scratch.workspace.data_ptr(), scratch.workspace.numel(),
            _lib.stream_ptr(hbm_kv_cache.device),
        ),
        "da_lru_update",
    )


def lru_candidates(page_access_time: torch.Tensor, scratch: LruScratch,
                   current_step: torch.Tensor) -> torch.Tensor:
    """Fill ``scratch.candidates`` with the least recently used slots of every head, in
    eviction order, as of now, stamped with ``current_step`` (one launch; normally this
    rides along with the top-k)."""
    H, N = page_access_time.shape
    cand = scratch.candidates
    _lib.require_gpu(page_access_time, "page_access_time")
    _lib.require_gpu(current_step, "current_step")
    check_candidate_list(cand)
    _lib.check(
        _lib.load().da_topk_pages_lru(
            None, 0, 0, 0, 1, H, 0, 0, None, 0, 0, 0, _lib.itype_code(torch.int64),
            page_access_time.data_ptr(), page_access_time.stride(0),
            _lib.time_code(page_access_time.dtype), N, cand.shape[1], cand.data_ptr(),
            current_step.data_ptr(), None, 0, _lib.stream_ptr(page_access_time.device)),
        "da_topk_pages_lru")
    return cand


def pages_gather(dram_kv_cache: torch.Tensor, hbm_kv_cache: torch.Tensor, scratch: LruScratch,
                 k: int, dram_device_ptr: Optional[int] = None, max_blocks: int = 0) -> None:
    """The data half: copy every page of the miss list into its slot (one launch
    on the current stream; the page store may be pinned host memory)."""
    num_heads, _, page_dim = dram_kv_cache.shape
    if dram_device_ptr is None:
        dram_device_ptr = _lib.device_visible_ptr(dram_kv_cache)
    esz = dram_kv_cache.element_size()
    lib = _lib.load()
    _lib.check(
        lib.da_pages_gather(
            dram_device_ptr, dram_kv_cache.stride(0) * esz, dram_kv_cache.stride(1) * esz,
            hbm_kv_cache.data_ptr(), hbm_kv_cache.stride(0) * esz, hbm_kv_cache.stride(1) * esz,
            page_dim * esz, scratch.miss_page.data_ptr(), scratch.miss_slot.data_ptr(),
            scratch.miss_count.data_ptr(), num_heads, k, max_blocks,
            _lib.stream_ptr(hbm_kv_cache.device),
        ),
        "da_pages_gather",
    )


GATHER_BLOCKS = 32  # workgroups of a page stream in all: few and fat saturate the host link

_link_gbps = {}


def host_link_gbps(device) -> float:
    """Pinned host -> HBM copy rate of this box in GB/s, measured once per device and
    process (three 16 MiB copies between two events, under a millisecond).  Only the
    scheduling of the stream + attention launch reads it, never a result."""
    device = torch.device(device)
    key = device.index if device.index is not None else torch.cuda.current_device()
    if key not in _link_gbps:
        n = 16 << 20
        src = torch.empty(n, dtype=torch.uint8, pin_memory=True)
        dst = torch.empty(n, dtype=torch.uint8, device=device)
        dst.copy_(src, non_blocking=True)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            dst.copy_(src, non_blocking=True)
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1)
        _link_gbps[key] = 3 * n / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
    return _link_gbps[key]


def gather_attend_supported(n_q_heads: int, n_kv_heads: int, head_dim: int, page_size: int,
                            dtype: torch.dtype) -> bool:
    """Whether pages_gather_attend takes this shape (else: pages_gather + tail pass)."""
    row = head_dim * torch.empty(0, dtype=dtype).element_size()
    return (row in (64, 128, 256, 512) and n_q_heads // n_kv_heads <= 8
            and page_size * 2 * row <= 16384 and n_kv_heads <= 64)


def pages_gather_attend(dram_kv_cache: torch.Tensor, hbm_kv_cache: torch.Tensor,
                        scratch: LruScratch, k: int, page_size: int, xq: torch.Tensor,
                        scale: float, p_len: int, c_capacity: int, workspace: torch.Tensor,
                        blocks_per_head: int, dram_device_ptr: Optional[int] = None) -> None:
    """pages_gather, with the attention of query ``xq`` (Hq, D) over every copied
    page computed on the way; the partial results land in ``workspace`` (the one
    the step's decode_attention calls use) for the final merge."""
    num_heads = dram_kv_cache.shape[0]
    Hq, D = xq.shape
    if dram_device_ptr is None:
        dram_device_ptr = _lib.device_visible_ptr(dram_kv_cache)
    esz = dram_kv_cache.element_size()
    if dram_kv_cache.shape[2] != page_size * 2 * D or xq.dtype != hbm_kv_cache.dtype:
        raise ValueError("pages must hold page_size tokens of (K row, V row) in the query's dtype")
    lib = _lib.load()
    _lib.check(
        lib.da_pages_gather_attend(
            dram_device_ptr, dram_kv_cache.stride(0) * esz, dram_kv_cache.stride(1) * esz,
            hbm_kv_cache.data_ptr(), hbm_kv_cache.stride(0) * esz, hbm_kv_cache.stride(1) * esz,
            page_size, scratch.miss_page.data_ptr(), scratch.miss_slot.data_ptr(),
            scratch.miss_count.data_ptr(), num_heads, k, blocks_per_head,
            xq.data_ptr(), xq.stride(0), Hq, D, _lib.dtype_code(xq.dtype), scale, p_len,
            c_capacity, workspace.data_ptr(), workspace.numel() * workspace.element_size(),
            _lib.stream_ptr(hbm_kv_cache.device),
        ),
        "da_pages_gather_attend",
    )


def lru_update_and_gather(
    dram_kv_cache: torch.Tensor,
    page_access_time: torch.Tensor,
    dram_page_to_hbm_page_mapping: torch.Tensor,
    hbm_page_to_dram_page_mapping: torch.Tensor,
    topk_dram_page_index: torch.Tensor,
    current_step: torch.Tensor,
    hbm_kv_cache: torch.Tensor,
    scratch: LruScratch,
    bump_step: bool,
    dram_device_ptr: Optional[int] = None,
    serial_walk: bool = False,
    use_candidates: bool = False,
) -> None:
    """Two launches on the current stream: metadata update, then page gather."""
    lru_update(dram_kv_cache, page_access_time, dram_page_to_hbm_page_mapping,
               hbm_page_to_dram_page_mapping, topk_dram_page_index, current_step, hbm_kv_cache,
               scratch, bump_step, serial_walk, use_candidates)
    pages_gather(dram_kv_cache, hbm_kv_cache, scratch, topk_dram_page_index.shape[1],
                 dram_device_ptr)


def load_lru_cache_(
    dram_kv_cache: torch.Tensor,
    page_access_time: torch.Tensor,
    dram_page_to_hbm_page_mapping: torch.Tensor,
    hbm_page_to_dram_page_mapping: torch.Tensor,
    topk_dram_page_index: torch.Tensor,
    *,
    current_step: torch.Tensor,
    hbm_kv_cache: torch.Tensor,
):
    """Touch / evict / assign / copy for one step, in place, as the reference's
    function of the same name; metadata may be int32 or int64, access times
    float32 or int32, the page store a GPU tensor or pinned host memory."""
    num_heads = dram_kv_cache.shape[0]
    k = topk_dram_page_index.shape[1]
    scratch = LruScratch.allocate(num_heads, k, hbm_kv_cache.device)
    lru_update_and_gather(
        dram_kv_cache, page_access_time, dram_page_to_hbm_page_mapping,
        hbm_page_to_dram_page_mapping, topk_dram_page_index, current_step, hbm_kv_cache,
        scratch, bump_step=False,
    )
