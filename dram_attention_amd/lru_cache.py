"""HBM page cache in front of a pinned-host KV page store, LRU replacement.

Mirrors dram_attention/lru_cache.py of the reference (CacheOutput :19,
DummyCache :24-37, LRUCache :40-265): same constructor, attributes, buffers and
``load_`` / ``get_kv_cache_`` behaviour; the work runs in HIP kernels.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import _lib
from .lru_kernel import (LruScratch, lru_update, lru_update_and_gather, pages_gather,
                         pages_gather_attend)
from .topk_selector import IPUpperboundTopKSelector


class CacheOutput(NamedTuple):
    k_cache: torch.Tensor
    v_cache: torch.Tensor


class DummyCache(torch.nn.Module):
    """A static KV cache that simply lives in HBM (prefix small enough to fit)."""

    def __init__(self, k_cache: torch.Tensor, v_cache: torch.Tensor, device: str, *args,
                 **kvargs):
        super().__init__()
        self.k_cache = k_cache.to(device=device, non_blocking=True)
        self.v_cache = v_cache.to(device=device, non_blocking=True)

    def get_kv_cache_(self, q: torch.Tensor) -> CacheOutput:
        return CacheOutput(k_cache=self.k_cache, v_cache=self.v_cache)


class LRUCache(torch.nn.Module):
    """Per-layer paged KV store: every page in pinned host DRAM, the most
    recently used ``num_hbm_pages`` of them in HBM slots.

    Buffers (names and shapes as in the reference):
        current_step                    (1,) int32
        dram_kv_cache                   (H, num_dram_pages, page_size*2*head_dim), pinned host;
                                        token t of a page: K at t*2*D, V at t*2*D + D
        hbm_kv_cache                    (H, num_hbm_pages, page_size*2*head_dim)
        page_access_time                (H, num_hbm_pages) float32
        dram_page_to_hbm_page_mapping   (H, num_dram_pages) int64, -1 = not resident
        hbm_page_to_dram_page_mapping   (H, num_hbm_pages) int64
    """

    def __init__(
        self,
        k_cache: torch.Tensor,
        v_cache: torch.Tensor,
        page_size: int,
        top_k: int,
        lru_hbm_cache_size: Optional[int] = None,
        hbm_kv_cache_fraction: float = 0.2,
        device: str = "cuda",
    ):
        super().__init__()
        assert k_cache.shape == v_cache.shape, "Key and value cache shapes must match."
        num_kv_heads, dram_kv_cache_size, head_dim = k_cache.shape
        dtype = k_cache.dtype
        assert dram_kv_cache_size % page_size == 0, "KV cache size must be divisible by page size."
        num_dram_pages = dram_kv_cache_size // page_size
        if lru_hbm_cache_size is None:
            num_hbm_pages = int(num_dram_pages * hbm_kv_cache_fraction)
        else:
            num_hbm_pages = lru_hbm_cache_size // page_size

        self.page_size = page_size
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.num_dram_pages = num_dram_pages
        self.num_hbm_pages = num_hbm_pages
        self.top_k = top_k

        self.top_k_selector = IPUpperboundTopKSelector(k_cache, num_dram_pages, device=device)
        self.register_buffer("current_step", torch.zeros(1, dtype=torch.int32, device=device))

        page_dim = page_size * 2 * head_dim
        dram = torch.empty((num_kv_heads, num_dram_pages, page_dim), dtype=dtype, device="cpu",
                           pin_memory=True)
        self.register_buffer("dram_kv_cache", dram)
        self.register_buffer(
            "hbm_kv_cache",
            torch.empty(num_kv_heads, num_hbm_pages, page_dim, dtype=dtype, device=device))
        self.register_buffer(
            "page_access_time",
            torch.zeros(num_kv_heads, num_hbm_pages, dtype=torch.float32, device=device))
        self.register_buffer(
            "dram_page_to_hbm_page_mapping",
            torch.full((num_kv_heads, num_dram_pages), -1, dtype=torch.int64, device=device))
        self.register_buffer(
            "hbm_page_to_dram_page_mapping",
            torch.full((num_kv_heads, num_hbm_pages), -1, dtype=torch.int64, device=device))
        assert num_hbm_pages <= num_dram_pages, "HBM cache size must be smaller than DRAM cache size."

        # Start with the most recent pages resident: slot s holds page P - N + s.
        first = num_dram_pages - num_hbm_pages
        row_bytes = head_dim * k_cache.element_size()
        if (k_cache.is_cuda and v_cache.is_cuda and row_bytes % 16 == 0 and num_dram_pages > 0
                and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
                and k_cache.stride() == v_cache.stride()
                and all(st * k_cache.element_size() % 16 == 0 for st in k_cache.stride()[:2])
                and k_cache.data_ptr() % 16 == 0 and v_cache.data_ptr() % 16 == 0):
            # one kernel packs every page into the pinned store and the resident ones into slots
            esz = k_cache.element_size()
            self._dram_device_ptr = _lib.device_visible_ptr(dram)
            _lib.check(
                _lib.load().da_pages_build(
                    k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(1), k_cache.stride(0),
                    num_kv_heads, num_dram_pages, page_size, head_dim, _lib.dtype_code(dtype),
                    self._dram_device_ptr, dram.stride(0) * esz, dram.stride(1) * esz,
                    self.hbm_kv_cache.data_ptr(), self.hbm_kv_cache.stride(0) * esz,
                    self.hbm_kv_cache.stride(1) * esz, first, num_hbm_pages,
                    _lib.stream_ptr(self.hbm_kv_cache.device)),
                "da_pages_build")
            torch.cuda.current_stream(self.hbm_kv_cache.device).synchronize()  # host store complete
        else:
            # host-resident or oddly shaped inputs: torch copies, then the slots from the store
            self._dram_device_ptr = None
            paged = dram.view(num_kv_heads, num_dram_pages, page_size, 2, head_dim)
            paged[..., 0, :].copy_(
                k_cache.reshape(num_kv_heads, num_dram_pages, page_size, head_dim), non_blocking=True)
            paged[..., 1, :].copy_(
                v_cache.reshape(num_kv_heads, num_dram_pages, page_size, head_dim), non_blocking=True)
            if k_cache.is_cuda or v_cache.is_cuda:
                torch.cuda.current_stream(self.hbm_kv_cache.device).synchronize()  # D2H copies
            self.hbm_kv_cache.copy_(dram[:, first:], non_blocking=True)
        slots = torch.arange(num_hbm_pages, dtype=torch.int64, device=device)
        self.dram_page_to_hbm_page_mapping[:, first:] = slots
        self.hbm_page_to_dram_page_mapping[:] = slots + first

        self._scratch = None
        self._topk_idx = None

    # -- internals ---------------------------------------------------------
    def _scratch_for(self, k: int) -> LruScratch:
        if self._scratch is None or self._scratch.miss_page.shape[1] != max(k, 1):
            self._scratch = LruScratch.allocate(self.num_kv_heads, k, self.hbm_kv_cache.device,
                                                self.num_hbm_pages)
        return self._scratch

    def _views(self) -> CacheOutput:
        paged = self.hbm_kv_cache.view(
            self.num_kv_heads, self.num_hbm_pages * self.page_size, 2, self.head_dim)
        k_cache, v_cache = paged.unbind(dim=2)
        return CacheOutput(k_cache=k_cache, v_cache=v_cache)

    # -- reference surface -------------------------------------------------
    def load_(self, top_k_dram_page_index: torch.Tensor) -> CacheOutput:
        """Make the listed DRAM pages (H, k) resident, evicting least recently used
        slots, and return K/V views over ALL slots, each (H, num_hbm_pages*page_size, D).
        Advances ``current_step`` by one (inside the kernel, no host sync)."""
        if self._dram_device_ptr is None:
            self._dram_device_ptr = _lib.device_visible_ptr(self.dram_kv_cache)
        scratch = self._scratch_for(top_k_dram_page_index.shape[1])
        lru_update_and_gather(
            self.dram_kv_cache, self.page_access_time, self.dram_page_to_hbm_page_mapping,
            self.hbm_page_to_dram_page_mapping, top_k_dram_page_index, self.current_step,
            self.hbm_kv_cache, scratch, bump_step=True, dram_device_ptr=self._dram_device_ptr,
            use_candidates=True,   # the kernel ignores a list whose stamp is not this step
        )
        return self._views()

    def get_kv_cache_(self, q: torch.Tensor) -> CacheOutput:
        """Score all pages against ``q`` (1, seq_len, Hq, D), select the top ones per
        query head, page them in, and return the HBM-resident K/V views."""
        bsz, seq_len, num_q_heads, _ = q.shape
        assert num_q_heads % self.num_kv_heads == 0
        rep = num_q_heads // self.num_kv_heads
        return self.load_(self.select_(q))

    # -- the same step in separable pieces (used by DRAMAttention to overlap the
    #    page stream with attention over the slots that keep their page) -------
    def select_(self, q: torch.Tensor) -> torch.Tensor:
        """Scores + ordered top-k: the (H, seq_len*rep*k) request list of this step."""
        bsz, seq_len, num_q_heads, _ = q.shape
        assert num_q_heads % self.num_kv_heads == 0
        rep = num_q_heads // self.num_kv_heads
        k = min(self.top_k, self.num_dram_pages)
        total = seq_len * rep * k
        if self._topk_idx is None or self._topk_idx.shape[1] != total:
            self._topk_idx = torch.empty(self.num_kv_heads, total, dtype=torch.int64,
                                         device=q.device)
        # the same launch lists the least recently used slots for update_ (the
        # order of the slots does not depend on the scores)
        scratch = self._scratch_for(total)
        return self.top_k_selector.top_k_for_lru(
            q, k, out=self._topk_idx, lru=(self.page_access_time, scratch.candidates, self.current_step))

    def update_(self, idx: torch.Tensor) -> LruScratch:
        """Metadata only: advance the step, touch/evict/assign, emit the miss list."""
        scratch = self._scratch_for(idx.shape[1])
        # the list select_ left carries the step it was made at: the kernel uses it only
        # if nothing has updated the cache since
        lru_update(self.dram_kv_cache, self.page_access_time, self.dram_page_to_hbm_page_mapping,
                   self.hbm_page_to_dram_page_mapping, idx, self.current_step, self.hbm_kv_cache,
                   scratch, bump_step=True, use_candidates=True)
        return scratch

    def gather_(self, k: int) -> None:
        """Stream the pages of the last miss list into their slots (current stream)."""
        if self._dram_device_ptr is None:
            self._dram_device_ptr = _lib.device_visible_ptr(self.dram_kv_cache)
        pages_gather(self.dram_kv_cache, self.hbm_kv_cache, self._scratch, k,
                     self._dram_device_ptr)

    def gather_attend_(self, k: int, xq: torch.Tensor, scale: float, c_capacity: int,
                       workspace: torch.Tensor, blocks_per_head: int) -> None:
        """gather_ with the step's attention over the streamed pages computed on the way."""
        if self._dram_device_ptr is None:
            self._dram_device_ptr = _lib.device_visible_ptr(self.dram_kv_cache)
        pages_gather_attend(self.dram_kv_cache, self.hbm_kv_cache, self._scratch, k,
                            self.page_size, xq, scale, self.num_hbm_pages * self.page_size,
                            c_capacity, workspace, blocks_per_head, self._dram_device_ptr)

    def page_stores(self):
        """(dram_kv_cache, its device-visible address, hbm_kv_cache) for a page stream
        that runs inside an attention launch."""
        if self._dram_device_ptr is None:
            self._dram_device_ptr = _lib.device_visible_ptr(self.dram_kv_cache)
        return self.dram_kv_cache, self._dram_device_ptr, self.hbm_kv_cache

    def views(self) -> CacheOutput:
        return self._views()

    # -- instrumentation (absent from the reference) -------------------------
    def last_miss_counts(self) -> torch.Tensor:
        """Distinct pages paged in by the last load_ per kv head (device int32)."""
        if self._scratch is None:
            return torch.zeros(self.num_kv_heads, dtype=torch.int32,
                               device=self.hbm_kv_cache.device)
        return self._scratch.miss_count
