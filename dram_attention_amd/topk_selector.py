"""Quest page selector on HIP kernels (page summaries, scores, ordered top-k).

Mirrors dram_attention/topk_selector.py of the reference
(IPUpperboundTopKSelector: __init__ :16-35, top_k :37-61).
"""

from __future__ import annotations

import torch

from . import _lib
from .max_ip_kernel import page_scores


def page_min_max(k_cache: torch.Tensor, num_pages: int) -> torch.Tensor:
    """(H, S, D) keys -> (H, num_pages, 2, D) per-page channel min ([..,0,:]) and max."""
    num_heads, length, head_dim = k_cache.shape
    assert length % num_pages == 0, "Cache size must be divisible by num_pages."
    _lib.require_gpu(k_cache, "k_cache")
    if k_cache.stride(-1) != 1:
        k_cache = k_cache.contiguous()
    page = length // num_pages
    out = torch.empty(num_heads, num_pages, 2, head_dim, dtype=k_cache.dtype,
                      device=k_cache.device)
    lib = _lib.load()
    _lib.check(
        lib.da_page_minmax(
            k_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1), num_heads, num_pages,
            page, head_dim, _lib.dtype_code(k_cache.dtype), out.data_ptr(),
            _lib.stream_ptr(k_cache.device),
        ),
        "da_page_minmax",
    )
    return out


_split_workspaces = {}


def _split_workspace(n_rows: int, n_heads: int, n_pages: int, k: int, device) -> torch.Tensor | None:
    """Candidate buffer of the two-launch selection of long rows (None: not needed).
    One buffer per shape and device, kept between calls: launches of one stream
    follow each other, and the buffer carries nothing from call to call."""
    need = _lib.load().da_topk_pages_workspace_bytes(n_rows, n_heads, n_pages, k)
    if need == 0:
        return None
    key = (n_rows, n_heads, n_pages, k, str(device), torch.cuda.current_stream(device).cuda_stream)
    ws = _split_workspaces.get(key)
    if ws is None:
        ws = _split_workspaces[key] = torch.empty(need, dtype=torch.uint8, device=device)
    return ws


def topk_pages(scores: torch.Tensor, rep: int, k: int, out: torch.Tensor,
               seq_stride: int, head_stride: int, rep_stride: int, lru=None,
               workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Ordered top-k of every row of fp32 ``scores`` (n_rows, H, L); row n of head h
    lands at (n // rep)*seq_stride + h*head_stride + (n % rep)*rep_stride in ``out``.
    ``lru`` = (page_access_time (H, N), candidates (H, k_cand) int32 from
    lru_kernel.candidate_list, current_step): the same launch also lists the k_cand
    least recently used slots of every head, stamped with the step counter's value,
    for the LRU update that follows.  ``workspace``: candidate buffer for rows longer than
    16384 pages (da_topk_pages_workspace_bytes); by default one per shape and stream
    is kept by this module."""
    n_rows, H, L = scores.shape
    assert scores.dtype == torch.float32 and (L <= 1 or scores.stride(-1) == 1)
    lib = _lib.load()
    if workspace is None and n_rows > 0 and k > 0 and L > 16384:
        workspace = _split_workspace(n_rows, H, L, k, scores.device)
    if lru is None:
        time_ptr, time_hs, time_code, n_slots, k_cand, cand_ptr, step_ptr = None, 0, 0, 0, 0, None, None
    else:
        from .lru_kernel import check_candidate_list

        access_time, candidates, current_step = lru
        assert access_time.shape[0] == H and candidates.shape[0] == H
        assert current_step.dtype == torch.int32
        check_candidate_list(candidates)
        step_ptr = current_step.data_ptr()
        time_ptr, time_hs = access_time.data_ptr(), access_time.stride(0)
        time_code, n_slots = _lib.time_code(access_time.dtype), access_time.shape[1]
        k_cand, cand_ptr = candidates.shape[1], candidates.data_ptr()
    _lib.check(
        lib.da_topk_pages_lru(
            scores.data_ptr(), scores.stride(0), scores.stride(1), n_rows, rep, H, L, k,
            out.data_ptr(), seq_stride, head_stride, rep_stride, _lib.itype_code(out.dtype),
            time_ptr, time_hs, time_code, n_slots, k_cand, cand_ptr, step_ptr,
            None if workspace is None else workspace.data_ptr(),
            0 if workspace is None else workspace.numel() * workspace.element_size(),
            _lib.stream_ptr(scores.device),
        ),
        "da_topk_pages",
    )
    return out


class IPUpperboundTopKSelector:
    """Inner-product upper-bound top-k page selector (Quest).

    Ranking contract: pages are ordered by descending score and, among equal
    scores, by ascending page index (the reference's argsort leaves ties open).
    Scores of 16-bit inputs are rounded to the input type before ranking, as the
    reference's kernel output is.
    """

    def __init__(self, k_cache: torch.Tensor, num_pages: int, device="cuda"):
        num_heads, dram_kv_cache_size, head_dim = k_cache.shape
        self.num_kv_heads = num_heads
        assert dram_kv_cache_size % num_pages == 0, "Cache size must be divisible by num_pages."
        self.device = torch.device(device)
        # the summaries are built on the GPU: host-resident keys are moved first
        self.chunk_min_max = page_min_max(k_cache.to(device=device), num_pages)
        # chunk_min_max comes from page_min_max, so min <= max in every channel and the
        # scorer may pick the bound by the sign of q; clear this after writing other
        # contents into chunk_min_max
        self.bounds_are_ordered = True
        self._scores = None
        self._split_ws = None   # candidate buffer of long rows: this selector's own, the largest so far

    def scores(self, q: torch.Tensor) -> torch.Tensor:
        """fp32 scores (seq_len*rep, num_kv_heads, num_pages); row s*rep + r is query
        head h*rep + r of token s."""
        bsz, seq_len, num_q_heads, head_dim = q.shape
        assert bsz == 1, f"Only batch size 1 is supported, but got batch size {bsz}"
        assert num_q_heads % self.num_kv_heads == 0
        rep = num_q_heads // self.num_kv_heads
        H, L = self.num_kv_heads, self.chunk_min_max.shape[1]
        if q.stride(-1) != 1:
            q = q.contiguous()
        n_rows = seq_len * rep
        if self._scores is None or self._scores.shape[0] != n_rows:
            self._scores = torch.empty(n_rows, H, L, dtype=torch.float32, device=q.device)
        if seq_len == 1:
            # (rep, H, D) view of the single token's heads: strides (D, rep*D, 1)
            qv = q[0, 0].view(H, rep, head_dim).transpose(0, 1)
        else:
            qv = q[0].view(seq_len, H, rep, head_dim).transpose(1, 2).reshape(n_rows, H, head_dim)
        return page_scores(qv, self.chunk_min_max, self._scores, round_to_input=True,
                           ordered_bounds=self.bounds_are_ordered)

    def _workspace(self, scores: torch.Tensor, k: int):
        """Candidate buffer of the two-launch selection of rows beyond 16384 pages (None
        when the shape needs none).  One buffer per selector, grown to the largest
        shape seen and shared by the smaller ones; it carries nothing from call to call,
        so the calls of one selector must follow each other on ONE stream (two streams
        stepping the same selector would race on it)."""
        n_rows, H, L = scores.shape
        need = _lib.load().da_topk_pages_workspace_bytes(n_rows, H, L, k)
        if need == 0:
            return None
        if self._split_ws is None or self._split_ws.numel() < need:
            self._split_ws = torch.empty(need, dtype=torch.uint8, device=scores.device)
        return self._split_ws

    def top_k(self, q: torch.Tensor, k: int) -> torch.Tensor:
        """Indices of the top k pages, (seq_len, num_kv_heads, rep, k) int64, best first."""
        bsz, seq_len, num_q_heads, _ = q.shape
        scores = self.scores(q)
        rep = num_q_heads // self.num_kv_heads
        H, L = self.num_kv_heads, scores.shape[-1]
        k = min(k, L)
        out = torch.empty(seq_len, H, rep, k, dtype=torch.int64, device=q.device)
        return topk_pages(scores, rep, k, out, H * rep * k, rep * k, k,
                          workspace=self._workspace(scores, k))

    def top_k_for_lru(self, q: torch.Tensor, k: int, out: torch.Tensor | None = None, lru=None):
        """The same selection laid out as the LRU consumes it, (num_kv_heads,
        seq_len*rep*k): what swapaxes(0,1).contiguous().view(H,-1) of top_k gives.
        ``lru``: see :func:`topk_pages`."""
        bsz, seq_len, num_q_heads, _ = q.shape
        scores = self.scores(q)
        rep = num_q_heads // self.num_kv_heads
        H, L = self.num_kv_heads, scores.shape[-1]
        k = min(k, L)
        if out is None:
            out = torch.empty(H, seq_len * rep * k, dtype=torch.int64, device=q.device)
        return topk_pages(scores, rep, k, out, rep * k, seq_len * rep * k, k, lru=lru,
                          workspace=self._workspace(scores, k))


class TokenMaxTopKSelector(IPUpperboundTopKSelector):
    """Ranks pages by their best token: score = max over the page's tokens of q.k, the
    quantity the min/max bound estimates from above.  The selector of the reference's
    accuracy ceiling for page selection (evaluation/quest-top-k-oracle/model.py:267-275);
    a comparison variant, not the hot path: it keeps every prefix key on the device and
    scores with torch ops in the input type, as that model does.  Ranking, tie order
    and the LRU-side layout are the parent's (the same top-k kernel)."""

    def __init__(self, k_cache: torch.Tensor, num_pages: int, device="cuda"):
        super().__init__(k_cache, num_pages, device=device)
        num_heads, length, head_dim = k_cache.shape
        self._paged_keys = k_cache.to(device=device).contiguous().view(
            num_heads, num_pages, length // num_pages, head_dim)

    def scores(self, q: torch.Tensor) -> torch.Tensor:
        bsz, seq_len, num_q_heads, head_dim = q.shape
        assert bsz == 1, f"Only batch size 1 is supported, but got batch size {bsz}"
        assert num_q_heads % self.num_kv_heads == 0
        rep = num_q_heads // self.num_kv_heads
        H, L = self.num_kv_heads, self._paged_keys.shape[1]
        n_rows = seq_len * rep
        if self._scores is None or self._scores.shape[0] != n_rows:
            self._scores = torch.empty(n_rows, H, L, dtype=torch.float32, device=q.device)
        qv = q[0].view(seq_len, H, rep, head_dim)
        best = torch.einsum("hptd,shrd->srhpt", self._paged_keys, qv).amax(dim=-1)
        self._scores.copy_(best.reshape(n_rows, H, L))
        return self._scores
