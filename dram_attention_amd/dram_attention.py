"""DRAM Attention: long prefix in pinned host DRAM, hot pages in an HBM LRU,
recent tokens in a local HBM window; decode attends over (resident pages ++
local window ++ new token) in one split-K pass.

Mirrors dram_attention/dram_attention.py of the reference (DRAMAttention
:7-238): constructor, buffers, ``init_cache`` and ``forward(xq, xk, xv, *,
start_pos, stage)`` keep their meaning and error behaviour.
"""

from __future__ import annotations

import ctypes
import math

import torch
import torch.nn.functional as F

from . import _lib
from .lru_cache import DummyCache, LRUCache
from .lru_kernel import GATHER_BLOCKS, gather_attend_supported, host_link_gbps
from .topk_selector import TokenMaxTopKSelector


class PagedPrefix:
    """Says that the prefix handed to :func:`decode_attention` is the slot array of
    an LRU page cache whose page stream for this step may still be running.

    FIRST attends over the local window and every slot that keeps its page,
    FIRST_MERGE folds those partial results into one (both may run next to the
    stream), SECOND (after the stream has finished) attends over the re-assigned
    slots and writes the output; FIRST | SECOND does everything at once.  With
    STREAM the page stream itself runs inside the launch of the FIRST pass;
    SECOND | MERGE_ALL is the final merge as a call of its own after FIRST (| STREAM)
    without FIRST_MERGE."""

    FIRST, SECOND, FIRST_MERGE, STREAM, MERGE_ALL = 1, 2, 4, 8, 16

    def __init__(self, page_size: int, scratch, current_step: torch.Tensor, phase: int,
                 gather_blocks: int = 0, page_stores=None, link_gbps: float = 0.0,
                 block_gbps: float = 0.0):
        self.page_size = page_size
        self.scratch = scratch
        self.current_step = current_step
        self.phase = phase
        # blocks per kv head of a page stream that attends over the pages it moves
        # (0: the SECOND pass attends over the re-assigned slots)
        self.gather_blocks = gather_blocks
        # STREAM: (dram_kv_cache, its device-visible address, hbm_kv_cache); the page
        # stream then runs inside the launch of the FIRST pass
        self.page_stores = page_stores
        # STREAM: the host link's rate for reads issued by a kernel and the rate at which
        # one workgroup reads HBM, GB/s (0 = the library's defaults); they decide how
        # many workgroups compute the first pass next to a long stream, not what it computes
        self.link_gbps = link_gbps
        self.block_gbps = block_gbps

    def as_struct(self) -> "_lib.PagedOverlap":
        s = self.scratch
        o = _lib.PagedOverlap(
            page_size=self.page_size, phase=self.phase, slot_epoch=s.slot_epoch.data_ptr(),
            slot_epoch_head_stride=s.slot_epoch.stride(0), epoch=self.current_step.data_ptr(),
            miss_slot=s.miss_slot.data_ptr(), miss_count=s.miss_count.data_ptr(),
            miss_capacity=s.miss_slot.shape[1], gather_blocks=self.gather_blocks)
        if self.phase & self.STREAM:
            dram, dram_ptr, hbm = self.page_stores
            esz = dram.element_size()
            o.dram, o.hbm, o.miss_page = dram_ptr, hbm.data_ptr(), s.miss_page.data_ptr()
            o.dram_head_stride_bytes = dram.stride(0) * esz
            o.dram_page_stride_bytes = dram.stride(1) * esz
            o.hbm_head_stride_bytes = hbm.stride(0) * esz
            o.hbm_slot_stride_bytes = hbm.stride(1) * esz
            o.link_gbps, o.block_gbps = self.link_gbps, self.block_gbps
        return o


def attention_workspace(Hq: int, Hkv: int, D: int, dtype: torch.dtype, p_len: int, capacity: int,
                        miss_tokens: int, device) -> torch.Tensor:
    need = _lib.load().da_decode_attention_workspace_bytes(
        Hq, Hkv, D, _lib.dtype_code(dtype), p_len, capacity, miss_tokens)
    if need == 0:
        raise RuntimeError(f"decode attention does not cover head_dim={D} dtype={dtype}")
    return torch.empty((need + 3) // 4, dtype=torch.float32, device=device)


def decode_attention(
    xq: torch.Tensor,
    prefix_k: torch.Tensor,
    prefix_v: torch.Tensor,
    cache_k: torch.Tensor,
    cache_v: torch.Tensor,
    cache_len,
    new_k: torch.Tensor | None,
    new_v: torch.Tensor | None,
    *,
    workspace: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    lse: torch.Tensor | None = None,
    scale: float | None = None,
    paged: PagedPrefix | None = None,
    cache_len_offset: int = 0,
) -> torch.Tensor:
    """One query token against [prefix ++ cache rows 0..cache_len ++ new token].

    xq (Hq, D); prefix_k/v (Hkv, T, D) views with a dense last axis (T may be 0);
    cache_k/v (capacity, Hkv, D); cache_len an int, or a one-element int32 GPU
    tensor to which ``cache_len_offset`` is added inside the kernel (so a device
    position counter needs no arithmetic launch); new_k/new_v (Hkv, D) are
    appended at row cache_len (or None).
    Returns (Hq, D) in xq.dtype; fills ``lse`` (Hq, fp32) when given.
    With ``paged`` the work is split around a concurrent page stream; the same
    workspace and ``out`` must be passed to every call of the step.
    """
    Hq, D = xq.shape
    Hkv = cache_k.shape[1]
    _lib.require_gpu(xq, "xq")
    lib = _lib.load()
    dt = _lib.dtype_code(xq.dtype)
    p_len = prefix_k.shape[1] if prefix_k is not None else 0
    capacity = cache_k.shape[0]
    if out is None:
        out = torch.empty(Hq, D, dtype=xq.dtype, device=xq.device)
    if workspace is None:
        miss_tokens = paged.scratch.miss_slot.shape[1] * paged.page_size if paged else 0
        workspace = attention_workspace(Hq, Hkv, D, xq.dtype, p_len, capacity, miss_tokens,
                                        xq.device)
    if isinstance(cache_len, torch.Tensor):
        _lib.require_gpu(cache_len, "cache_len")
        if cache_len.dtype != torch.int32:
            raise TypeError("a device-side cache length must be int32")
        len_host, len_dev = int(cache_len_offset), cache_len.data_ptr()
    else:
        len_host, len_dev = int(cache_len), None
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    for t in (xq, prefix_k, prefix_v, cache_k, cache_v, new_k, new_v):
        if t is not None and t.numel() and t.stride(-1) != 1:
            raise ValueError("head_dim must be the dense axis of every operand")
    overlap = paged.as_struct() if paged is not None else None
    _lib.check(
        lib.da_decode_attention_paged(
            xq.data_ptr(), xq.stride(0), Hq, Hkv, D, dt,
            prefix_k.data_ptr() if p_len else None, prefix_v.data_ptr() if p_len else None,
            prefix_k.stride(1) if p_len else 0, prefix_k.stride(0) if p_len else 0, p_len,
            cache_k.data_ptr(), cache_v.data_ptr(), cache_k.stride(0), cache_k.stride(1),
            capacity, len_host, len_dev,
            new_k.data_ptr() if new_k is not None else None,
            new_v.data_ptr() if new_v is not None else None,
            new_k.stride(0) if new_k is not None else 0,
            scale, out.data_ptr(), out.stride(0),
            lse.data_ptr() if lse is not None else None,
            workspace.data_ptr(), workspace.numel() * workspace.element_size(),
            ctypes.byref(overlap) if overlap is not None else None,
            _lib.stream_ptr(xq.device),
        ),
        "da_decode_attention",
    )
    return out


def prefill_attention_supported(xq: torch.Tensor) -> bool:
    """Whether the library's own causal prefill kernel takes this query tensor."""
    return (xq.is_cuda and xq.dtype in (torch.bfloat16, torch.float16)
            and xq.shape[-1] in (64, 128))


def prefill_attention(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, *,
                      scale: float | None = None, lse: torch.Tensor | None = None) -> torch.Tensor:
    """Causal attention over the prompt on the library's kernel (da_prefill_attention):
    (1,S,Hq,D), (1,S,Hkv,D) x 2 -> (1,S,Hq,D); fills ``lse`` (Hq, S) fp32 when given.
    Replaces flash_attn_func(xq, xk, xv, causal=True), reference dram_attention.py:136."""
    bsz, S, Hq, D = xq.shape
    assert bsz == 1, "Only support batch size 1"
    Hkv = xk.shape[2]
    for name, t in (("xq", xq), ("xk", xk), ("xv", xv)):
        _lib.require_gpu(t, name)
        if t.stride(-1) != 1:
            raise ValueError("head_dim must be the dense axis of every operand")
    if xk.shape != xv.shape or xk.shape[1] != S or xk.shape[3] != D or not (
            xq.dtype == xk.dtype == xv.dtype):
        raise ValueError("query, keys and values must agree in length, head size and type")
    out = torch.empty(1, S, Hq, D, dtype=xq.dtype, device=xq.device)
    if lse is not None and (lse.shape != (Hq, S) or lse.dtype != torch.float32
                            or not lse.is_contiguous()):
        raise ValueError("lse must be a contiguous fp32 tensor of shape (Hq, S)")
    _lib.check(
        _lib.load().da_prefill_attention(
            xq.data_ptr(), xq.stride(1), xq.stride(2), xk.data_ptr(), xk.stride(1), xk.stride(2),
            xv.data_ptr(), xv.stride(1), xv.stride(2), S, Hq, Hkv, D, _lib.dtype_code(xq.dtype),
            float(scale) if scale is not None else 1.0 / math.sqrt(D), out.data_ptr(),
            out.stride(1), out.stride(2), lse.data_ptr() if lse is not None else None,
            _lib.stream_ptr(xq.device)),
        "da_prefill_attention")
    return out


def causal_prefill_attention(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor,
                             backend: str = "auto") -> torch.Tensor:
    """Dense causal attention over the prompt, (1,S,Hq,D) -> (1,S,Hq,D), in place of
    flash_attn_func (reference dram_attention.py:136).  ``backend``:
      "native"  the library's kernel (16-bit types, head_dim 64 or 128; raises otherwise)
      "sdpa"    torch's fused scaled_dot_product_attention (raises if no fused kernel
                takes the shape)
      "blocked" torch's attention over blocks of query rows with an explicit mask, the
                block sized so that the scores torch may materialise for it (Hq x rows x S
                fp32) stay within 1 GiB: at most 1024 rows, 64 at 128K tokens and 32
                heads (any type, CPU too)
      "auto"    native where it applies, else sdpa, else blocked."""
    if backend not in ("auto", "native", "sdpa", "blocked"):
        raise RuntimeError(f"Unsupported prefill backend: {backend}")
    if backend == "native" or (backend == "auto" and prefill_attention_supported(xq)):
        return prefill_attention(xq, xk, xv)
    bsz, S, Hq, D = xq.shape
    Hkv = xk.shape[2]
    q = xq.transpose(1, 2)
    k = xk.transpose(1, 2)
    v = xv.transpose(1, 2)
    gqa = Hq != Hkv
    if backend == "sdpa" or (backend == "auto" and xq.is_cuda):
        from torch.nn.attention import SDPBackend, sdpa_kernel

        try:
            with sdpa_kernel([SDPBackend.FLASH_ATTENTION, SDPBackend.EFFICIENT_ATTENTION]):
                o = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=gqa)
            return o.transpose(1, 2).contiguous()
        except RuntimeError:
            if backend == "sdpa":
                raise
    out = torch.empty_like(xq)
    block = max(16, min(1024, (1 << 28) // max(1, Hq * S)))
    for s0 in range(0, S, block):
        s1 = min(S, s0 + block)
        # rows s0..s1 see keys 0..s1; row i of the block may look at key j <= s0 + i
        mask = torch.ones(s1 - s0, s1, dtype=torch.bool, device=xq.device).tril_(diagonal=s0)
        o = F.scaled_dot_product_attention(q[:, :, s0:s1], k[:, :, :s1], v[:, :, :s1],
                                           attn_mask=mask, enable_gqa=gqa)
        out[:, s0:s1] = o.transpose(1, 2)
    return out


class DRAMAttention(torch.nn.Module):
    """Drop-in for the reference module of the same name.

    Two caches: ``cache_k/cache_v`` hold the local window (last
    ``local_cache_size`` prompt tokens, rounded to pages, plus everything
    generated); the rest of the prompt is paged, in host DRAM behind an
    ``LRUCache`` (or entirely in HBM behind a ``DummyCache`` when it fits
    into ``lru_hbm_cache_size``).
    """

    def __init__(
        self,
        max_output_length: int,
        lru_hbm_cache_size: int,
        local_cache_size: int,
        page_size: int,
        top_k: int,
        n_kv_heads: int,
        head_dim: int,
        device: str = "cuda",
        dtype: torch.dtype = torch.bfloat16,
    ):
        super().__init__()
        self.max_output_length = max_output_length
        self.page_size = page_size
        self.dram_kv_cache_size = None  # set by init_cache
        self.lru_hbm_cache_size = lru_hbm_cache_size
        self.local_cache_size = local_cache_size
        self.top_k = top_k
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.num_page = self.lru_hbm_cache_size // self.page_size
        self.device = device
        cache_shape = (1, local_cache_size + max_output_length, n_kv_heads, head_dim)
        self.register_buffer("cache_k", torch.zeros(cache_shape, device=device, dtype=dtype))
        self.register_buffer("cache_v", torch.zeros(cache_shape, device=device, dtype=dtype))
        self._workspace = None
        self._side_stream = None
        # run the page stream and the first attention pass concurrently (two streams)
        self.overlap_page_stream = True
        # attend over the streamed pages inside the page stream itself (when the
        # shape allows) instead of a pass over them after the stream
        self.attend_on_page_stream = True
        # "resident": the prefix pass covers every slot of the page cache, as the
        # reference does (dram_attention.py:195-205).  "selected": only the pages this
        # step selected, each query head over its own list: the Quest baseline the
        # reference compares itself with (evaluation/quest/model.py:263-316), on the
        # same page cache and kernels.
        self.attention_scope = "resident"
        # "bound": pages ranked by the min/max upper bound (topk_selector.py:37-61 of the
        # reference).  "token_max": by the best token of each page, the accuracy ceiling
        # of page selection (evaluation/quest-top-k-oracle/model.py:267-275); keeps all
        # prefix keys on the device.  Read by init_cache.
        self.page_selector = "bound"
        # Workgroups of the page stream in all, and two rates of the machine (GB/s) that
        # time the stream + attention launch: what a kernel's reads of the pinned store
        # reach (set by init_cache from one timed pinned copy; a kernel gets about 0.95
        # of a copy engine's rate) and what one workgroup alone reads from HBM (0 = the
        # library's default).  Results do not depend on any of the three.
        self.stream_blocks = GATHER_BLOCKS
        # which implementation stage="prefill" attends with: see causal_prefill_attention
        self.prefill_backend = "auto"
        self.link_gbps = 0.0
        self.block_gbps = 0.0

    def init_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor):
        """Split the prompt's (1,S,Hkv,D) keys/values into the paged prefix and the
        local window, and build the page cache."""
        bsz, seqlen, H, D = k_cache.shape
        assert bsz == 1, "Only support batch size 1"
        paged = (seqlen - self.local_cache_size + self.page_size) // self.page_size
        self.dram_kv_cache_size = paged * self.page_size
        tail = seqlen - self.dram_kv_cache_size
        self.cache_k[:, :tail].copy_(k_cache[:, self.dram_kv_cache_size:], non_blocking=True)
        self.cache_v[:, :tail].copy_(v_cache[:, self.dram_kv_cache_size:], non_blocking=True)
        prefix_k = k_cache[0, : self.dram_kv_cache_size].transpose(0, 1)
        prefix_v = v_cache[0, : self.dram_kv_cache_size].transpose(0, 1)
        if self.dram_kv_cache_size > self.lru_hbm_cache_size:
            self.lru_cache = LRUCache(
                k_cache=prefix_k,
                v_cache=prefix_v,
                page_size=self.page_size,
                top_k=self.top_k // self.page_size,
                lru_hbm_cache_size=self.lru_hbm_cache_size,
                device=self.device,
            )
            self.link_gbps = 0.95 * host_link_gbps(self.cache_k.device)
            if self.page_selector == "token_max":
                self.lru_cache.top_k_selector = TokenMaxTopKSelector(
                    prefix_k, self.lru_cache.num_dram_pages, device=self.device)
            elif self.page_selector != "bound":
                raise RuntimeError(f"Unsupported page selector: {self.page_selector}")
        else:
            self.lru_cache = DummyCache(k_cache=prefix_k, v_cache=prefix_v, device=self.device)
        self._workspace = None

    def _attend_selected(self, xq, xk, xv, cache_len, offset, idx, out):
        """The Quest baseline's attention (evaluation/quest/model.py:263-316): query head
        j attends over the pages of ITS top-k list, plus the local window and the new
        token; the two partial results are combined by their log-sum-exp.  A comparison
        variant, not the hot path: the selected pages are gathered from their slots by
        torch ops and the two passes are separate calls of the decode kernel."""
        lru = self.lru_cache
        Hq, D = xq.shape[2], xq.shape[3]
        Hkv, K = idx.shape
        if K > lru.num_hbm_pages:
            raise RuntimeError("the selected-pages scope needs every selected page resident: "
                               f"{K} requests per kv head exceed {lru.num_hbm_pages} slots")
        lru.gather_(K)                                   # the missed pages land in their slots
        slots = torch.gather(lru.dram_page_to_hbm_page_mapping, 1, idx)        # (Hkv, rep*kp)
        pages = lru.hbm_kv_cache
        sel = torch.gather(pages, 1, slots[..., None].expand(-1, -1, pages.shape[2]))
        sel = sel.view(Hq, (K // (Hq // Hkv)) * self.page_size, 2, D)   # rows of q head h*rep + r
        no_cache = xq.new_empty(0, Hq, D)
        lse_p = torch.empty(Hq, dtype=torch.float32, device=xq.device)
        lse_s = torch.empty_like(lse_p)
        out_p = decode_attention(xq[0, 0], sel[:, :, 0], sel[:, :, 1], no_cache, no_cache, 0, None,
                                 None, lse=lse_p)
        out_s = decode_attention(xq[0, 0], None, None, self.cache_k[0], self.cache_v[0], cache_len,
                                 xk[0, 0], xv[0, 0], lse=lse_s, cache_len_offset=offset)
        lse = torch.logaddexp(lse_p, lse_s)
        mixed = (out_p.float() * torch.exp(lse_p - lse)[:, None]
                 + out_s.float() * torch.exp(lse_s - lse)[:, None])
        out[0, 0].copy_(mixed)

    def init_cache_from_file(self, cache_dir: str, index: int) -> int:
        """init_cache from the chat example's per-layer file ``NN_cache.pth``; returns
        the prompt length (the position of the first generated token)."""
        from .kv_file import load_layer_cache

        k, v = load_layer_cache(cache_dir, index, self.device)
        self.init_cache(k.to(self.cache_k.dtype), v.to(self.cache_v.dtype))
        return k.shape[1]

    def forward(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, *, start_pos,
                stage: str):
        bsz, seqlen, H, D = xq.shape
        assert bsz == 1, "Only support batch size 1"
        if stage == "prefill":
            output = causal_prefill_attention(xq, xk, xv, self.prefill_backend)
            self.init_cache(xk, xv)
            return output
        elif stage == "generate":
            return self._generate(xq, xk, xv, start_pos)
        else:
            raise RuntimeError(f"Unsupported stage: {stage}")

    def _generate(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, start_pos):
        """One decode step: select pages, update the LRU, then one attention pass
        over resident pages, local window and the new token (appended in place).
        The missed pages stream in on a side stream while attention already
        covers the local window and every slot that keeps its page."""
        return self.attend_(xq, xk, xv, start_pos, self.select_(xq))

    def select_(self, xq: torch.Tensor):
        """First half of a decode step: page scores, ordered top-k and the LRU update
        (three launches that touch neither the host link nor K/V).  Returns what
        :meth:`attend_` needs to finish the step, or None with a static cache.  The
        two halves may be issued on different streams as long as attend_ is ordered
        after select_ of the same step and before select_ of the next one."""
        bsz, seqlen, Hq, D = xq.shape
        if seqlen != 1:
            raise RuntimeError("generate handles one token per call")
        lru = self.lru_cache
        if not isinstance(lru, LRUCache):
            return None
        idx = lru.select_(xq)
        return idx, lru.update_(idx)

    def attend_(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor, start_pos, selected,
                defer_merge: bool = False):
        """Second half of a decode step: the page stream for the misses select_ found
        and attention over resident pages, local window and the new token.
        ``defer_merge``: when the step's final merge is a launch of its own (page
        stream and first pass in one launch), leave it out and return (out, merge)
        where ``merge()`` issues it on whatever stream is current, ordered after
        this call; ``out`` is complete only then.  Otherwise returns (out, None)."""
        bsz, seqlen, Hq, D = xq.shape
        if seqlen != 1:
            raise RuntimeError("generate handles one token per call")
        if isinstance(start_pos, torch.Tensor):
            # the position stays on the device; the kernel subtracts the paged prefix
            cache_len = start_pos if start_pos.dtype == torch.int32 else start_pos.to(torch.int32)
            offset = -self.dram_kv_cache_size
        else:
            cache_len, offset = int(start_pos) - self.dram_kv_cache_size, 0
        out = torch.empty(1, 1, Hq, D, dtype=xq.dtype, device=xq.device)
        lru = self.lru_cache
        if not isinstance(lru, LRUCache):
            prefix_k, prefix_v = lru.get_kv_cache_(xq)
            if self._workspace is None:
                self._workspace = attention_workspace(Hq, self.n_kv_heads, D, xq.dtype,
                                                      prefix_k.shape[1], self.cache_k.shape[1], 0,
                                                      xq.device)
            decode_attention(xq[0, 0], prefix_k, prefix_v, self.cache_k[0], self.cache_v[0],
                             cache_len, xk[0, 0], xv[0, 0], workspace=self._workspace,
                             out=out[0, 0], cache_len_offset=offset)
            return (out, None) if defer_merge else out

        idx, scratch = selected
        if self.attention_scope == "selected":
            self._attend_selected(xq, xk, xv, cache_len, offset, idx, out)
            return (out, None) if defer_merge else out
        if self.attention_scope != "resident":
            raise RuntimeError(f"Unsupported attention scope: {self.attention_scope}")
        prefix_k, prefix_v = lru.views()
        if self._workspace is None:
            self._workspace = attention_workspace(
                Hq, self.n_kv_heads, D, xq.dtype, prefix_k.shape[1], self.cache_k.shape[1],
                scratch.miss_slot.shape[1] * self.page_size, xq.device)
        args = (xq[0, 0], prefix_k, prefix_v, self.cache_k[0], self.cache_v[0], cache_len,
                xk[0, 0], xv[0, 0])
        k = idx.shape[1]
        # Attention over the pages paged in this step rides on the page stream when
        # the shape allows; otherwise a tail pass covers them after the stream.
        fused = self.attend_on_page_stream and gather_attend_supported(
            Hq, self.n_kv_heads, D, self.page_size, xq.dtype)
        blocks = max(1, min(self.stream_blocks // self.n_kv_heads, k)) if fused else 0

        def stream_pages():
            if fused:
                lru.gather_attend_(k, xq[0, 0], 1.0 / math.sqrt(D), self.cache_k.shape[1],
                                   self._workspace, blocks)
            else:
                lru.gather_(k)

        def attend(phase):
            decode_attention(*args, workspace=self._workspace, out=out[0, 0],
                             cache_len_offset=offset,
                             paged=PagedPrefix(self.page_size, scratch, lru.current_step, phase,
                                               blocks))

        P = PagedPrefix
        if not self.overlap_page_stream:
            stream_pages()
            # the same kernels as the concurrent order, so the same bits
            attend((P.FIRST | P.SECOND) if fused else (P.FIRST | P.FIRST_MERGE | P.SECOND))
            return (out, None) if defer_merge else out
        if fused:
            # page stream and first attention pass in one launch, then the merge: the
            # step stays a plain chain of launches on the caller's stream
            def launch(phase):
                decode_attention(*args, workspace=self._workspace, out=out[0, 0],
                                 cache_len_offset=offset,
                                 paged=PagedPrefix(self.page_size, scratch, lru.current_step,
                                                   phase, blocks, lru.page_stores(),
                                                   self.link_gbps, self.block_gbps))

            if defer_merge:
                launch(P.STREAM | P.FIRST)
                return out, (lambda: launch(P.SECOND | P.MERGE_ALL))
            launch(P.STREAM | P.FIRST | P.SECOND)
            return out
        # Shapes the fused stream does not take: pages stream in on a side stream
        # next to the first pass, and a tail pass covers them after the join.
        main = torch.cuda.current_stream(xq.device)
        if self._side_stream is None:
            self._side_stream = torch.cuda.Stream(device=xq.device)
        side = self._side_stream
        side.wait_stream(main)                      # the miss list is ready
        with torch.cuda.stream(side):
            stream_pages()
        attend(P.FIRST | P.FIRST_MERGE)
        main.wait_stream(side)                      # the pages have landed
        attend(P.SECOND)
        return (out, None) if defer_merge else out
