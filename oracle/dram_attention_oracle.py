"""CPU oracle for the DRAM Attention decode path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU with torch/numpy, the algorithm of the
reference's generate-stage hot path.  It is the checker for the HIP kernels:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
it; the package `dram_attention_amd` never does.

Each function cites the reference lines it follows (paths relative to the
reference checkout, dram_attention/...).

How each function is pinned (tests/test_oracle.py):
  page_min_max        brute-force loops on small inputs; torch.aminmax.
  max_ip              independent einsum-free loop form; upper-bound property
                      score >= max_t q.k_t; equality at page_size 1; the second
                      statement of the formula in evaluation/quest/model.py:263-266.
  top_k_pages         brute-force selection on tiny rows incl. ties; torch.sort(stable).
  lru_load            the three known-answer tests of lru_triton_kernel_test.py:17-204
                      (restated as data), structural invariants (maps inverse of each
                      other, payload equals source page), LRU order on a hand-walked trace.
  LruState.initial    numbers of lru_cache_test.py:16-29,60-66 (512 / 102 / 64 pages).
  attention / combine dense softmax in fp64 over the concatenated tokens
                      (the LSE-merge identity).  The reference delegates this part to
                      flash-attn (not vendored, setup.py:21) and its own tests check
                      shapes only, so bit-level behaviour of that library (split order,
                      internal roundings) is PARITY UNPINNED; the closed form is the
                      contract, at the tolerance atol 2e-2 / rtol 1e-2 for bf16.
  decode geometry     lru_cache_test.py numbers; init_cache arithmetic by hand.
The fp16 scorer is unpinned as well (see max_ip), and the last-ulp fp32 summation
order of the reference's Triton scorer is likewise
unpinned (no GPU run of it is possible here); selection parity is therefore
stated "given identical scores".
"""

from __future__ import annotations

import math
import time
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np
import torch


# --------------------------------------------------------------------------
# subsystem 1: page summaries            topk_selector.py:25-34
# --------------------------------------------------------------------------
def page_min_max(k_cache: torch.Tensor, num_pages: int) -> torch.Tensor:
    """(H, S, D) -> (H, P, 2, D); [..., 0, :] = per-channel min over the page's
    tokens, [..., 1, :] = max.  Exact (comparisons only)."""
    H, S, D = k_cache.shape
    assert S % num_pages == 0, "Cache size must be divisible by num_pages."
    page = S // num_pages
    chunks = k_cache.reshape(H, num_pages, page, D).float()
    lo = chunks.amin(dim=2)
    hi = chunks.amax(dim=2)
    return torch.stack((lo, hi), dim=2).to(k_cache.dtype)


# --------------------------------------------------------------------------
# subsystem 2: page scores               max_ip_triton_kernel.py:95-133
# --------------------------------------------------------------------------
def max_ip(q: torch.Tensor, min_max: torch.Tensor) -> torch.Tensor:
    """score[n,h,l] = sum_d max(q[n,h,d]*mm[h,l,0,d], q[n,h,d]*mm[h,l,1,d]),
    returned in q.dtype (:99).  For 16-bit inputs the products are formed in the
    input type (rounded, :72,79), the maximum and the sum are fp32, and the sum is
    rounded once on output; for fp32 everything is fp32.
    That is what Triton does for bf16 (tl.maximum promotes bf16 to fp32).  For fp16
    Triton would stay in fp16 through the maximum and the sum, in a reduction order
    of its choosing; this function (and the HIP kernel) use the bf16 scheme for
    fp16 too.  PARITY UNPINNED for fp16: the reference's own test of that case
    checks the dtype only (max_ip_triton_kernel_test.py:18-26)."""
    N, H, D = q.shape
    H1, L, R, D1 = min_max.shape
    assert H1 == H and D1 == D and R == 2
    dt = q.dtype
    out = torch.empty(N, H, L, dtype=dt)
    for n in range(N):  # row by row keeps the (H, L, D) temporaries small
        qn = q[n].reshape(H, 1, D)
        lo = (qn * min_max[:, :, 0, :])  # rounded to dt by torch for 16-bit types
        hi = (qn * min_max[:, :, 1, :])
        # tl.maximum with its default PropagateNan.NONE (:80): a NaN product loses
        # against the other one, as with fmax; max_ip_ref's amax (:132) would
        # propagate it, the two statements differ only there
        best = torch.fmax(lo.float(), hi.float())
        out[n] = best.sum(dim=-1, dtype=torch.float32).to(dt)
    return out


def scores_for_selection(q: torch.Tensor, min_max: torch.Tensor) -> torch.Tensor:
    """fp32 view of the values the reference ranks on, for q (1, seq, Hq, D):
    rows are (seq*rep, Hkv, P) with row s*rep + r = query head h*rep + r
    (topk_selector.py:52-56)."""
    bsz, seq, Hq, D = q.shape
    assert bsz == 1
    Hkv = min_max.shape[0]
    assert Hq % Hkv == 0
    rep = Hq // Hkv
    qv = q[0].reshape(seq, Hkv, rep, D).transpose(1, 2).reshape(seq * rep, Hkv, D)
    return max_ip(qv, min_max).float()


# --------------------------------------------------------------------------
# subsystem 3: ordered top-k             topk_selector.py:57-61
# --------------------------------------------------------------------------
def top_k_pages(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest entries along the last axis, best first; equal
    scores in ascending index order (the reference's argsort leaves ties open;
    the contract of this build is the stable order)."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices
    return order[..., :k]


def select_pages(scores_rows: torch.Tensor, seq: int, rep: int, k: int) -> torch.Tensor:
    """(seq*rep, Hkv, P) scores -> (seq, Hkv, rep, k) page indices (:57-61)."""
    n_rows, Hkv, P = scores_rows.shape
    ip = scores_rows.reshape(seq, rep, Hkv, P).transpose(1, 2)
    return top_k_pages(ip, k)


def lru_index_list(topk: torch.Tensor) -> torch.Tensor:
    """(seq, Hkv, rep, k) -> (Hkv, seq*rep*k), the visiting order of the LRU walk
    (lru_cache.py:260-265)."""
    seq, Hkv, rep, k = topk.shape
    return topk.transpose(0, 1).reshape(Hkv, seq * rep * k)


# --------------------------------------------------------------------------
# subsystem 4: LRU state and the serial walk
#   lru_cache.py:112-209 (state), lru_triton_kernel.py:6-194 (walk)
# --------------------------------------------------------------------------
@dataclass
class LruState:
    time: np.ndarray   # (H, N_hbm) last-use step per slot
    d2h: np.ndarray    # (H, P) slot of a DRAM page, -1 = not resident
    h2d: np.ndarray    # (H, N_hbm) DRAM page held by a slot
    step: int = 0

    @staticmethod
    def initial(num_heads: int, num_dram_pages: int, num_hbm_pages: int) -> "LruState":
        """Most recent pages preloaded: slot s holds page P - N + s, all times 0
        (lru_cache.py:155-209)."""
        assert num_hbm_pages <= num_dram_pages, "HBM cache size must be smaller than DRAM cache size."
        d2h = np.full((num_heads, num_dram_pages), -1, dtype=np.int64)
        first = num_dram_pages - num_hbm_pages
        d2h[:, first:] = np.arange(num_hbm_pages)
        h2d = np.tile(np.arange(first, num_dram_pages, dtype=np.int64), (num_heads, 1))
        return LruState(np.zeros((num_heads, num_hbm_pages), dtype=np.float32), d2h, h2d, 0)

    def copy(self) -> "LruState":
        return LruState(self.time.copy(), self.d2h.copy(), self.h2d.copy(), self.step)


def hbm_page_count(num_dram_pages: int, page_size: int, lru_hbm_cache_size: Optional[int],
                   fraction: float = 0.2) -> int:
    """lru_cache.py:96-100."""
    if lru_hbm_cache_size is None:
        return int(num_dram_pages * fraction)
    return lru_hbm_cache_size // page_size


def lru_load(state: LruState, idx: np.ndarray, step: int,
             dram: Optional[np.ndarray] = None, hbm: Optional[np.ndarray] = None):
    """One call of load_lru_cache_ with current_step == step, in place on `state`
    (and on `hbm` when page payloads are given).

    Per head: (A) every requested page that is resident gets its slot's time set
    to `step` (:110-137); (B) the slots are ordered by time, ties by slot index
    (stable argsort, :170); (C) the requests are walked in order: a resident page
    is touched, a missing one takes the next slot of that order, whose old page
    is unmapped, both maps are rewritten and the page is copied (:34-107).

    Returns (hit_mask (H,K) bool, misses: list per head of (page, slot) in walk order).
    A slot whose map entry is -1 (never filled) unmaps nothing.
    """
    H, K = idx.shape
    n_hbm = state.h2d.shape[1]
    hit = np.zeros((H, K), dtype=bool)
    misses = []
    for h in range(H):
        time, d2h, h2d = state.time[h], state.d2h[h], state.h2d[h]
        req = idx[h]
        slots = d2h[req]
        time[slots[slots >= 0]] = step                       # (A)
        order = np.argsort(time, kind="stable")              # (B)
        ep = 0
        head_misses = []
        for k in range(K):                                   # (C)
            p = int(req[k])
            s = int(d2h[p])
            if s < 0:
                v = int(order[ep])
                time[v] = step
                old = int(h2d[v])
                if old >= 0:
                    d2h[old] = -1
                h2d[v] = p
                d2h[p] = v
                if hbm is not None:
                    hbm[h, v] = dram[h, p]
                head_misses.append((p, v))
                ep = (ep + 1) % n_hbm
            else:
                time[s] = step
                hit[h, k] = True
        misses.append(head_misses)
    state.step = step
    return hit, misses


# --------------------------------------------------------------------------
# subsystem 5: decode attention          dram_attention.py:179-238
# --------------------------------------------------------------------------
def attention_partial(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """softmax(q k^T * scale) v for one query token with GQA.
    q (Hq, D); k, v (Hkv, T, D); query head j uses kv head j // (Hq/Hkv).
    Returns (out (Hq, D) fp32, lse (Hq,) fp32, natural log).  What
    flash_attn_with_kvcache computes for a single query row (:195-223), with the
    library's default scale D**-0.5, in fp32."""
    Hq, D = q.shape
    Hkv, T, _ = k.shape
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    qf = q.float().reshape(Hkv, rep, D)
    s = torch.einsum("hrd,htd->hrt", qf, k.float()) * scale
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    out = torch.einsum("hrt,htd->hrd", p, v.float())
    return out.reshape(Hq, D), lse.reshape(Hq)


def combine(out_p: torch.Tensor, lse_p: torch.Tensor, out_s: torch.Tensor,
            lse_s: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Merge two partial attentions through their log-sum-exp (:225-238)."""
    lse = torch.logaddexp(lse_p, lse_s)
    w_p = torch.exp(lse_p - lse)[:, None]
    w_s = torch.exp(lse_s - lse)[:, None]
    return (out_p.float() * w_p + out_s.float() * w_s).to(dtype)


def split_hbm_pages(hbm: torch.Tensor, page_size: int, head_dim: int):
    """(H, N_hbm, page*2*D) slot array -> K, V each (H, N_hbm*page, D): token t of
    a page keeps K at t*2*D and V at t*2*D + D (lru_cache.py:131-141,236-240)."""
    H, n, _ = hbm.shape
    paged = hbm.reshape(H, n * page_size, 2, head_dim)
    return paged[:, :, 0, :], paged[:, :, 1, :]


def pack_pages(k: torch.Tensor, v: torch.Tensor, page_size: int) -> torch.Tensor:
    """(H, S, D) keys and values -> (H, P, page*2*D) page store (lru_cache.py:131-141)."""
    H, S, D = k.shape
    P = S // page_size
    out = torch.empty(H, P, page_size, 2, D, dtype=k.dtype)
    out[:, :, :, 0, :] = k.reshape(H, P, page_size, D)
    out[:, :, :, 1, :] = v.reshape(H, P, page_size, D)
    return out.reshape(H, P, page_size * 2 * D)


def dram_split(seqlen: int, local_cache_size: int, page_size: int) -> int:
    """Tokens that go to the paged prefix (dram_attention.py:76-77)."""
    return (seqlen - local_cache_size + page_size) // page_size * page_size


class DecodeOracle:
    """End-to-end restatement of DRAMAttention for one layer: init_cache
    (dram_attention.py:65-105) and the generate step (:144-238) with the LRU
    cache of lru_cache.py.  `round_partials` rounds the two partial outputs to
    the tensor dtype before the merge, as flash-attn's outputs are (:237)."""

    def __init__(self, max_output_length, lru_hbm_cache_size, local_cache_size, page_size,
                 top_k, n_kv_heads, head_dim, dtype=torch.bfloat16, round_partials=True):
        self.max_output_length = max_output_length
        self.lru_hbm_cache_size = lru_hbm_cache_size
        self.local_cache_size = local_cache_size
        self.page_size = page_size
        self.top_k = top_k
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.round_partials = round_partials
        self.cache_k = torch.zeros(local_cache_size + max_output_length, n_kv_heads, head_dim,
                                   dtype=dtype)
        self.cache_v = torch.zeros_like(self.cache_k)
        self.dram_kv_cache_size = None
        self.uses_lru = False

    def init_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor, force_lru: bool = False):
        """k_cache, v_cache: (1, S, Hkv, D).  `force_lru` builds the page cache even when
        the prefix fits it (what constructing LRUCache directly over the prefix gives,
        lru_cache.py:188-190 only asks for num_hbm_pages <= num_dram_pages): every page
        is resident from the start and every request hits."""
        bsz, S, H, D = k_cache.shape
        assert bsz == 1, "Only support batch size 1"
        self.dram_kv_cache_size = dram_split(S, self.local_cache_size, self.page_size)
        tail = S - self.dram_kv_cache_size
        self.cache_k[:tail] = k_cache[0, self.dram_kv_cache_size:]
        self.cache_v[:tail] = v_cache[0, self.dram_kv_cache_size:]
        pk = k_cache[0, : self.dram_kv_cache_size].transpose(0, 1).contiguous()
        pv = v_cache[0, : self.dram_kv_cache_size].transpose(0, 1).contiguous()
        self.uses_lru = force_lru or self.dram_kv_cache_size > self.lru_hbm_cache_size
        if self.uses_lru:
            P = self.dram_kv_cache_size // self.page_size
            n_hbm = self.lru_hbm_cache_size // self.page_size
            self.min_max = page_min_max(pk, P)
            self.dram = pack_pages(pk, pv, self.page_size)
            self.state = LruState.initial(H, P, n_hbm)
            self.hbm = self.dram[:, P - n_hbm:].clone()
            self.kp = self.top_k // self.page_size
        else:
            self.static_k, self.static_v = pk, pv

    def select(self, xq: torch.Tensor, scores: Optional[torch.Tensor] = None,
               timings: Optional[dict] = None) -> torch.Tensor:
        """(Hkv, rep*kp) page list of this step; `scores` overrides the oracle's own
        (seq*rep, Hkv, P) scores (used to test selection on identical scores)."""
        bsz, seq, Hq, D = xq.shape
        rep = Hq // self.n_kv_heads
        t0 = time.perf_counter()
        if scores is None:
            scores = scores_for_selection(xq, self.min_max)
        t1 = time.perf_counter()
        idx = lru_index_list(select_pages(scores, seq, rep, min(self.kp, self.min_max.shape[1])))
        if timings is not None:
            timings["score"] = timings.get("score", 0.0) + t1 - t0
            timings["top_k"] = timings.get("top_k", 0.0) + time.perf_counter() - t1
        return idx

    def generate(self, xq, xk, xv, start_pos: int, scores: Optional[torch.Tensor] = None,
                 idx: Optional[torch.Tensor] = None, timings: Optional[dict] = None):
        """xq (1,1,Hq,D), xk/xv (1,1,Hkv,D) -> (1,1,Hq,D) in xq.dtype.  `timings`, when
        given, accumulates seconds per stage (score, top_k, lru, attention)."""
        if self.uses_lru:
            if idx is None:
                idx = self.select(xq, scores, timings)
            self.last_idx = idx
            t0 = time.perf_counter()
            hbm_np = self.hbm.view(torch.int16).numpy() if self.hbm.element_size() == 2 \
                else self.hbm.numpy()
            dram_np = self.dram.view(torch.int16).numpy() if self.dram.element_size() == 2 \
                else self.dram.numpy()
            self.last_hit, self.last_misses = lru_load(
                self.state, idx.numpy(), self.state.step + 1, dram_np, hbm_np)
            pk, pv = split_hbm_pages(self.hbm, self.page_size, self.head_dim)
            if timings is not None:
                timings["lru"] = timings.get("lru", 0.0) + time.perf_counter() - t0
        else:
            pk, pv = self.static_k, self.static_v
        t0 = time.perf_counter()
        c = int(start_pos) - self.dram_kv_cache_size
        self.cache_k[c] = xk[0, 0]
        self.cache_v[c] = xv[0, 0]
        q = xq[0, 0]
        out_p, lse_p = attention_partial(q, pk, pv)
        out_s, lse_s = attention_partial(q, self.cache_k[: c + 1].transpose(0, 1),
                                         self.cache_v[: c + 1].transpose(0, 1))
        if self.round_partials:
            out_p, out_s = out_p.to(self.dtype), out_s.to(self.dtype)
        out = combine(out_p, lse_p, out_s, lse_s, xq.dtype).reshape(1, 1, *q.shape)
        if timings is not None:
            timings["attention"] = timings.get("attention", 0.0) + time.perf_counter() - t0
        return out
