"""One decode step of the HIP module against the CPU oracle, or against the invariants
that need no CPU walk; shared by the GPU tests."""

import math

import numpy as np
import torch

from oracle import dram_attention_oracle as O
from tests.util import close, same


def check_step(m, o, xq, xk, xv, start, out, t, atol, rtol, payload=True, output=True,
               own_scores=None):
    """`m` (a DRAMAttention with an LRUCache) has just run the step whose host-side
    inputs are xq/xk/xv at position `start` and returned `out`; `o` is the
    DecodeOracle in the state before that step.  The oracle is fed the kernel's
    scores (the contract is 'given identical scores'), which are themselves held
    within one rounding step of the oracle's own.  Request list, step counter,
    access times, both maps, hit mask and (with `payload`) the slots' contents must
    match bit for bit, the attention output (with `output`) within (atol, rtol).
    `own_scores`: the checker's scores when the module ranks by something other than the
    min/max bound."""
    lru = m.lru_cache
    scores = lru.top_k_selector._scores.cpu()
    own = O.scores_for_selection(xq, o.min_max) if own_scores is None else own_scores
    assert torch.all((scores - own).abs() <= own.abs() * 2.0 ** -7 + 1e-4), f"scores, step {t}"
    want = o.generate(xq, xk, xv, start, scores=scores)
    assert same(lru._topk_idx.cpu(), o.last_idx), f"selection, step {t}"
    assert lru.current_step.item() == o.state.step, f"step counter, step {t}"
    assert np.array_equal(lru.page_access_time.cpu().numpy(), o.state.time), f"time, step {t}"
    assert np.array_equal(lru.dram_page_to_hbm_page_mapping.cpu().numpy(), o.state.d2h), f"d2h, step {t}"
    assert np.array_equal(lru.hbm_page_to_dram_page_mapping.cpu().numpy(), o.state.h2d), f"h2d, step {t}"
    assert np.array_equal(lru._scratch.hit_mask.cpu().numpy().astype(bool), o.last_hit), f"hits, step {t}"
    if payload:
        assert same(lru.hbm_kv_cache.cpu(), o.hbm), f"slot payload, step {t}"
    if output:
        assert close(out.cpu().float(), want.float(), atol, rtol), f"output, step {t}"
    return want


def check_invariants(m, w, xq, xk, xv, out, t, dram_dev, step=None):
    """`m` (a DRAMAttention with an LRUCache over workload `w`) has just run decode step
    `t` (0-based) on the device tensors xq/xk/xv and returned `out`; `dram_dev` is a
    device copy of its page store.  Size-independent properties of the step, all on the
    GPU: the selection is ordered by (score descending, page ascending) and no
    unselected page beats it; the two maps are mutually inverse, every request is
    resident and stamped with this step; every slot holds exactly the page the map
    names; the output equals a dense fp32 softmax over all resident slots, the local
    window and the new token (atol 2e-2 / rtol 1e-2); the new token was appended."""
    lru = m.lru_cache
    dev = xq.device
    H, rep, kp, D = w.n_kv_heads, w.rep, w.pages_per_q_head, w.head_dim
    N, P, page = w.n_hbm_pages, w.n_dram_pages, w.page_size
    step = t + 1 if step is None else step
    idx, d2h, h2d = lru._topk_idx, lru.dram_page_to_hbm_page_mapping, lru.hbm_page_to_dram_page_mapping
    assert idx.shape == (H, rep * kp)
    scores = lru.top_k_selector._scores                         # (rep, H, P)
    sel = idx.view(H, rep, kp)
    s_sel = torch.gather(scores.transpose(0, 1), 2, sel)          # (H, rep, kp)
    assert torch.all((s_sel[..., :-1] > s_sel[..., 1:]) |
                     ((s_sel[..., :-1] == s_sel[..., 1:]) & (sel[..., :-1] < sel[..., 1:]))), f"order, step {t}"
    mask = torch.ones(H, rep, P, dtype=torch.bool, device=dev).scatter_(2, sel, False)
    rest = scores.transpose(0, 1).masked_fill(~mask, -float("inf"))
    best_rest, best_idx = rest.max(dim=-1)
    last, last_idx = s_sel[..., -1], sel[..., -1]
    assert torch.all((best_rest < last) | ((best_rest == last) & (best_idx > last_idx))), f"maximal, step {t}"
    # LRU maps: inverse of each other, all requests resident and touched now
    assert same(torch.gather(d2h, 1, h2d), torch.arange(N, device=dev).expand(H, N)), f"maps, step {t}"
    assert (d2h >= 0).sum().item() == H * N
    slots = torch.gather(d2h, 1, idx)
    assert torch.all(slots >= 0)
    assert torch.all(torch.gather(lru.page_access_time, 1, slots) == step)
    assert lru.current_step.item() == step
    # payload: every slot holds exactly the page the map names
    want_pages = torch.gather(dram_dev, 1, h2d[:, :, None].expand(-1, -1, dram_dev.shape[2]))
    assert same(lru.hbm_kv_cache, want_pages), f"payload, step {t}"
    # attention over all resident slots ++ local window ++ new token
    c = w.prompt_tokens + t - w.dram_tokens
    slots_kv = lru.hbm_kv_cache.view(H, N * page, 2, D)
    kk = torch.cat([slots_kv[:, :, 0], m.cache_k[0, : c + 1].transpose(0, 1)], 1).float()
    vv = torch.cat([slots_kv[:, :, 1], m.cache_v[0, : c + 1].transpose(0, 1)], 1).float()
    s = torch.einsum("hrd,htd->hrt", xq[0, 0].float().view(H, rep, D), kk) / math.sqrt(D)
    want = torch.einsum("hrt,htd->hrd", torch.softmax(s, -1), vv).reshape(H * rep, D)
    assert close(out[0, 0].float(), want, 2e-2, 1e-2), f"output, step {t}"
    assert same(m.cache_k[0, c], xk[0, 0]) and same(m.cache_v[0, c], xv[0, 0])
