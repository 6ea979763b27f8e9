"""One decode step of the HIP module against the CPU oracle, shared by the GPU tests."""

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
