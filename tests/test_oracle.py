"""Pins the CPU oracle: reference known-answer vectors, brute force on tiny
inputs, closed forms and invariants.  No GPU needed."""

import itertools
import math

import numpy as np
import pytest
import torch

from oracle import dram_attention_oracle as O
from tests.golden import lru_kats


# ---------------------------------------------------------------- page min/max
def test_page_min_max_brute_force():
    g = torch.Generator().manual_seed(1)
    k = torch.randn(3, 40, 5, generator=g)
    mm = O.page_min_max(k, 10)
    assert mm.shape == (3, 10, 2, 5)
    for h, p, d in itertools.product(range(3), range(10), range(5)):
        vals = [k[h, p * 4 + t, d].item() for t in range(4)]
        assert mm[h, p, 0, d].item() == min(vals)
        assert mm[h, p, 1, d].item() == max(vals)


def test_page_min_max_matches_aminmax_bf16():
    g = torch.Generator().manual_seed(2)
    k = torch.randn(2, 64, 8, generator=g).bfloat16()
    mm = O.page_min_max(k, 4)
    lo, hi = torch.aminmax(k.view(2, 4, 16, 8), dim=2)
    assert torch.equal(mm[:, :, 0], lo) and torch.equal(mm[:, :, 1], hi)
    assert mm.dtype == torch.bfloat16


# ---------------------------------------------------------------- scorer
def test_max_ip_loop_form_fp32():
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 3, 6, generator=g)
    mm = torch.randn(3, 5, 2, 6, generator=g)
    got = O.max_ip(q, mm)
    for n, h, l in itertools.product(range(2), range(3), range(5)):
        want = sum(max(q[n, h, d].item() * mm[h, l, 0, d].item(),
                       q[n, h, d].item() * mm[h, l, 1, d].item()) for d in range(6))
        assert got[n, h, l].item() == pytest.approx(want, rel=1e-5, abs=1e-5)


def test_max_ip_is_upper_bound_and_tight_for_single_token_pages():
    g = torch.Generator().manual_seed(4)
    H, S, D, page = 2, 64, 16, 8
    k = torch.randn(H, S, D, generator=g)
    q = torch.randn(3, H, D, generator=g)
    score = O.max_ip(q, O.page_min_max(k, S // page))           # (3, H, 8)
    dots = torch.einsum("nhd,hsd->nhs", q, k).view(3, H, S // page, page)
    assert torch.all(score >= dots.amax(dim=-1) - 1e-5)          # Quest's bound
    # page of one token: min == max == the key, the bound is the dot product
    score1 = O.max_ip(q, O.page_min_max(k, S))
    assert torch.allclose(score1, torch.einsum("nhd,hsd->nhs", q, k), atol=1e-5)


def test_max_ip_quest_statement():
    # the same bound written Quest's way: sign(q) picks max or min per channel
    g = torch.Generator().manual_seed(5)
    q = torch.randn(4, 2, 8, generator=g)
    k = torch.randn(2, 32, 8, generator=g)
    mm = O.page_min_max(k, 8)
    pick = torch.where(q[:, :, None, :] >= 0, mm[None, :, :, 1, :], mm[None, :, :, 0, :])
    assert torch.allclose(O.max_ip(q, mm), (q[:, :, None, :] * pick).sum(-1), atol=1e-5)


def test_max_ip_nan_product_loses_against_the_other_product():
    """tl.maximum with its default (PropagateNan.NONE, the reference kernel's call at
    max_ip_triton_kernel.py:80) returns the other operand when one product is NaN:
    0 * inf contributes max(0 * min, NaN) = 0 * min, not NaN.  Both NaN stays NaN."""
    q = torch.tensor([[[0.0, 2.0]]])                                   # (1, 1, 2)
    mm = torch.tensor([[[[1.0, -1.0], [float("inf"), 3.0]]]])          # min (1,-1), max (inf,3)
    assert O.max_ip(q, mm).item() == 0.0 * 1.0 + 2.0 * 3.0
    mm_nan = torch.tensor([[[[float("nan"), -1.0], [float("nan"), 3.0]]]])
    assert torch.isnan(O.max_ip(torch.tensor([[[1.0, 2.0]]]), mm_nan)).all()
    # hand-written loop over the same rule
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 1, 6, generator=g)
    q[0, 0, 2] = 0.0
    mm = torch.randn(1, 3, 2, 6, generator=g)
    mm[0, 1, 1, 2] = float("inf")
    want = torch.zeros(2, 1, 3)
    for n in range(2):
        for l in range(3):
            acc = 0.0
            for d in range(6):
                a, b = float(q[n, 0, d] * mm[0, l, 0, d]), float(q[n, 0, d] * mm[0, l, 1, d])
                acc += b if a != a else (a if b != b else max(a, b))
            want[n, 0, l] = acc
    assert torch.allclose(O.max_ip(q, mm), want, atol=1e-5)


def test_max_ip_bf16_rounding_points():
    g = torch.Generator().manual_seed(6)
    q = torch.randn(2, 2, 32, generator=g).bfloat16()
    mm = torch.randn(2, 7, 2, 32, generator=g).bfloat16()
    got = O.max_ip(q, mm)
    assert got.dtype == torch.bfloat16
    # products rounded to bf16, fp32 max and sum, one final rounding
    lo = (q.float()[:, :, None, :] * mm.float()[None, :, :, 0, :]).bfloat16().float()
    hi = (q.float()[:, :, None, :] * mm.float()[None, :, :, 1, :]).bfloat16().float()
    want = torch.maximum(lo, hi).sum(-1).bfloat16()
    assert torch.equal(got, want)
    # symmetric in (min, max)
    assert torch.equal(got, O.max_ip(q, mm.flip(2)))


# ---------------------------------------------------------------- top-k
def brute_topk(row, k):
    idx = list(range(len(row)))
    idx.sort(key=lambda i: (-row[i], i))
    return idx[:k]


def test_top_k_pages_brute_force_with_ties():
    g = torch.Generator().manual_seed(7)
    s = torch.randint(0, 4, (3, 2, 11), generator=g).float()  # heavy ties
    got = O.top_k_pages(s, 5)
    for a, b in itertools.product(range(3), range(2)):
        assert got[a, b].tolist() == brute_topk(s[a, b].tolist(), 5)


def test_select_pages_layout():
    # row s*rep + r of the score matrix is query head h*rep + r of token s
    seq, rep, H, P, k = 2, 3, 2, 9, 4
    g = torch.Generator().manual_seed(8)
    rows = torch.randn(seq * rep, H, P, generator=g)
    sel = O.select_pages(rows, seq, rep, k)
    assert sel.shape == (seq, H, rep, k)
    for s, h, r in itertools.product(range(seq), range(H), range(rep)):
        assert sel[s, h, r].tolist() == brute_topk(rows[s * rep + r, h].tolist(), k)
    flat = O.lru_index_list(sel)
    assert flat.shape == (H, seq * rep * k)
    assert flat[1, :k].tolist() == sel[0, 1, 0].tolist()
    assert flat[1, (1 * rep + 2) * k:(1 * rep + 3) * k].tolist() == sel[1, 1, 2].tolist()


# ---------------------------------------------------------------- LRU
@pytest.mark.parametrize("name", sorted(lru_kats.CASES))
def test_lru_load_reference_kats(name):
    case = lru_kats.CASES[name]
    H, P, N, PD = (lru_kats.NUM_HEADS, lru_kats.NUM_DRAM_PAGES, lru_kats.NUM_HBM_PAGES,
                   lru_kats.PAGE_DIM)
    rng = np.random.default_rng(0)
    dram = rng.standard_normal((H, P, PD)).astype(np.float32)
    hbm = np.zeros((H, N, PD), dtype=np.float32)
    st = O.LruState(np.tile(np.arange(N, dtype=np.int32), (H, 1)),
                    np.array(case["d2h"], dtype=np.int32), np.array(case["h2d"], dtype=np.int32))
    for h in range(H):  # a full cache starts with its pages loaded
        for s, p in enumerate(st.h2d[h]):
            if p >= 0:
                hbm[h, s] = dram[h, p]
    O.lru_load(st, np.array(case["topk"]), lru_kats.STEP, dram, hbm)
    for (h, s), t in case["time"].items():
        assert st.time[h, s] == t
    for (h, p), s in case["d2h_after"].items():
        assert st.d2h[h, p] == s
    for (h, s), p in case["h2d_after"].items():
        assert st.h2d[h, s] == p
    for h, s, p in case["payload"]:
        assert np.array_equal(hbm[h, s], dram[h, p])


def test_lru_geometry_numbers():
    geo = lru_kats.GEOMETRY
    P = geo["tokens"] // geo["page_size"]
    assert P == geo["dram_pages"]
    assert O.hbm_page_count(P, geo["page_size"], None) == geo["default_hbm_pages"]
    assert O.hbm_page_count(P, geo["page_size"], 1024) == geo["hbm_pages_for_1024_tokens"]
    st = O.LruState.initial(4, P, 102)
    assert np.array_equal(st.d2h[:, -102:], np.tile(np.arange(102), (4, 1)))
    assert np.all(st.d2h[:, :-102] == -1)
    assert np.array_equal(st.h2d[0], np.arange(P - 102, P))


def test_lru_hand_walked_trace():
    # 1 head, 6 pages, 3 slots holding pages 3,4,5 (times 0).
    st = O.LruState.initial(1, 6, 3)
    # step 1: [4, 0, 4, 1]: 4 hits (slot 1); 0 and 1 miss -> untouched slots in
    # (time, slot) order: slot 0 then slot 2; the repeat of 4 is a hit.
    hit, miss = O.lru_load(st, np.array([[4, 0, 4, 1]]), 1)
    assert hit.tolist() == [[True, False, True, False]]
    assert miss == [[(0, 0), (1, 2)]]
    assert st.h2d.tolist() == [[0, 4, 1]] and st.d2h.tolist() == [[0, 2, -1, -1, 1, -1]]
    assert st.time.tolist() == [[1, 1, 1]]
    # step 2: [5]: miss; all times equal 1 -> lowest slot (0) is the victim
    hit, miss = O.lru_load(st, np.array([[5]]), 2)
    assert miss == [[(5, 0)]] and st.d2h.tolist() == [[-1, 2, -1, -1, 1, 0]]
    # step 3: [4]: hit only; step 4: [0, 2]: victims are the oldest slots: 2 (t=1), then 0 (t=2)
    O.lru_load(st, np.array([[4]]), 3)
    hit, miss = O.lru_load(st, np.array([[0, 2]]), 4)
    assert miss == [[(0, 2), (2, 0)]]
    assert st.h2d.tolist() == [[2, 4, 0]]


def test_lru_invariants_random_trace():
    rng = np.random.default_rng(3)
    H, P, N, K = 3, 40, 12, 12
    dram = rng.integers(0, 1 << 15, (H, P, 4)).astype(np.int16)
    st = O.LruState.initial(H, P, N)
    hbm = dram[:, P - N:].copy()
    for step in range(1, 30):
        idx = rng.integers(0, P, (H, K))
        O.lru_load(st, idx, step, dram, hbm)
        for h in range(H):
            assert len(set(st.h2d[h])) == N                       # injective
            assert np.array_equal(st.d2h[h, st.h2d[h]], np.arange(N))
            assert np.all(st.d2h[h, idx[h]] >= 0)                 # every request resident
            assert np.array_equal(hbm[h], dram[h, st.h2d[h]])      # payload follows the map
            assert (st.d2h[h] >= 0).sum() == N


def test_lru_wraps_when_requests_exceed_slots():
    # K > N_hbm: the eviction pointer wraps and can evict a page loaded in the same call
    st = O.LruState.initial(1, 8, 2)           # slots hold pages 6, 7
    hit, miss = O.lru_load(st, np.array([[0, 1, 2]]), 1)
    assert miss == [[(0, 0), (1, 1), (2, 0)]]  # third miss reuses slot 0
    assert st.h2d.tolist() == [[2, 1]] and st.d2h[0, 0] == -1


# ---------------------------------------------------------------- attention
def test_attention_partial_matches_dense_fp64():
    g = torch.Generator().manual_seed(9)
    Hq, Hkv, T, D = 4, 2, 37, 8
    q = torch.randn(Hq, D, generator=g)
    k = torch.randn(Hkv, T, D, generator=g)
    v = torch.randn(Hkv, T, D, generator=g)
    out, lse = O.attention_partial(q, k, v)
    for j in range(Hq):
        h = j // 2
        s = (k[h].double() @ q[j].double()) / math.sqrt(D)
        p = torch.softmax(s, 0)
        assert torch.allclose(out[j].double(), p @ v[h].double(), atol=1e-6)
        assert lse[j].item() == pytest.approx(torch.logsumexp(s, 0).item(), abs=1e-5)


def test_combine_equals_attention_over_concatenation():
    g = torch.Generator().manual_seed(10)
    Hq, Hkv, D = 4, 2, 8
    q = torch.randn(Hq, D, generator=g)
    k = torch.randn(Hkv, 50, D, generator=g)
    v = torch.randn(Hkv, 50, D, generator=g)
    full, _ = O.attention_partial(q, k, v)
    a = O.attention_partial(q, k[:, :19], v[:, :19])
    b = O.attention_partial(q, k[:, 19:], v[:, 19:])
    assert torch.allclose(O.combine(a[0], a[1], b[0], b[1], torch.float32), full, atol=1e-6)


def test_page_layout_round_trip():
    g = torch.Generator().manual_seed(11)
    k = torch.randn(2, 32, 4, generator=g)
    v = torch.randn(2, 32, 4, generator=g)
    pages = O.pack_pages(k, v, 8)
    assert pages.shape == (2, 4, 8 * 2 * 4)
    # token t of a page: K at t*2*D, V at t*2*D + D
    assert torch.equal(pages[1, 2, 3 * 8:3 * 8 + 4], k[1, 2 * 8 + 3])
    assert torch.equal(pages[1, 2, 3 * 8 + 4:3 * 8 + 8], v[1, 2 * 8 + 3])
    kk, vv = O.split_hbm_pages(pages, 8, 4)
    assert torch.equal(kk, k) and torch.equal(vv, v)


def test_decode_oracle_geometry_and_full_attention_equivalence():
    # prefix small enough for the static path: generate == dense attention over everything
    assert O.dram_split(66 * 1024, 4096 + 512, 16) == 66 * 1024 - 4608 + 16
    g = torch.Generator().manual_seed(12)
    Hq, Hkv, D, S = 4, 2, 8, 96
    o = O.DecodeOracle(8, 128, 32, 16, 32, Hkv, D, dtype=torch.float32, round_partials=False)
    k = torch.randn(1, S, Hkv, D, generator=g)
    v = torch.randn(1, S, Hkv, D, generator=g)
    o.init_cache(k, v)
    assert o.dram_kv_cache_size == 80 and not o.uses_lru      # 80 <= 128: static cache
    xq = torch.randn(1, 1, Hq, D, generator=g)
    xk = torch.randn(1, 1, Hkv, D, generator=g)
    xv = torch.randn(1, 1, Hkv, D, generator=g)
    out = o.generate(xq, xk, xv, S)
    kk = torch.cat([k[0], xk[0]], 0).transpose(0, 1)
    vv = torch.cat([v[0], xv[0]], 0).transpose(0, 1)
    want, _ = O.attention_partial(xq[0, 0], kk, vv)
    assert torch.allclose(out[0, 0], want, atol=1e-5)


def test_decode_oracle_lru_path_attends_over_all_resident_slots():
    g = torch.Generator().manual_seed(13)
    Hq, Hkv, D, S, page = 4, 2, 8, 176, 16
    o = O.DecodeOracle(8, 64, 32, page, 32, Hkv, D, dtype=torch.float32, round_partials=False)
    k = torch.randn(1, S, Hkv, D, generator=g)
    v = torch.randn(1, S, Hkv, D, generator=g)
    o.init_cache(k, v)
    assert o.dram_kv_cache_size == 160 and o.uses_lru and o.kp == 2
    assert o.state.h2d.tolist() == [[6, 7, 8, 9]] * 2       # last 4 of 10 pages resident
    for step in range(3):
        xq = torch.randn(1, 1, Hq, D, generator=g)
        xk = torch.randn(1, 1, Hkv, D, generator=g)
        xv = torch.randn(1, 1, Hkv, D, generator=g)
        out = o.generate(xq, xk, xv, S + step)
        assert o.last_idx.shape == (Hkv, 2 * 2)
        # dense attention over exactly: tokens of resident pages ++ local window ++ new tokens
        c = S + step - 160
        for j in range(Hq):
            h = j // 2
            toks = [p * page + t for p in o.state.h2d[h] for t in range(page)]
            kk = torch.cat([k[0, toks, h], o.cache_k[: c + 1, h]], 0).double()
            vv = torch.cat([v[0, toks, h], o.cache_v[: c + 1, h]], 0).double()
            p_ = torch.softmax(kk @ xq[0, 0, j].double() / math.sqrt(D), 0)
            assert torch.allclose(out[0, 0, j].double(), p_ @ vv, atol=1e-5)
        assert o.state.step == step + 1


def test_lru_load_when_the_step_ties_with_stored_times():
    """Hand-walked case (tests/golden/lru_kats.py STAMP_TIES): a slot hit by the touch pass
    is still first in the eviction order when the caller's step equals the stored times,
    so the walk evicts it and pages the same page in again later."""
    import numpy as np
    from tests.golden import lru_kats

    c = lru_kats.STAMP_TIES
    st = O.LruState(np.array(c["time"], dtype=np.float32), np.array(c["d2h"], dtype=np.int64),
                    np.array(c["h2d"], dtype=np.int64), c["step"])
    dram = np.arange(6 * 4, dtype=np.float32).reshape(1, 6, 4)
    hbm = dram[:, 3:6].copy()
    hit, misses = O.lru_load(st, np.array(c["topk"]), c["step"], dram, hbm)
    assert st.d2h.tolist() == c["d2h_after"] and st.h2d.tolist() == c["h2d_after"]
    assert st.time.tolist() == c["time_after"]
    assert hit.tolist() == c["hit"] and [list(m) for m in misses] == c["misses"]
    assert np.array_equal(hbm[0], dram[0, [0, 1, 3]])
