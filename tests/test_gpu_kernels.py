"""Parity of every HIP kernel (called through the C ABI) against the CPU oracle."""

import math

import numpy as np
import pytest
import torch

from oracle import dram_attention_oracle as O
from tests.golden import lru_kats

from tests.util import close, same

pytestmark = pytest.mark.gpu

DEV = "cuda"


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ page min/max
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,P,page,D", [(2, 5, 16, 64), (8, 33, 16, 128), (3, 7, 4, 24),
                                        (2, 9, 8, 5), (1, 1, 1, 1)])
def test_page_minmax_exact(dtype, H, P, page, D):
    from dram_attention_amd.topk_selector import page_min_max

    k = torch.randn(H, P * page, D, generator=gen(1)).to(dtype)
    got = page_min_max(k.to(DEV), P)
    assert same(got.cpu(), O.page_min_max(k, P))
    # the layout init_cache hands over: a (S, H, D) tensor viewed as (H, S, D)
    kt = k.transpose(0, 1).contiguous().to(DEV).transpose(0, 1)
    assert not kt.is_contiguous() or H == 1 or P * page == 1
    assert same(page_min_max(kt, P).cpu(), O.page_min_max(k, P))


def test_page_minmax_nan_propagates():
    from dram_attention_amd.topk_selector import page_min_max

    k = torch.randn(1, 32, 8, generator=gen(2))
    k[0, 5, 3] = float("nan")
    got = page_min_max(k.to(DEV), 2).cpu()
    assert torch.isnan(got[0, 0, :, 3]).all() and not torch.isnan(got[0, 1]).any()
    assert not torch.isnan(got[0, 0, :, :3]).any()


# ------------------------------------------------------------------ scorer
def test_max_inner_product_reference_cases():
    """The five cases of the reference's max_ip_triton_kernel_test.py."""
    from dram_attention_amd import max_inner_product, max_ip_ref

    q = torch.randn(2, 4, 64, generator=gen(3))
    mm = torch.randn(4, 16, 2, 64, generator=gen(4))
    out = max_inner_product(q.to(DEV), mm.to(DEV))
    assert out.shape == (2, 4, 16) and out.dtype == torch.float32
    assert close(out.cpu(), O.max_ip(q, mm), 1e-3, 1e-3)   # :29-38 tolerance
    assert close(out, max_ip_ref(q.to(DEV), mm.to(DEV)), 1e-3, 1e-3)
    out16 = max_inner_product(q.half().to(DEV), mm.half().to(DEV))
    assert out16.dtype == torch.float16
    q1, mm1 = torch.randn(1, 1, 1, generator=gen(5)), torch.randn(1, 1, 2, 1, generator=gen(6))
    o1 = max_inner_product(q1.to(DEV), mm1.to(DEV))
    assert o1.shape == (1, 1, 1)
    assert o1.item() == pytest.approx(max(q1.item() * mm1[0, 0, 0, 0].item(),
                                          q1.item() * mm1[0, 0, 1, 0].item()), rel=1e-6)
    qL = torch.randn(32, 32, 128, generator=gen(7))
    mmL = torch.randn(32, 1024, 2, 128, generator=gen(8))
    oL = max_inner_product(qL.to(DEV), mmL.to(DEV))
    assert oL.shape == (32, 32, 1024)
    assert close(oL.cpu(), O.max_ip(qL, mmL), 1e-3, 1e-3)


@pytest.mark.parametrize("N,H,D,L", [(4, 8, 128, 515), (8, 2, 64, 130), (1, 3, 128, 4),
                                     (5, 2, 40, 37), (3, 2, 256, 9)])
def test_page_score_bf16_matches_reference_rounding(N, H, D, L):
    from dram_attention_amd import max_inner_product

    q = torch.randn(N, H, D, generator=gen(9)).bfloat16()
    mm = torch.randn(H, L, 2, D, generator=gen(10)).bfloat16()
    got = max_inner_product(q.to(DEV), mm.to(DEV)).cpu()
    want = O.max_ip(q, mm)
    assert got.dtype == torch.bfloat16
    # same rounding points; fp32 summation order differs, so a sum that lands on a
    # bf16 rounding boundary may fall to the neighbouring value: at most one ulp, rarely
    diff = (got.float() - want.float()).abs()
    ulp = want.float().abs() * 2.0 ** -7
    assert torch.all(diff <= ulp + 1e-30)
    assert (diff > 0).float().mean().item() < 0.02


def test_page_score_strided_query_view():
    """The (rep, Hkv, D) view of one token's query heads: strides (D, rep*D, 1)."""
    from dram_attention_amd.max_ip_kernel import page_scores

    Hkv, rep, D, L = 8, 4, 128, 300
    q = torch.randn(1, 1, Hkv * rep, D, generator=gen(11)).bfloat16()
    mm = torch.randn(Hkv, L, 2, D, generator=gen(12)).bfloat16()
    qd = q.to(DEV)
    qv = qd[0, 0].view(Hkv, rep, D).transpose(0, 1)
    out = torch.empty(rep, Hkv, L, dtype=torch.float32, device=DEV)
    page_scores(qv, mm.to(DEV), out, round_to_input=True)
    want = O.scores_for_selection(q, mm)
    diff = (out.cpu() - want).abs()
    assert torch.all(diff <= want.abs() * 2.0 ** -7)
    # fp32 output holds bf16-representable values
    assert same(out.cpu(), out.cpu().bfloat16().float())


def test_page_score_fp16_follows_the_bf16_scheme():
    """fp16 inputs: products rounded to fp16, fp32 maximum and sum, one rounding at the
    end (the oracle's statement).  The reference's Triton kernel would accumulate in
    fp16 in an order of its own, which nothing here can reproduce (parity unpinned,
    its test checks the dtype only): this documents the deviation and bounds it by
    the error of an fp16 accumulation."""
    from dram_attention_amd import max_inner_product

    N, H, D, L = 4, 2, 128, 300
    q = torch.randn(N, H, D, generator=gen(31)).half()
    mm = torch.randn(H, L, 2, D, generator=gen(32)).half()
    got = max_inner_product(q.to(DEV), mm.to(DEV)).cpu()
    assert got.dtype == torch.float16
    want = O.max_ip(q, mm)
    diff = (got.float() - want.float()).abs()
    assert torch.all(diff <= want.float().abs() * 2.0 ** -10 + 1e-30)      # one fp16 step, rarely
    assert (diff > 0).float().mean().item() < 0.02
    # a sequential fp16 accumulation of the same rounded terms differs by far more
    terms = torch.maximum(q[:, :, None, :] * mm[None, :, :, 0, :], q[:, :, None, :] * mm[None, :, :, 1, :])
    acc = torch.zeros(N, H, L, dtype=torch.float16)
    for d in range(D):
        acc = acc + terms[..., d]
    assert (acc.float() - want.float()).abs().max() > diff.max()


def ordered_summaries(H, L, D, seed):
    """Random (H, L, 2, D) bf16 summaries with min <= max in every channel."""
    a = torch.randn(H, L, 2, D, generator=gen(seed)).bfloat16()
    return torch.stack((torch.minimum(a[:, :, 0], a[:, :, 1]), torch.maximum(a[:, :, 0], a[:, :, 1])), dim=2)


def check_scores(got, want, changed_frac=0.02):
    """Same rounding points as the oracle; the fp32 summation order differs, so a sum
    on a bf16 rounding boundary may land on the neighbouring value: one step, rarely."""
    got, want = got.float().cpu(), want.float()
    diff = (got - want).abs()
    assert torch.all(diff <= want.abs() * 2.0 ** -7 + 1e-30)
    assert (diff > 0).float().mean().item() < changed_frac


@pytest.mark.parametrize("N,H,D,L", [
    (4, 8, 128, 8192),      # the decode shape of the 128K workload: one round of 8 steps
    (8, 8, 128, 3000),      # 8 query rows, ragged page count
    (4, 2, 128, 70001),     # several rounds per wave, odd length
    (8, 3, 128, 40000),     # 8 rows, several rounds
    (4, 8, 64, 2048), (8, 2, 64, 777), (4, 4, 32, 515), (8, 1, 32, 4096),
    (1, 1, 128, 1), (3, 2, 128, 5), (5, 2, 128, 33), (12, 2, 128, 130), (4, 8, 128, 2048),
])
def test_page_score_ordered_bounds_matches_oracle(N, H, D, L):
    """The decode step's scorer (bf16 summaries with min <= max, fp32 output): bound picked
    by the sign of q, products by packed dot instructions, sum over D on the matrix cores."""
    from dram_attention_amd.max_ip_kernel import page_scores

    q = torch.randn(N, H, D, generator=gen(N * 1000 + L)).bfloat16()
    mm = ordered_summaries(H, L, D, seed=L + D)
    for rounded in (True, False):
        out = torch.full((N, H, L), float("nan"), dtype=torch.float32, device=DEV)
        page_scores(q.to(DEV), mm.to(DEV), out, round_to_input=rounded, ordered_bounds=True)
        if rounded:
            check_scores(out, O.max_ip(q, mm))
            assert same(out.cpu(), out.cpu().bfloat16().float())
        else:
            # unrounded sums: against the plain kernel (both products, max, vector sum)
            plain = torch.empty_like(out)
            page_scores(q.to(DEV), mm.to(DEV), plain, round_to_input=False, ordered_bounds=False)
            terms = (q.float()[:, :, None, None, :] * mm.float()[None]).abs().amax(dim=3).sum(-1)
            assert torch.all((out - plain).abs().cpu() <= 1e-6 * terms + 1e-30)


def test_page_score_ordered_bounds_special_values():
    """Signed zeros and denormal-range products in the query, and non-finite bounds: a
    page with an infinite or NaN bound scores as the reference kernel's formula says
    (+-inf, NaN, or, where a zero query channel meets an infinite bound, the other
    product: tl.maximum drops a NaN operand), and leaves its neighbours alone."""
    from dram_attention_amd.max_ip_kernel import page_scores

    N, H, D, L = 4, 2, 128, 200
    q = torch.randn(N, H, D, generator=gen(70)).bfloat16()
    q[0, 0, :8] = 0.0
    q[1, 0, :8] = -0.0
    q[2, 1, 5] = 1e-30
    mm = ordered_summaries(H, L, D, seed=71)
    inf = float("inf")
    mm[0, 3, 1, 7] = inf                       # max = +inf
    mm[0, 4, 0, 9] = -inf                      # min = -inf
    mm[1, 5, :, 11] = float("nan")             # NaN in both bounds (what aminmax gives)
    mm[1, 6, 0, 2], mm[1, 6, 1, 2] = -inf, inf
    mm[1, 7, :, 0] = 1e-38                     # tiny bounds
    out = torch.empty(N, H, L, dtype=torch.float32, device=DEV)
    page_scores(q.to(DEV), mm.to(DEV), out, round_to_input=True, ordered_bounds=True)
    want = O.max_ip(q, mm).float()
    got = out.cpu()
    special = torch.zeros(H, L, dtype=torch.bool)
    for h, l in ((0, 3), (0, 4), (1, 5), (1, 6)):
        special[h, l] = True
    assert same(got[:, special], want[:, special])          # inf / NaN exactly as the formula
    assert not torch.isfinite(want[:, special]).all()
    assert torch.isfinite(want[:2, 0, 3]).all()             # zero query channel x infinite bound
    # the plain kernel (both products, fmax) agrees entry for entry on where they are finite
    plain = torch.empty_like(out)
    page_scores(q.to(DEV), mm.to(DEV), plain, round_to_input=True, ordered_bounds=False)
    assert same(torch.isfinite(plain.cpu()), torch.isfinite(got))
    assert same(torch.isnan(plain.cpu()), torch.isnan(got))
    check_scores(got[:, ~special], want[:, ~special])


def test_page_score_ordered_bounds_strided_query_view():
    from dram_attention_amd.max_ip_kernel import page_scores

    for Hkv, rep, D, L in ((8, 4, 128, 8192), (8, 8, 128, 4100), (2, 4, 64, 300)):
        q = torch.randn(1, 1, Hkv * rep, D, generator=gen(21 + rep)).bfloat16()
        mm = ordered_summaries(Hkv, L, D, seed=22)
        qv = q.to(DEV)[0, 0].view(Hkv, rep, D).transpose(0, 1)
        out = torch.empty(rep, Hkv, L, dtype=torch.float32, device=DEV)
        page_scores(qv, mm.to(DEV), out, round_to_input=True, ordered_bounds=True)
        check_scores(out, O.scores_for_selection(q, mm))


# ------------------------------------------------------------------ top-k
def run_topk(scores, rep, k, one_launch=False):
    """one_launch: no candidate buffer, so rows longer than 16384 pages take the
    single-workgroup walk instead of the two-launch selection."""
    from dram_attention_amd.topk_selector import topk_pages

    n_rows, H, L = scores.shape
    seq = n_rows // rep
    out = torch.empty(seq, H, rep, k, dtype=torch.int64, device=DEV)
    ws = torch.empty(0, dtype=torch.uint8, device=DEV) if one_launch else None
    topk_pages(scores.to(DEV), rep, k, out, H * rep * k, rep * k, k, workspace=ws)
    return out.cpu()


@pytest.mark.parametrize("rows,rep,H,L,k", [(4, 4, 8, 8192, 256), (2, 2, 2, 512, 32),
                                            (3, 1, 2, 1000, 1000), (6, 3, 1, 77, 5),
                                            (1, 1, 1, 1, 1), (2, 1, 2, 5000, 1),
                                            (8, 8, 2, 20000, 512), (1, 1, 1, 300, 299),
                                            (2, 1, 1, 65536, 8192), (8, 8, 1, 65536, 512),
                                            (1, 1, 1, 16385, 600), (2, 2, 1, 16390, 8190),
                                            (1, 1, 2, 300000, 64), (1, 1, 1, 40000, 30000)])
def test_topk_pages_exact(rows, rep, H, L, k):
    """Rows beyond 16384 pages go through the two-launch selection (parts, then
    candidates) where the parts can each hold k pages, and through one workgroup
    per row otherwise or without a candidate buffer: all against the stable sort."""
    from dram_attention_amd import _lib

    scores = torch.randn(rows, H, L, generator=gen(13))
    want = O.select_pages(scores, rows // rep, rep, k)
    if k <= 8192:
        assert same(run_topk(scores, rep, k), want)
        assert same(run_topk(scores, rep, k, one_launch=True), want)
    split = _lib.load().da_topk_pages_workspace_bytes(rows, H, L, k) > 0
    assert split == ((rows, rep, H, L, k) in [(8, 8, 2, 20000, 512), (2, 1, 1, 65536, 8192),
                                              (8, 8, 1, 65536, 512), (1, 1, 1, 16385, 600),
                                              (2, 2, 1, 16390, 8190), (1, 1, 2, 300000, 64)])
    if k > 8192:
        with pytest.raises(RuntimeError, match="survivors"):
            run_topk(scores, rep, k)


def test_topk_pages_long_rows_with_ties_across_parts():
    """Few distinct values over rows of 50 000 pages: the winners of equal score must be
    the lowest page numbers whichever part they lie in, also when one part alone could
    fill the list."""
    scores = torch.randint(0, 3, (2, 2, 50000), generator=gen(17)).float()
    scores[0, 0, 30000:] = 5.0          # one part holds more than k pages of the top value
    scores[1, 1, :] = -2.0              # a constant row: pages 0..k-1
    for k in (700, 8192):
        want = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :k]
        got = run_topk(scores, 2, k)
        assert same(got[0], want.transpose(0, 1)), k
        assert same(run_topk(scores, 2, k, one_launch=True), got), k


def test_topk_pages_bf16_rounded_scores_at_1m_row_length():
    """65 536 pages per row with scores that share their low 16 bits (rounded to
    bf16, as the selector produces them): many exact ties, lowest index first."""
    scores = (torch.randn(4, 2, 65536, generator=gen(15)) * 8).bfloat16().float()
    got = run_topk(scores, 4, 512)
    want = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :512]
    assert same(got[0], want.transpose(0, 1))


@pytest.mark.parametrize("L,k", [(1000, 1000), (5000, 5000), (8192, 8192), (700, 513), (9000, 1025),
                                 (16384, 4096), (3000, 2999), (64, 64), (1, 1)])
@pytest.mark.parametrize("kind", ["normal", "rounded", "levels", "steps"])
def test_topk_pages_long_lists_and_complete_orderings(L, k, kind):
    """More than 512 winners are ordered by the stable radix sort of the survivors, and
    k == L (a complete ordering) skips the selection: random fp32 scores (all four
    digits differ), scores rounded to bf16 with both signs, a handful of levels (ties
    by lowest page everywhere) and small whole numbers as the LRU's time stamps are."""
    g = gen(100 + L + k)
    if kind == "normal":
        scores = torch.randn(2, 2, L, generator=g)
    elif kind == "rounded":
        scores = (torch.randn(2, 2, L, generator=g) * 8).bfloat16().float()
    elif kind == "levels":
        scores = torch.randint(-3, 4, (2, 2, L), generator=g).float()
    else:
        scores = -torch.randint(0, 300, (2, 2, L), generator=g).float()
    want = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :k]
    assert same(run_topk(scores, 2, k)[0], want.transpose(0, 1))


@pytest.mark.parametrize("k", [1, 37, 256, 700])
@pytest.mark.parametrize("family", ["byte0", "byte1", "byte2", "byte3", "bytes12", "bits_10_21",
                                    "signs_and_byte2", "signs_and_byte0", "rounded_both_signs",
                                    "all_equal", "two_values", "bits_13_23", "sign_and_bits_20_22",
                                    "negative_low_bits", "negative_bits_6_17"])
def test_topk_pages_keys_that_differ_in_few_bits(family, k):
    """The selection skips every digit in which no two keys differ and orders its winners on
    the 16 bits that do when they fit a window: float scores built from bit patterns that
    differ in one byte, in two, across a byte boundary, in the sign plus one byte, all
    against the stable sort (values stay finite: exponent bits come from 0x3f.. or 0x40..)."""
    g = gen(sum(map(ord, family)) + k)
    L = 3000
    r = lambda hi: torch.randint(0, hi, (2, 2, L), generator=g, dtype=torch.int64)
    base = 0x40490000
    bits = {
        "byte0": base | r(256), "byte1": base | (r(256) << 8), "byte2": 0x40000000 | (r(128) << 16),
        "byte3": (0x3f + r(3)) << 24 | 0x00400000, "bytes12": 0x40000000 | (r(65536) << 8) & 0x007fff00,
        "bits_10_21": 0x40000000 | (r(4096) << 10),
        "signs_and_byte2": (r(2) << 31) | 0x40000000 | (r(128) << 16),
        "signs_and_byte0": (r(2) << 31) | base | r(256),
        "rounded_both_signs": (r(2) << 31) | 0x3f000000 | (r(512) << 16),
        "all_equal": torch.full((2, 2, L), base, dtype=torch.int64),
        "two_values": base + 0x101 * r(2),
        "bits_13_23": 0x40000000 | (r(2048) << 13),                       # one pass over 11 bits
        "sign_and_bits_20_22": (r(2) << 31) | ((0x3f0 + r(8)) << 20),     # 12 bits up to the sign
        "negative_low_bits": 0xC0490000 | (r(512) << 4),                  # complemented low half
        "negative_bits_6_17": 0xC0400000 | (r(4096) << 6),                # window across both halves
    }[family]
    scores = torch.from_numpy((bits & 0xffffffff).numpy().astype(np.uint32).view(np.float32))
    assert torch.isfinite(scores).all()
    want = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :k]
    assert same(run_topk(scores, 2, k)[0], want.transpose(0, 1))


@pytest.mark.parametrize("ttype", [torch.float32, torch.int32])
@pytest.mark.parametrize("lo,hi", [(0, 40), (4600, 5000), (60000, 70000), (16777000, 16777216),
                                   (255, 258), (1000, 1001)])
def test_lru_candidates_at_late_steps(lo, hi, ttype):
    """Access times of a long decoding run (large step counts, a narrow window of them):
    the short list of least recent slots is still the head of the stable order."""
    from dram_attention_amd.lru_kernel import LruScratch, candidate_list, lru_candidates

    H, N, kc = 2, 2048, 256
    time = torch.randint(lo, hi, (H, N), generator=gen(lo + hi)).to(ttype)
    sc = LruScratch.allocate(H, 16, DEV, N)._replace(candidates=candidate_list(H, kc, DEV))
    step = torch.tensor([hi], dtype=torch.int32, device=DEV)
    got = lru_candidates(time.to(DEV), sc, step).cpu().long()
    assert same(got, torch.sort(time, dim=-1, stable=True).indices[:, :kc])


@pytest.mark.parametrize("ttype", [torch.float32, torch.int32])
@pytest.mark.parametrize("N,kc", [(4096, 4096), (2048, 2048), (4096, 1500), (600, 600), (5000, 256)])
def test_lru_candidates_are_the_stable_order_of_the_access_times(N, kc, ttype):
    """The candidate list is the head of argsort(access_time, stable=True), up to the
    complete order of all slots."""
    from dram_attention_amd.lru_kernel import LruScratch, candidate_list, lru_candidates

    H = 3
    time = torch.randint(0, 900, (H, N), generator=gen(N + kc)).to(ttype)
    time[1] = 7                                  # one head with every slot tied
    sc = LruScratch.allocate(H, 16, DEV, N)._replace(candidates=candidate_list(H, kc, DEV))
    step = torch.tensor([901], dtype=torch.int32, device=DEV)
    cand = lru_candidates(time.to(DEV), sc, step)
    got = cand.cpu().long()
    want = torch.sort(time, dim=-1, stable=True).indices[:, :kc]
    assert same(got, want)
    # every head's list carries the step counter's value as its stamp, behind the lists
    stamps = torch.as_strided(cand, (H,), (1,), cand.storage_offset() + H * kc)
    assert stamps.cpu().tolist() == [901] * H


def test_empty_inputs_are_no_ops():
    """Zero rows, zero pages, zero requests: every entry point returns without a launch."""
    from dram_attention_amd import max_inner_product
    from dram_attention_amd.lru_kernel import LruScratch, lru_update_and_gather

    assert max_inner_product(torch.zeros(0, 2, 64, device=DEV), torch.zeros(2, 8, 2, 64, device=DEV)).shape == (0, 2, 8)
    assert max_inner_product(torch.zeros(3, 2, 64, device=DEV), torch.zeros(2, 0, 2, 64, device=DEV)).shape == (3, 2, 0)
    H, P, N = 2, 8, 4
    dram = torch.randn(H, P, 32, device=DEV)
    hbm = dram[:, P - N:].clone()
    time = torch.zeros(H, N, device=DEV)
    d2h = torch.full((H, P), -1, dtype=torch.int64, device=DEV)
    d2h[:, P - N:] = torch.arange(N, device=DEV)
    h2d = torch.arange(P - N, P, device=DEV).repeat(H, 1)
    step = torch.zeros(1, dtype=torch.int32, device=DEV)
    before = (hbm.clone(), d2h.clone(), h2d.clone())
    lru_update_and_gather(dram, time, d2h, h2d, torch.zeros(H, 0, dtype=torch.int64, device=DEV), step,
                          hbm, LruScratch.allocate(H, 0, DEV), bump_step=True)
    torch.cuda.synchronize()
    assert step.item() == 1 and same(hbm, before[0]) and same(d2h, before[1]) and same(h2d, before[2])


@pytest.mark.parametrize("levels", [2, 7, 200])
def test_topk_pages_ties_lowest_index_first(levels):
    scores = torch.randint(0, levels, (4, 4, 4096), generator=gen(14)).float() - levels / 2
    got = run_topk(scores, 4, 256)
    assert same(got, O.select_pages(scores, 1, 4, 256))
    # bf16-rounded scores, the production case
    s2 = (torch.randn(4, 8, 8192, generator=gen(15)) * 20).bfloat16().float()
    assert same(run_topk(s2, 4, 256), O.select_pages(s2, 1, 4, 256))


def test_topk_pages_special_values():
    s = torch.randn(2, 1, 600, generator=gen(16))
    s[0, 0, 10] = float("inf")
    s[0, 0, 20] = -float("inf")
    s[0, 0, 30] = 0.0
    s[0, 0, 31] = -0.0
    s[1, 0, :] = 1.5                      # one constant row: indices 0..k-1
    s[1, 0, 100] = float("nan")           # torch ranks NaN first when descending
    got = run_topk(s, 1, 300)
    want = O.select_pages(s, 2, 1, 300)
    assert same(got, want)
    assert got[1, 0, 0, 0].item() == 100 and got[1, 0, 0, 1:5].tolist() == [0, 1, 2, 3]


def test_topk_for_lru_layout():
    from dram_attention_amd.topk_selector import topk_pages

    seq, rep, H, L, k = 3, 2, 4, 200, 6
    scores = torch.randn(seq * rep, H, L, generator=gen(17))
    out = torch.empty(H, seq * rep * k, dtype=torch.int64, device=DEV)
    topk_pages(scores.to(DEV), rep, k, out, rep * k, seq * rep * k, k)
    want = O.lru_index_list(O.select_pages(scores, seq, rep, k))
    assert same(out.cpu(), want)
    out32 = torch.empty(H, seq * rep * k, dtype=torch.int32, device=DEV)
    topk_pages(scores.to(DEV), rep, k, out32, rep * k, seq * rep * k, k)
    assert same(out32.cpu().long(), want)


# ------------------------------------------------------------------ LRU
@pytest.mark.parametrize("name", sorted(lru_kats.CASES))
def test_load_lru_cache_reference_kats(name):
    from dram_attention_amd import load_lru_cache_

    case = lru_kats.CASES[name]
    H, P, N, PD = (lru_kats.NUM_HEADS, lru_kats.NUM_DRAM_PAGES, lru_kats.NUM_HBM_PAGES,
                   lru_kats.PAGE_DIM)
    dram = torch.randn(H, P, PD, generator=gen(18)).to(DEV)
    hbm = torch.zeros(H, N, PD, device=DEV)
    time = torch.arange(N, dtype=torch.int32, device=DEV).repeat(H, 1)
    d2h = torch.tensor(case["d2h"], dtype=torch.int32, device=DEV)
    h2d = torch.tensor(case["h2d"], dtype=torch.int32, device=DEV)
    for h in range(H):
        for s, p in enumerate(case["h2d"][h]):
            if p >= 0:
                hbm[h, s] = dram[h, p]
    topk = torch.tensor(case["topk"], dtype=torch.int32, device=DEV)
    step = torch.tensor([lru_kats.STEP], dtype=torch.int32, device=DEV)
    load_lru_cache_(dram_kv_cache=dram, page_access_time=time,
                    dram_page_to_hbm_page_mapping=d2h, hbm_page_to_dram_page_mapping=h2d,
                    topk_dram_page_index=topk, current_step=step, hbm_kv_cache=hbm)
    for (h, s), t in case["time"].items():
        assert time[h, s].item() == t
    for (h, p), s in case["d2h_after"].items():
        assert d2h[h, p].item() == s
    for (h, s), p in case["h2d_after"].items():
        assert h2d[h, s].item() == p
    for h, s, p in case["payload"]:
        assert same(hbm[h, s], dram[h, p])
    assert step.item() == lru_kats.STEP        # the raw function does not advance the step


@pytest.mark.parametrize("itype,ttype", [(torch.int32, torch.int32), (torch.int64, torch.float32)])
def test_load_lru_cache_when_the_step_ties_with_stored_times(itype, ttype):
    """The raw function takes the caller's step as the time stamp; when it equals stored
    access times, a slot the touch pass has just hit is still first in the eviction
    order, and the reference's walk evicts it and pages the same page in again later
    (hand-walked in tests/golden/lru_kats.py).  Calls without the step bump therefore
    take the literal walk."""
    from dram_attention_amd import load_lru_cache_

    c = lru_kats.STAMP_TIES
    dram = torch.randn(1, c["n_dram_pages"], 64, generator=gen(19)).to(DEV)
    hbm = dram[:, 3:6].clone()
    time = torch.tensor(c["time"], dtype=ttype, device=DEV)
    d2h = torch.tensor(c["d2h"], dtype=itype, device=DEV)
    h2d = torch.tensor(c["h2d"], dtype=itype, device=DEV)
    step = torch.tensor([c["step"]], dtype=torch.int32, device=DEV)
    load_lru_cache_(dram_kv_cache=dram, page_access_time=time,
                    dram_page_to_hbm_page_mapping=d2h, hbm_page_to_dram_page_mapping=h2d,
                    topk_dram_page_index=torch.tensor(c["topk"], dtype=itype, device=DEV),
                    current_step=step, hbm_kv_cache=hbm)
    assert d2h.cpu().tolist() == c["d2h_after"] and h2d.cpu().tolist() == c["h2d_after"]
    assert time.cpu().float().tolist() == c["time_after"]
    assert same(hbm[0], dram[0, [0, 1, 3]])
    # and against the oracle on a random trace where every step repeats the stamp
    rng = np.random.default_rng(5)
    H, P, N, K = 3, 40, 12, 9
    dram = torch.randn(H, P, 64, generator=gen(20))
    st = O.LruState.initial(H, P, N)
    hbm_o = dram[:, P - N:].clone()
    hbm = hbm_o.to(DEV)
    time = torch.zeros(H, N, dtype=ttype, device=DEV)
    d2h = torch.from_numpy(st.d2h).to(itype).to(DEV)
    h2d = torch.from_numpy(st.h2d).to(itype).to(DEV)
    for s in (0, 0, 1, 1, 1, 3):
        idx = rng.integers(0, P, (H, K))
        O.lru_load(st, idx, s, dram.numpy(), hbm_o.numpy())
        load_lru_cache_(dram_kv_cache=dram.to(DEV), page_access_time=time,
                        dram_page_to_hbm_page_mapping=d2h, hbm_page_to_dram_page_mapping=h2d,
                        topk_dram_page_index=torch.from_numpy(idx).to(itype).to(DEV),
                        current_step=torch.tensor([s], dtype=torch.int32, device=DEV),
                        hbm_kv_cache=hbm)
        assert np.array_equal(time.cpu().numpy().astype(np.float32), st.time), f"time, stamp {s}"
        assert np.array_equal(d2h.cpu().numpy(), st.d2h) and np.array_equal(h2d.cpu().numpy(), st.h2d)
        assert same(hbm.cpu(), hbm_o)


def lru_trace(H, P, N, K, steps, seed, itype, ttype, pinned, dtype=torch.bfloat16, page_dim=256,
              hot=None, serial_walk=False, candidates=False, refresh_every=1):
    """Random request trace on LRUCache-like state; compares every buffer with the
    oracle's serial walk after every step."""
    from dram_attention_amd.lru_kernel import LruScratch, lru_candidates, lru_update_and_gather

    rng = np.random.default_rng(seed)
    dram = torch.randn(H, P, page_dim, generator=gen(seed)).to(dtype)
    dram_dev = dram.pin_memory() if pinned else dram.to(DEV)
    st = O.LruState.initial(H, P, N)
    hbm_o = dram[:, P - N:].clone()
    hbm = hbm_o.to(DEV)
    time = torch.zeros(H, N, dtype=ttype, device=DEV)
    d2h = torch.from_numpy(st.d2h).to(itype).to(DEV)
    h2d = torch.from_numpy(st.h2d).to(itype).to(DEV)
    step = torch.zeros(1, dtype=torch.int32, device=DEV)
    scratch = LruScratch.allocate(H, K, DEV, N)
    as_np = (lambda t: t.view(torch.int16).numpy()) if dtype != torch.float32 else (lambda t: t.numpy())
    for s in range(1, steps + 1):
        if hot:  # skewed requests with duplicates, like overlapping per-head top-k lists
            idx = np.where(rng.random((H, K)) < 0.7, rng.integers(0, hot, (H, K)),
                           rng.integers(0, P, (H, K)))
        else:
            idx = rng.integers(0, P, (H, K))
        hit_o, miss_o = O.lru_load(st, idx, s, as_np(dram), as_np(hbm_o))
        if candidates and (s - 1) % refresh_every:
            pass             # the update below is handed the list of an earlier step
        elif candidates:     # the least recent slots listed ahead of the update, as the module does
            order = lru_candidates(time, scratch, step).cpu()
            want = torch.sort(time.cpu().float(), dim=1, stable=True).indices[:, :order.shape[1]]
            assert same(order.long(), want), f"candidates, step {s}"
        lru_update_and_gather(dram_dev, time, d2h, h2d, torch.from_numpy(idx).to(itype).to(DEV),
                              step, hbm, scratch, bump_step=True, serial_walk=serial_walk,
                              use_candidates=candidates)
        torch.cuda.synchronize()
        assert step.item() == s
        assert np.array_equal(time.cpu().numpy().astype(np.float32), st.time), f"time, step {s}"
        assert np.array_equal(d2h.cpu().numpy(), st.d2h), f"d2h, step {s}"
        assert np.array_equal(h2d.cpu().numpy(), st.h2d), f"h2d, step {s}"
        assert np.array_equal(scratch.hit_mask.cpu().numpy().astype(bool), hit_o), f"hits, step {s}"
        counts = scratch.miss_count.cpu().tolist()
        mp, ms = scratch.miss_page.cpu().numpy(), scratch.miss_slot.cpu().numpy()
        for h in range(H):
            assert counts[h] == len(miss_o[h])
            got = [(int(mp[h, i]), int(ms[h, i])) for i in range(counts[h])]
            if K <= N:
                assert got == miss_o[h]
            else:  # serial walk: only the last entry that targets a slot stays live
                last = {}
                for i, (p, v) in enumerate(miss_o[h]):
                    last[v] = i
                assert [(p, v) for p, v in got if v >= 0] == \
                    [(p, v) for i, (p, v) in enumerate(miss_o[h]) if last[v] == i]
                live_slots = [v for p, v in got if v >= 0]
                assert len(live_slots) == len(set(live_slots))
        assert same(hbm.cpu(), hbm_o), f"payload, step {s}"


@pytest.mark.parametrize("H,P,N,K,itype,ttype,pinned", [
    (2, 64, 16, 8, torch.int64, torch.float32, True),
    (8, 512, 128, 128, torch.int64, torch.float32, True),      # K == N_hbm
    (3, 300, 100, 37, torch.int32, torch.int32, False),
    (4, 2048, 1024, 1024, torch.int64, torch.float32, False),  # K == N_hbm, several scan rounds
    (2, 4096, 2048, 1500, torch.int64, torch.float32, True),
])
def test_lru_update_matches_serial_walk(H, P, N, K, itype, ttype, pinned):
    lru_trace(H, P, N, K, 12, 100 + K, itype, ttype, pinned)
    lru_trace(H, P, N, K, 12, 200 + K, itype, ttype, pinned, hot=max(2, P // 8))


@pytest.mark.parametrize("H,P,N,K,ttype", [
    (8, 8192, 2048, 1024, torch.float32),     # the 128K layer: list of 256, ~120 victims per step
    (4, 1024, 256, 200, torch.float32),       # list of 256 with up to 200 of them touched: falls back
    (2, 4096, 600, 64, torch.int32),          # list of 256 of 600 slots
    (3, 300, 100, 37, torch.float32),
    (2, 16384, 4096, 4096, torch.float32),    # the 1M layer's shape: list of 2048, filtered in two rounds
    (2, 9000, 3000, 2500, torch.int32),       # list of 1250: a partial second round
])
def test_lru_update_with_candidate_list_matches_serial_walk(H, P, N, K, ttype):
    """Victims taken from the list of least recent slots made ahead of the update
    (touched ones dropped), with the kernel's own ordering as the fallback."""
    lru_trace(H, P, N, K, 10, 400 + K, torch.int64, ttype, False, candidates=True)
    lru_trace(H, P, N, K, 10, 500 + K, torch.int64, ttype, False, hot=max(2, P // 8),
              candidates=True)


@pytest.mark.parametrize("H,P,N,K,ttype", [
    (8, 8192, 2048, 1024, torch.float32),     # the 128K layer
    (2, 16384, 4096, 4096, torch.float32),    # the 1M layer's shape: the complete order as the list
    (3, 300, 100, 37, torch.int32),
])
def test_lru_update_ignores_a_stale_candidate_list(H, P, N, K, ttype):
    """A list of least recent slots made one or two updates ago no longer describes the
    access times.  Its stamp (the step counter when it was made) says so: the update
    orders the slots itself and ends in the serial walk's state, as without a list."""
    lru_trace(H, P, N, K, 9, 600 + K, torch.int64, ttype, False, candidates=True, refresh_every=3)
    lru_trace(H, P, N, K, 9, 700 + K, torch.int64, ttype, False, hot=max(2, P // 8),
              candidates=True, refresh_every=3)


def test_lru_update_forced_serial_walk_gives_the_same_state():
    """The literal walk, forced where the parallel form applies: same end state."""
    lru_trace(4, 1024, 256, 200, 10, 77, torch.int64, torch.float32, False, serial_walk=True)
    lru_trace(2, 512, 128, 128, 6, 78, torch.int32, torch.int32, True, hot=64, serial_walk=True)


def test_lru_update_rejects_maps_that_do_not_match_the_page_stores():
    """The kernel indexes the access times and the slot->page map by slot and the
    page->slot map by page: extents that differ from the stores' raise on the host,
    before any launch."""
    from dram_attention_amd.lru_kernel import LruScratch, lru_update

    H, P, N, K = 2, 64, 8, 4
    dram = torch.zeros(H, P, 16, device=DEV)
    hbm = torch.zeros(H, N, 16, device=DEV)
    good = dict(time=torch.zeros(H, N, device=DEV),
                d2h=torch.full((H, P), -1, dtype=torch.int64, device=DEV),
                h2d=torch.full((H, N), -1, dtype=torch.int64, device=DEV))
    idx = torch.zeros(H, K, dtype=torch.int64, device=DEV)
    step = torch.zeros(1, dtype=torch.int32, device=DEV)
    sc = LruScratch.allocate(H, K, DEV, N)
    for name, bad in (("time", torch.zeros(H, N - 1, device=DEV)),
                      ("d2h", torch.full((H, P + 3), -1, dtype=torch.int64, device=DEV)),
                      ("h2d", torch.full((H, 2 * N), -1, dtype=torch.int64, device=DEV))):
        a = dict(good, **{name: bad})
        with pytest.raises(ValueError, match="the page stores need"):
            lru_update(dram, a["time"], a["d2h"], a["h2d"], idx, step, hbm, sc, True)
    with pytest.raises(ValueError, match="one row per head"):
        lru_update(dram, good["time"], good["d2h"], good["h2d"], idx[:1], step, hbm, sc, True)
    assert step.item() == 0


@pytest.mark.parametrize("H,P,N,K", [(2, 40, 6, 17), (1, 8, 2, 3), (3, 200, 50, 120),
                                     (2, 60, 10, 70)])
def test_lru_update_more_requests_than_slots(H, P, N, K):
    lru_trace(H, P, N, K, 8, 300 + K, torch.int64, torch.float32, False, dtype=torch.float32,
              page_dim=32)
    # requests crowded onto few pages: a page comes back to the slot it was evicted from
    lru_trace(H, P, N, K, 8, 350 + K, torch.int64, torch.float32, False, dtype=torch.float32,
              page_dim=32, hot=max(3, N + 2))
    lru_trace(H, P, N, K, 8, 400 + K, torch.int64, torch.float32, False, dtype=torch.float32,
              page_dim=32, hot=max(2, P // 4))


# ------------------------------------------------------------------ decode attention
def dense_reference(q, segments):
    k = torch.cat([s[0] for s in segments], dim=1)
    v = torch.cat([s[1] for s in segments], dim=1)
    return O.attention_partial(q, k, v)


@pytest.mark.parametrize("dtype,atol,rtol", [(torch.float32, 2e-5, 1e-4),
                                             (torch.bfloat16, 2e-2, 1e-2),
                                             (torch.float16, 4e-3, 1e-2)])
@pytest.mark.parametrize("Hq,Hkv,D,p_len,c_len,cap", [
    (32, 8, 128, 2048, 500, 640), (8, 2, 64, 512, 1008, 1040), (4, 4, 128, 0, 77, 128),
    (16, 2, 64, 333, 0, 64), (6, 2, 128, 1000, 31, 32), (2, 1, 256, 40, 3, 8),
    (64, 8, 128, 4096, 100, 200), (12, 2, 128, 700, 45, 64), (32, 2, 64, 300, 9, 16)])
def test_decode_attention_matches_dense(dtype, atol, rtol, Hq, Hkv, D, p_len, c_len, cap):
    from dram_attention_amd import decode_attention

    g = gen(19)
    q = torch.randn(Hq, D, generator=g).to(dtype)
    # the prefix as the LRU hands it over: K/V interleaved per token
    inter = torch.randn(Hkv, max(p_len, 1), 2, D, generator=g).to(dtype)[:, :p_len]
    ck = torch.zeros(cap, Hkv, D, dtype=dtype)
    cv = torch.zeros(cap, Hkv, D, dtype=dtype)
    ck[:c_len] = torch.randn(c_len, Hkv, D, generator=g).to(dtype)
    cv[:c_len] = torch.randn(c_len, Hkv, D, generator=g).to(dtype)
    nk = torch.randn(Hkv, D, generator=g).to(dtype)
    nv = torch.randn(Hkv, D, generator=g).to(dtype)
    want, want_lse = dense_reference(q, [
        (inter[:, :, 0], inter[:, :, 1]),
        (ck[:c_len].transpose(0, 1), cv[:c_len].transpose(0, 1)),
        (nk[:, None], nv[:, None])])
    inter_d, ckd, cvd = inter.to(DEV), ck.to(DEV), cv.to(DEV)
    lse = torch.empty(Hq, dtype=torch.float32, device=DEV)
    out = decode_attention(q.to(DEV), inter_d[:, :, 0], inter_d[:, :, 1], ckd, cvd, c_len,
                           nk.to(DEV), nv.to(DEV), lse=lse)
    assert out.dtype == dtype
    assert close(out.cpu().float(), want, atol, rtol)
    assert torch.allclose(lse.cpu(), want_lse, atol=2e-3 if dtype != torch.float32 else 1e-4)
    # the append happened in place, nothing else moved
    assert same(ckd[c_len].cpu(), nk) and same(cvd[c_len].cpu(), nv)
    assert same(ckd[:c_len].cpu(), ck[:c_len]) and same(ckd[c_len + 1:].cpu(), ck[c_len + 1:])
    # device-side length gives the same bits
    ckd2, cvd2 = ck.to(DEV), cv.to(DEV)
    out2 = decode_attention(q.to(DEV), inter_d[:, :, 0], inter_d[:, :, 1], ckd2, cvd2,
                            torch.tensor([c_len], dtype=torch.int32, device=DEV),
                            nk.to(DEV), nv.to(DEV))
    assert same(out2, out) and same(ckd2, ckd)


def test_decode_attention_large_logits_and_no_append():
    from dram_attention_amd import decode_attention

    g = gen(20)
    Hq, Hkv, D, T = 8, 2, 128, 700
    q = (torch.randn(Hq, D, generator=g) * 6).bfloat16()
    k = (torch.randn(Hkv, T, D, generator=g) * 3).bfloat16()
    v = torch.randn(Hkv, T, D, generator=g).bfloat16()
    ck = k[:, 400:].transpose(0, 1).contiguous()
    cv = v[:, 400:].transpose(0, 1).contiguous()
    out = decode_attention(q.to(DEV), k[:, :400].to(DEV), v[:, :400].to(DEV), ck.to(DEV),
                           cv.to(DEV), 300, None, None)
    want, _ = O.attention_partial(q, k, v)
    assert close(out.cpu().float(), want, 2e-2, 1e-2)


def test_decode_attention_rejects_overflow_and_bad_dim():
    from dram_attention_amd import decode_attention

    q = torch.zeros(4, 64, device=DEV)
    c = torch.zeros(8, 2, 64, device=DEV)
    n = torch.zeros(2, 64, device=DEV)
    with pytest.raises(RuntimeError, match="overflow"):
        decode_attention(q, None, None, c, c.clone(), 8, n, n)
    with pytest.raises(RuntimeError):
        decode_attention(torch.zeros(4, 24, device=DEV), None, None,
                         torch.zeros(8, 2, 24, device=DEV), torch.zeros(8, 2, 24, device=DEV), 1,
                         None, None)


def test_lru_update_with_a_caller_stamp_and_more_slots_than_the_walk_orders_is_refused():
    """Without the step bump the stamp may tie with stored times and only the literal walk
    is right; the walk orders at most 8192 slots per head, so such a call with more slots
    is refused before any launch instead of running a form that could evict a slot it hit."""
    from dram_attention_amd.lru_kernel import LruScratch, lru_update

    H, P, N, K = 1, 20000, 9000, 8
    dram = torch.zeros(H, P, 16, device=DEV)
    hbm = torch.zeros(H, N, 16, device=DEV)
    time = torch.zeros(H, N, device=DEV)
    d2h = torch.full((H, P), -1, dtype=torch.int64, device=DEV)
    h2d = torch.full((H, N), -1, dtype=torch.int64, device=DEV)
    idx = torch.arange(K, device=DEV)[None]
    step = torch.ones(1, dtype=torch.int32, device=DEV)
    sc = LruScratch.allocate(H, K, DEV, N)
    with pytest.raises(RuntimeError, match="caller-supplied time stamp"):
        lru_update(dram, time, d2h, h2d, idx, step, hbm, sc, bump_step=False)
    lru_update(dram, time, d2h, h2d, idx, step, hbm, sc, bump_step=True)      # the bumped form runs
    torch.cuda.synchronize()
    assert step.item() == 2 and sc.miss_count.item() == K
