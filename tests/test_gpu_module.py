"""The drop-in surface (LRUCache, DRAMAttention) on the GPU: the reference's own
object-level tests restated, and step-by-step parity of whole decode runs with
the CPU oracle."""

import math

import numpy as np
import pytest
import torch

from dram_attention_amd.synthetic import WORKLOADS, DecodeInputs, make_prompt
from oracle import dram_attention_oracle as O

from tests.parity import check_invariants, check_step
from tests.util import close, same

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ------------------------------------------------------------ reference lru_cache_test.py
@pytest.fixture
def sample_cache():
    from dram_attention_amd import LRUCache

    g = torch.Generator().manual_seed(0)
    k = torch.randn(4, 1024 * 8, 64, generator=g).to(DEV)
    v = torch.randn(4, 1024 * 8, 64, generator=g).to(DEV)
    return LRUCache(k, v, page_size=16, top_k=10)


def test_lru_cache_initialization(sample_cache):
    c = sample_cache
    assert (c.num_kv_heads, c.num_dram_pages, c.num_hbm_pages) == (4, 512, 102)
    assert (c.head_dim, c.page_size, c.top_k) == (64, 16, 10)
    assert torch.all(c.dram_page_to_hbm_page_mapping[:, -102:] == torch.arange(102, device=DEV))
    assert torch.all(c.dram_page_to_hbm_page_mapping[:, :-102] == -1)
    assert c.dram_kv_cache.is_pinned() and c.dram_kv_cache.shape == (4, 512, 16 * 2 * 64)
    assert same(c.hbm_kv_cache.cpu(), c.dram_kv_cache[:, -102:])


def test_lru_cache_load_inline_method(sample_cache):
    idx = torch.randint(0, 512, (4, 10), device=DEV)
    k_cache, v_cache = sample_cache.load_(idx)
    assert k_cache.shape == (4, 102 * 16, 64) and v_cache.shape == (4, 102 * 16, 64)
    assert sample_cache.current_step == 1
    # every requested page is resident and its payload sits in the slot the map names
    slots = torch.gather(sample_cache.dram_page_to_hbm_page_mapping, 1, idx)
    assert torch.all(slots >= 0)
    for h in range(4):
        got = sample_cache.hbm_kv_cache[h, slots[h]].cpu()
        assert same(got, sample_cache.dram_kv_cache[h, idx[h].cpu()])


@pytest.mark.parametrize("page_size", [8, 16, 32])
def test_lru_cache_different_page_sizes(page_size):
    from dram_attention_amd import LRUCache

    k = torch.randn(4, 1024 * 8, 64)
    v = torch.randn(4, 1024 * 8, 64)
    cache = LRUCache(k, v, page_size=page_size, top_k=10)     # host tensors are accepted
    assert cache.page_size == page_size and cache.num_dram_pages == 1024 * 8 // page_size
    assert cache.top_k == 10
    assert cache.top_k_selector.chunk_min_max.shape == (4, 1024 * 8 // page_size, 2, 64)


@pytest.mark.parametrize("dtype,H,S,D,page,lru", [
    (torch.bfloat16, 8, 4096, 128, 16, 1024), (torch.float32, 2, 512, 64, 8, 64),
    (torch.float16, 3, 960, 64, 32, 320), (torch.float32, 2, 256, 24, 16, 64),   # D=24: rows of 96 B
    (torch.bfloat16, 2, 256, 36, 16, 32),                                       # rows of 72 B: torch copies
])
def test_page_store_build_matches_layout(dtype, H, S, D, page, lru):
    """Pinned page store and initial slots, from the strided views init_cache hands
    over: token t of page p holds K[h, p*page+t] then V[h, p*page+t]; slot s holds
    page P - N + s; the maps say so."""
    from dram_attention_amd import LRUCache

    g = torch.Generator().manual_seed(5)
    k = torch.randn(S, H, D, generator=g).to(dtype)
    v = torch.randn(S, H, D, generator=g).to(dtype)
    cache = LRUCache(k.to(DEV).transpose(0, 1), v.to(DEV).transpose(0, 1), page_size=page,
                     top_k=4 * page, lru_hbm_cache_size=lru)
    P, N = S // page, lru // page
    want = O.pack_pages(k.transpose(0, 1), v.transpose(0, 1), page)
    assert cache.dram_kv_cache.is_pinned() and same(cache.dram_kv_cache, want)
    assert same(cache.hbm_kv_cache.cpu(), want[:, P - N:])
    assert same(cache.hbm_page_to_dram_page_mapping.cpu(),
                torch.arange(P - N, P).repeat(H, 1))
    d2h = cache.dram_page_to_hbm_page_mapping.cpu()
    assert (d2h[:, :P - N] == -1).all() and same(d2h[:, P - N:], torch.arange(N).repeat(H, 1))


def test_lru_cache_invalid_initialization_and_hbm_size():
    from dram_attention_amd import LRUCache

    with pytest.raises(AssertionError):
        LRUCache(torch.randn(4, 1007 * 8, 64), torch.randn(4, 1007 * 8, 64), page_size=16, top_k=10)
    k = torch.randn(4, 1024 * 8, 64)
    cache = LRUCache(k, k.clone(), page_size=16, lru_hbm_cache_size=1024, top_k=10)
    assert cache.num_hbm_pages == 64 and cache.top_k == 10


def test_lru_cache_get_kv_cache_inline(sample_cache):
    query = torch.randn(1, 10, 4, 64, generator=torch.Generator().manual_seed(1)).to(DEV)
    out = sample_cache.get_kv_cache_(query)
    assert out.k_cache.shape == (4, 102 * 16, 64) and out.v_cache.shape == (4, 102 * 16, 64)
    assert sample_cache.current_step == 1
    sample_cache.get_kv_cache_(query)
    assert sample_cache.current_step == 2
    assert out.k_cache.device.type == "cuda" and out.v_cache.device.type == "cuda"
    assert torch.any(out.k_cache != 0) and torch.any(out.v_cache != 0)
    # selection of a 10-token query block equals the oracle's on the kernel's own scores
    sel = sample_cache.top_k_selector
    scores = sel.scores(query).cpu()
    want = O.select_pages(scores, 10, 1, 10)
    assert same(sel.top_k(query, 10).cpu(), want)


# ------------------------------------------------------------ reference dram_attention_test.py
def make_module(**kw):
    from dram_attention_amd import DRAMAttention

    args = dict(max_output_length=64, lru_hbm_cache_size=32 * 1024, local_cache_size=4096 + 512,
                page_size=16, top_k=4096, n_kv_heads=8, head_dim=128, device=DEV)
    args.update(kw)
    return DRAMAttention(**args)


def test_module_init_and_errors():
    m = make_module()
    assert (m.max_output_length, m.lru_hbm_cache_size, m.local_cache_size) == (64, 32768, 4608)
    assert (m.page_size, m.top_k, m.n_kv_heads, m.head_dim) == (16, 4096, 8, 128)
    assert m.cache_k.shape == (1, 4608 + 64, 8, 128) and m.cache_k.dtype == torch.bfloat16
    x = torch.randn(1, 1, 8, 128, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="Unsupported stage"):
        m(x, x, x, start_pos=0, stage="invalid")
    x2 = torch.randn(2, 1, 8, 128, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="Only support batch size 1"):
        m(x2, x2, x2, start_pos=0, stage="prefill")


def test_init_cache_from_layer_file(tmp_path):
    """A layer set up from the chat example's cache file holds the page store the oracle
    packs from the same K/V, decodes step by step like the oracle, and like a layer
    set up from the tensors themselves."""
    from dram_attention_amd import DRAMAttention, save_layer_cache

    w = WORKLOADS["128k"].scaled(dram_tokens=4096, local_cache=256, lru_tokens=1024,
                                 top_k_tokens=256, steps=3)
    prompt = make_prompt(w, 11)
    save_layer_cache(str(tmp_path), 3, prompt.k, prompt.v)
    mods = []
    for from_file in (True, False):
        m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        if from_file:
            assert m.init_cache_from_file(str(tmp_path), 3) == w.prompt_tokens
        else:
            m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        mods.append(m)
    assert same(mods[0].lru_cache.dram_kv_cache, mods[1].lru_cache.dram_kv_cache)
    # the page store built from the file is the reference's layout of the file's K/V
    S = mods[0].dram_kv_cache_size
    assert same(mods[0].lru_cache.dram_kv_cache,
                O.pack_pages(prompt.k[0, :S].transpose(0, 1), prompt.v[0, :S].transpose(0, 1), w.page_size))
    o = O.DecodeOracle(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    inputs = DecodeInputs(w, prompt.q0, 11)
    for t in range(w.steps):
        xq, xk, xv = inputs.next()
        a = mods[0](xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        b = mods[1](xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        assert same(a, b)
        check_step(mods[0], o, xq, xk, xv, w.prompt_tokens + t, a, t, 2e-2, 1e-2)


def test_module_prefill_then_generate_shapes():
    """The reference's prefill/generate smoke at its 66K-token shape."""
    m = make_module()
    S = 66 * 1024
    g = torch.Generator(device=DEV).manual_seed(0)
    xq = torch.randn(1, S, 32, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    xk = torch.randn(1, S, 8, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    xv = torch.randn(1, S, 8, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    out = m(xq, xk, xv, start_pos=0, stage="prefill")
    assert out.shape == (1, S, 32, 128)
    assert m.dram_kv_cache_size == (S - 4608 + 16) // 16 * 16
    # causal check on a few rows against a direct softmax
    for row in (0, 17, 5000):
        qs = xq[0, row].float().view(8, 4, 128)
        s = torch.einsum("hrd,thd->hrt", qs, xk[0, : row + 1].float()) / math.sqrt(128)
        want = torch.einsum("hrt,thd->hrd", torch.softmax(s, -1), xv[0, : row + 1].float())
        assert close(out[0, row].float().view(8, 4, 128), want, 2e-2, 2e-2)
    q1 = torch.randn(1, 1, 32, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    k1 = torch.randn(1, 1, 8, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    v1 = torch.randn(1, 1, 8, 128, device=DEV, dtype=torch.bfloat16, generator=g)
    o1 = m(q1, k1, v1, start_pos=S, stage="generate")
    assert o1.shape == (1, 1, 32, 128) and torch.isfinite(o1.float()).all()


def test_prefill_call_then_generate_matches_oracle():
    """The model-side sequence of the reference (forward with stage="prefill" and
    start_pos=0, then one generate call per token with integer positions): the cache
    the prefill call builds decodes like the oracle's built from the same K/V."""
    from dram_attention_amd import DRAMAttention, LRUCache

    w = WORKLOADS["128k"].scaled(dram_tokens=8192, local_cache=512, lru_tokens=2048,
                                 top_k_tokens=512, steps=4)
    prompt = make_prompt(w, 21)
    S = w.prompt_tokens
    g = torch.Generator().manual_seed(22)
    xq0 = torch.randn(1, S, w.n_q_heads, w.head_dim, generator=g).to(w.dtype)
    m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                      w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
    out0 = m(xq0.to(DEV), prompt.k.to(DEV), prompt.v.to(DEV), start_pos=0, stage="prefill")
    assert out0.shape == xq0.shape and isinstance(m.lru_cache, LRUCache)
    o = O.DecodeOracle(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    assert m.dram_kv_cache_size == o.dram_kv_cache_size
    assert same(m.lru_cache.dram_kv_cache, o.dram)
    inputs = DecodeInputs(w, prompt.q0, 21)
    for t in range(w.steps):
        xq, xk, xv = inputs.next()
        got = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=S + t, stage="generate")
        want = o.generate(xq, xk, xv, S + t, scores=m.lru_cache.top_k_selector._scores.cpu())
        assert same(m.lru_cache._topk_idx.cpu(), o.last_idx)
        assert close(got.cpu().float(), want.float(), 2e-2, 1e-2), f"step {t}"


def test_prefill_call_at_the_headline_size_builds_the_same_layer_as_init_cache():
    """configs[2] as a model would run it: forward(stage="prefill") over the whole
    135 152-token prompt (the library's causal kernel, summaries, page store, slots), then
    generate calls.  The state the call leaves is bit-equal to what init_cache builds from
    the same K/V, the decode steps that follow are bit-equal too, and the prefill output
    is held against a dense fp32 causal softmax on sampled rows."""
    from dram_attention_amd import DRAMAttention

    w = WORKLOADS["128k"]
    prompt = make_prompt(w, 31)
    S = w.prompt_tokens
    g = torch.Generator(device=DEV).manual_seed(32)
    xq0 = torch.randn(1, S, w.n_q_heads, w.head_dim, device=DEV, generator=g).to(w.dtype)
    k, v = prompt.k.to(DEV), prompt.v.to(DEV)

    def layer():
        return DRAMAttention(8, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                             w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)

    m, r = layer(), layer()
    out0 = m(xq0, k, v, start_pos=0, stage="prefill")
    r.init_cache(k, v)
    assert out0.shape == xq0.shape and m.dram_kv_cache_size == r.dram_kv_cache_size
    for name in ("dram_kv_cache", "hbm_kv_cache", "page_access_time", "dram_page_to_hbm_page_mapping",
                 "hbm_page_to_dram_page_mapping"):
        assert same(getattr(m.lru_cache, name), getattr(r.lru_cache, name)), name
    assert same(m.cache_k, r.cache_k) and same(m.cache_v, r.cache_v)
    assert same(m.lru_cache.top_k_selector.chunk_min_max, r.lru_cache.top_k_selector.chunk_min_max)

    # the prefill output on sampled rows of every head
    rep = w.n_q_heads // w.n_kv_heads
    rows = torch.tensor(sorted(set(list(range(0, 40)) + [4095, 4096, 65535, 65536, 100000] + list(range(S - 40, S)))),
                        device=DEV)
    keys = torch.arange(S, device=DEV)
    for h in range(w.n_kv_heads):
        q = xq0[0, rows, h * rep:(h + 1) * rep].float().transpose(0, 1)
        sc = torch.matmul(q, k[0, :, h].float().t()) / math.sqrt(w.head_dim)
        sc.masked_fill_(keys[None, None, :] > rows[None, :, None], float("-inf"))
        want = torch.matmul(torch.softmax(sc, dim=-1), v[0, :, h].float()).transpose(0, 1)
        assert close(out0[0, rows, h * rep:(h + 1) * rep].float(), want, 2e-2, 1e-2)

    inputs = DecodeInputs(w, prompt.q0, 31)
    for t in range(3):
        xq, xk, xv = (x.to(DEV) for x in inputs.next())
        got = m(xq, xk, xv, start_pos=S + t, stage="generate")
        ref = r(xq, xk, xv, start_pos=S + t, stage="generate")
        assert same(got, ref), f"step {t}"
        assert same(m.lru_cache._topk_idx, r.lru_cache._topk_idx)


# ------------------------------------------------------------ whole decode runs vs the oracle
def run_parity(w, seed, steps, atol, rtol, device_pos=False):
    """Drives the module and the oracle with the same inputs.  Selection and LRU
    state are compared bit for bit at every step, the oracle being fed the
    kernel's scores (the contract is 'given identical scores'); the kernel's
    scores themselves are compared with the oracle's within one rounding step."""
    from dram_attention_amd import DRAMAttention, LRUCache

    prompt = make_prompt(w, seed)
    m = DRAMAttention(max_output_length=w.steps, lru_hbm_cache_size=w.lru_tokens,
                      local_cache_size=w.local_cache, page_size=w.page_size,
                      top_k=w.top_k_tokens, n_kv_heads=w.n_kv_heads, head_dim=w.head_dim,
                      device=DEV, dtype=w.dtype)
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    o = O.DecodeOracle(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    assert m.dram_kv_cache_size == o.dram_kv_cache_size == w.dram_tokens
    assert isinstance(m.lru_cache, LRUCache) and o.uses_lru
    lru = m.lru_cache
    assert same(lru.top_k_selector.chunk_min_max.cpu(), o.min_max)
    assert same(lru.dram_kv_cache, o.dram)
    inputs = DecodeInputs(w, prompt.q0, seed)
    pos = torch.tensor([w.prompt_tokens], dtype=torch.int32, device=DEV)
    hits = total = 0
    for t in range(steps):
        xq, xk, xv = inputs.next()
        start = w.prompt_tokens + t
        out = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=pos if device_pos else start,
                stage="generate")
        pos += 1
        check_step(m, o, xq, xk, xv, start, out, t, atol, rtol)
        if t == 0:
            for h, page in prompt.planted:
                assert (o.last_idx[h] == page).any(), "planted page not selected"
        hits += int(o.last_hit.sum())
        total += o.last_hit.size
    c = w.prompt_tokens + steps - w.dram_tokens
    assert same(m.cache_k[0, :c].cpu(), o.cache_k[:c])
    assert same(m.cache_v[0, :c].cpu(), o.cache_v[:c])
    return hits / total


def test_decode_parity_cpu_reference_config():
    """configs[0] exactly: fp32, 8/2 heads, D 64, 8192-token prefix, K == N_hbm."""
    w = WORKLOADS["cpu"]
    rate = run_parity(w, 0, w.steps, atol=1e-4, rtol=1e-4)
    assert 0.0 < rate < 1.0


@pytest.mark.parametrize("name,steps", [("128k", 64), ("1m", 8)])
def test_decode_parity_full_size(name, steps):
    """configs[2] for all of its 64 steps and configs[4] for its first 8, at full size,
    step by step against the oracle (which is fed the kernel's scores): request lists,
    hit masks, both maps, access times and slot payload bit for bit, attention within
    the bf16 tolerance; the position stays on the device."""
    rate = run_parity(WORKLOADS[name], 0, steps, atol=2e-2, rtol=1e-2, device_pos=True)
    assert 0.5 < rate < 0.95


def test_decode_parity_bf16_scaled_llama_shape():
    """The 128K layer shape scaled to a prefix the oracle walks in seconds."""
    w = WORKLOADS["128k"].scaled(dram_tokens=16384, local_cache=1024, lru_tokens=4096,
                                 top_k_tokens=1024, steps=12)
    run_parity(w, 1, w.steps, atol=2e-2, rtol=1e-2)


def test_decode_parity_device_side_position_and_rep8():
    w = WORKLOADS["1m"].scaled(dram_tokens=8192, local_cache=512, lru_tokens=2048,
                               top_k_tokens=256, steps=6, planted_pages=8)
    run_parity(w, 2, w.steps, atol=2e-2, rtol=1e-2, device_pos=True)


def test_decode_parity_more_requests_than_slots():
    """rep * pages-per-head > slots: the LRU takes the serial walk, victims wrap
    onto slots handed out earlier in the same step, and the superseded entries of
    the miss list must be skipped by the page stream and by its attention."""
    w = WORKLOADS["128k"].scaled(dram_tokens=8192, local_cache=512, lru_tokens=1024,
                                 top_k_tokens=512, steps=5)
    assert w.rep * w.pages_per_q_head > w.n_hbm_pages
    run_parity(w, 3, w.steps, atol=2e-2, rtol=1e-2)


def test_decode_parity_wide_gqa_group_takes_the_tail_pass():
    """16 query heads per kv head: outside what the attending page stream takes, so
    pages stream in on a side stream and a tail pass covers them."""
    from dram_attention_amd.lru_kernel import gather_attend_supported

    w = WORKLOADS["128k"].scaled(n_q_heads=32, n_kv_heads=2, dram_tokens=8192, local_cache=512,
                                 lru_tokens=2048, top_k_tokens=128, steps=4)
    assert not gather_attend_supported(w.n_q_heads, w.n_kv_heads, w.head_dim, w.page_size, w.dtype)
    run_parity(w, 5, w.steps, atol=2e-2, rtol=1e-2)


def test_decode_parity_page_size_not_a_power_of_two():
    """24-token pages: no shift for the page index, three 16-byte loads per lane and
    page in the stream, chunks that straddle pages in the first pass."""
    w = WORKLOADS["128k"].scaled(dram_tokens=24 * 320, local_cache=24 * 20, lru_tokens=24 * 96,
                                 top_k_tokens=24 * 12, steps=5, page_size=24)
    run_parity(w, 9, w.steps, atol=2e-2, rtol=1e-2)


def test_decode_parity_fp16():
    w = WORKLOADS["128k"].scaled(dram_tokens=8192, local_cache=512, lru_tokens=2048,
                                 top_k_tokens=512, steps=6, dtype=torch.float16)
    run_parity(w, 12, w.steps, atol=4e-3, rtol=1e-2)


def test_decode_parity_long_run_with_heavy_eviction():
    """150 steps on a small cache that turns over many times: every slot is
    re-assigned repeatedly and the step counter leaves the single digits."""
    w = WORKLOADS["128k"].scaled(n_q_heads=8, n_kv_heads=2, dram_tokens=4096, local_cache=128,
                                 lru_tokens=512, top_k_tokens=128, steps=150)
    rate = run_parity(w, 13, w.steps, atol=2e-2, rtol=1e-2)
    assert rate < 0.95      # the run really paged


def random_small_workload(rng):
    dtype = [torch.bfloat16, torch.float16, torch.float32][rng.integers(0, 3)]
    head_dim = int(rng.choice([64, 128] if dtype != torch.float32 else [32, 64]))
    n_kv = int(rng.integers(1, 5))
    rep = int(rng.choice([1, 2, 3, 4, 7, 8]))
    page = int(rng.choice([8, 16, 32]))
    n_pages = int(rng.integers(40, 200))
    n_slots = int(rng.integers(8, n_pages // 2))
    kp = int(rng.integers(1, min(n_slots, 24) + 1))
    local_pages = int(rng.integers(1, 9))
    return WORKLOADS["128k"].scaled(
        dtype=dtype, n_q_heads=n_kv * rep, n_kv_heads=n_kv, head_dim=head_dim, page_size=page,
        dram_tokens=n_pages * page, local_cache=local_pages * page, lru_tokens=n_slots * page,
        top_k_tokens=kp * page, steps=int(rng.integers(2, 6)))


@pytest.mark.parametrize("seed", range(96))
def test_decode_parity_random_small_shapes(seed):
    """Seeded sweep over head counts, GQA widths (also 3 and 7), head sizes, page sizes,
    cache geometries with more or fewer requests than slots, and the three dtypes."""
    rng = np.random.default_rng(1000 + seed)
    w = random_small_workload(rng)
    tol = {torch.float32: (1e-4, 1e-4), torch.float16: (4e-3, 1e-2), torch.bfloat16: (2e-2, 1e-2)}
    run_parity(w, 100 + seed, w.steps, *tol[w.dtype])


@pytest.mark.parametrize("seed", range(12))
def test_decode_parity_random_mid_size_shapes(seed):
    """Seeded sweep at sizes where the first attention pass has many chunks per kv head and
    the page stream of a step is long against it: the launch that carries both then lets
    a few workgroups per kv head walk the chunks (several rounds, a ragged last one),
    with 1, 2, 4 and 8 kv heads, GQA widths up to 8, both head sizes and three page sizes."""
    rng = np.random.default_rng(7000 + seed)
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    n_kv = [8, 4, 2, 1][seed % 4]
    rep = int(rng.choice([1, 2, 4, 8]))
    head_dim = int(rng.choice([64, 128]))
    page = int(rng.choice([8, 16, 32]))
    n_slots = int(rng.integers(160, 420))
    n_pages = int(rng.integers(3 * n_slots, 5 * n_slots))
    kp = int(rng.integers(n_slots // 8, n_slots // 3)) // rep + 1
    w = WORKLOADS["128k"].scaled(
        dtype=dtype, n_q_heads=n_kv * rep, n_kv_heads=n_kv, head_dim=head_dim, page_size=page,
        dram_tokens=n_pages * page, local_cache=int(rng.integers(4, 40)) * page,
        lru_tokens=n_slots * page, top_k_tokens=kp * page, steps=3)
    tol = {torch.float16: (4e-3, 1e-2), torch.bfloat16: (2e-2, 1e-2)}
    rate = run_parity(w, 300 + seed, w.steps, *tol[w.dtype])
    assert rate < 0.98          # the steps really paged


@pytest.mark.parametrize("seed", range(32))
def test_stream_variants_agree_on_random_small_shapes(seed):
    """Same workload through the three ways of running the page stream: inside the
    attention launch, as its own launch before attention (same bits), and copy-only
    with a tail pass (same state, output equal up to the merge order)."""
    from dram_attention_amd import DRAMAttention

    rng = np.random.default_rng(6000 + seed)
    w = random_small_workload(rng)
    prompt = make_prompt(w, 200 + seed)
    mods = []
    for overlap, fused in ((True, True), (False, True), (True, False)):
        m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        m.overlap_page_stream, m.attend_on_page_stream = overlap, fused
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        mods.append(m)
    inputs = DecodeInputs(w, prompt.q0, 200 + seed)
    atol, rtol = {torch.float32: (1e-5, 1e-4), torch.float16: (2e-3, 1e-2),
                  torch.bfloat16: (1e-2, 1e-2)}[w.dtype]
    for t in range(w.steps):
        xq, xk, xv = (x.to(DEV) for x in inputs.next())
        outs = [m(xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate") for m in mods]
        torch.cuda.synchronize()
        assert same(outs[0], outs[1]), f"step {t}"
        assert close(outs[0].float(), outs[2].float(), atol, rtol), f"step {t}"
        for m in mods[1:]:
            assert same(m.lru_cache.hbm_kv_cache, mods[0].lru_cache.hbm_kv_cache)
            assert same(m.lru_cache.page_access_time, mods[0].lru_cache.page_access_time)
            assert same(m.cache_k, mods[0].cache_k)


def test_machine_rates_of_the_stream_launch_move_time_only():
    """The stream + attention launch reads two rates of the machine (host link, one
    workgroup's HBM read rate) to decide how many workgroups compute the first pass
    next to the page stream.  Both extremes (every step leaves the pass to a few
    workgroups per kv head; no step does) give the same output, slots and cache rows
    bit for bit; another count of stream workgroups cuts the miss list differently, so
    the output agrees up to the order of the softmax merge and the state bit for bit."""
    from dram_attention_amd import DRAMAttention

    w = WORKLOADS["128k"].scaled(dram_tokens=32768, local_cache=2048, lru_tokens=8192,
                                 top_k_tokens=1024, steps=5)
    prompt = make_prompt(w, 9)
    mods = []
    for link, block, blocks in ((0.0, 0.0, 32), (1e-3, 1e6, 32), (1e6, 1e-3, 32), (54.0, 30.0, 16),
                                (1e-3, 1e6, 64)):
        m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        assert 10.0 < m.link_gbps < 200.0          # init_cache measured the box's link
        m.link_gbps, m.block_gbps, m.stream_blocks = link, block, blocks
        mods.append(m)
    inputs = DecodeInputs(w, prompt.q0, 9)
    for t in range(w.steps):
        xq, xk, xv = (x.to(DEV) for x in inputs.next())
        outs = [m(xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate") for m in mods]
        torch.cuda.synchronize()
        assert mods[0].lru_cache.last_miss_counts().sum().item() > 0
        for m, out in zip(mods[1:], outs[1:]):
            if m.stream_blocks == mods[0].stream_blocks:
                assert same(out, outs[0]), f"step {t}"
            else:
                assert close(out.float(), outs[0].float(), 1e-2, 1e-2), f"step {t}"
            assert same(m.lru_cache.hbm_kv_cache, mods[0].lru_cache.hbm_kv_cache)
            assert same(m.cache_k, mods[0].cache_k) and same(m.cache_v, mods[0].cache_v)


def test_page_stream_overlap_changes_nothing():
    """Attention issued around a concurrent page stream (two phases, side stream)
    gives the bits of the serialised order, and both agree with one plain pass."""
    from dram_attention_amd import DRAMAttention, decode_attention

    w = WORKLOADS["128k"].scaled(dram_tokens=16384, local_cache=1024, lru_tokens=4096,
                                 top_k_tokens=1024, steps=5)
    prompt = make_prompt(w, 4)
    mods = []
    for overlap in (True, False):
        m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, 16, w.top_k_tokens, w.n_kv_heads,
                          w.head_dim, device=DEV, dtype=w.dtype)
        m.overlap_page_stream = overlap
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        mods.append(m)
    inputs = DecodeInputs(w, prompt.q0, 4)
    for t in range(w.steps):
        xq, xk, xv = (x.to(DEV) for x in inputs.next())
        a = mods[0](xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate")
        b = mods[1](xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate")
        torch.cuda.synchronize()
        assert mods[0].lru_cache.last_miss_counts().sum().item() > 0
        assert same(a, b), f"step {t}"
        assert same(mods[0].lru_cache.hbm_kv_cache, mods[1].lru_cache.hbm_kv_cache)
        # one plain pass over the final slot contents (the token is already appended)
        lru = mods[1].lru_cache
        pk, pv = lru.views()
        c = w.prompt_tokens + t - w.dram_tokens
        plain = decode_attention(xq[0, 0], pk, pv, mods[1].cache_k[0], mods[1].cache_v[0], c + 1,
                                 None, None)
        assert close(plain, b[0, 0], 1e-2, 1e-2)


@pytest.mark.parametrize("base,kw", [
    ("128k", dict(dram_tokens=16384, local_cache=1024, lru_tokens=4096, top_k_tokens=1024, steps=5)),
    ("1m", dict(dram_tokens=8192, local_cache=512, lru_tokens=2048, top_k_tokens=256, steps=4,
                planted_pages=8)),
    ("cpu", dict(steps=4)),
    ("128k", dict(dram_tokens=8192, local_cache=512, lru_tokens=2048, top_k_tokens=512, steps=4,
                  page_size=32, dtype=torch.float16)),
    ("128k", dict(dram_tokens=4096, local_cache=256, lru_tokens=1024, top_k_tokens=128, steps=4,
                  page_size=8, head_dim=64, n_q_heads=4, n_kv_heads=2)),
    ("cpu", dict(steps=3, head_dim=128)),                       # fp32 rows of 512 bytes: one token per wave
    ("128k", dict(dram_tokens=4096, local_cache=256, lru_tokens=1024, top_k_tokens=256, steps=3,
                  n_q_heads=48, n_kv_heads=48, head_dim=64)),   # more kv heads than stream blocks
])
def test_attention_on_the_page_stream_equals_tail_pass(base, kw):
    """Attending over the streamed pages inside the page stream, or in a pass
    over them afterwards: the same slots, maps and cache rows bit for bit, and
    the same output up to the order of the softmax merge."""
    from dram_attention_amd import DRAMAttention
    from dram_attention_amd.lru_kernel import gather_attend_supported

    w = WORKLOADS[base].scaled(**kw)
    assert gather_attend_supported(w.n_q_heads, w.n_kv_heads, w.head_dim, w.page_size, w.dtype)
    prompt = make_prompt(w, 8)
    mods = []
    for fused in (True, False):
        m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        m.attend_on_page_stream = fused
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        mods.append(m)
    inputs = DecodeInputs(w, prompt.q0, 8)
    atol, rtol = (1e-5, 1e-4) if w.dtype == torch.float32 else (1e-2, 1e-2)
    misses = 0
    for t in range(w.steps):
        xq, xk, xv = (x.to(DEV) for x in inputs.next())
        a = mods[0](xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate")
        b = mods[1](xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate")
        torch.cuda.synchronize()
        misses += mods[0].lru_cache.last_miss_counts().sum().item()
        assert close(a.float(), b.float(), atol, rtol), f"step {t}"
        la, lb = mods[0].lru_cache, mods[1].lru_cache
        assert same(la.hbm_kv_cache, lb.hbm_kv_cache), f"slots, step {t}"
        assert same(la.dram_page_to_hbm_page_mapping, lb.dram_page_to_hbm_page_mapping)
        assert same(mods[0].cache_k, mods[1].cache_k)
    assert misses > 0


@pytest.mark.parametrize("fused", [True, False])
def test_graph_replay_equals_eager_steps(fused):
    """The whole step (selection, LRU, page stream on its side stream, two-phase
    attention, append) captured once and replayed: every replay, with eager work
    and synchronisations in between, matches the CPU oracle step by step (state bit
    for bit, output within tolerance) and gives the eager module's bits and state."""
    from dram_attention_amd import DRAMAttention

    w = WORKLOADS["128k"].scaled(dram_tokens=16384, local_cache=1024, lru_tokens=4096,
                                 top_k_tokens=1024, steps=7)
    prompt = make_prompt(w, 6)
    mods = []
    for _ in range(2):
        m = DRAMAttention(w.steps + 1, w.lru_tokens, w.local_cache, 16, w.top_k_tokens, w.n_kv_heads,
                          w.head_dim, device=DEV, dtype=w.dtype)
        m.attend_on_page_stream = fused   # False: page stream on a side stream, fork/join captured
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        mods.append(m)
    graphed, eager = mods
    o = O.DecodeOracle(w.steps + 1, w.lru_tokens, w.local_cache, 16, w.top_k_tokens, w.n_kv_heads,
                       w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    inputs = DecodeInputs(w, prompt.q0, 6)
    host_steps = [inputs.next() for _ in range(w.steps)]
    steps = [tuple(x.to(DEV) for x in hs) for hs in host_steps]
    xq, xk, xv = (torch.empty_like(x) for x in steps[0])
    pos = torch.tensor([w.prompt_tokens], dtype=torch.int32, device=DEV)

    def feed(t):
        for dst, src in zip((xq, xk, xv), steps[t]):
            dst.copy_(src)

    # step 0 eagerly on both (resolves the pinned mapping, sizes the workspaces)
    feed(0)
    a = graphed(xq, xk, xv, start_pos=pos, stage="generate")
    b = eager(*steps[0], start_pos=w.prompt_tokens, stage="generate")
    assert same(a, b)
    check_step(graphed, o, *host_steps[0], w.prompt_tokens, a, 0, 2e-2, 1e-2)
    pos += 1
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    feed(1)
    with torch.cuda.graph(g):
        out = graphed(xq, xk, xv, start_pos=pos, stage="generate")
        pos += 1
    # capture executes nothing, so the counters still stand at step 1
    for t in range(1, w.steps):
        feed(t)
        g.replay()
        want = eager(*steps[t], start_pos=w.prompt_tokens + t, stage="generate")
        torch.cuda.synchronize()
        assert pos.item() == w.prompt_tokens + t + 1
        assert same(out, want), f"step {t}"
        # the replayed step against the oracle: request list, maps, times, hit mask,
        # slot payload bit for bit, output within the bf16 tolerance
        check_step(graphed, o, *host_steps[t], w.prompt_tokens + t, out, t, 2e-2, 1e-2)
        la, lb = graphed.lru_cache, eager.lru_cache
        assert same(la.hbm_kv_cache, lb.hbm_kv_cache), f"slots, step {t}"
        assert same(la.page_access_time, lb.page_access_time)
        assert same(la.dram_page_to_hbm_page_mapping, lb.dram_page_to_hbm_page_mapping)
        assert la.current_step.item() == lb.current_step.item() == t + 1
        assert la.last_miss_counts().sum().item() > 0
    c = w.prompt_tokens + w.steps - w.dram_tokens
    assert same(graphed.cache_k[0, :c], eager.cache_k[0, :c])


def test_selected_pages_scope_matches_dense_over_the_selection():
    """The Quest-baseline variant (evaluation/quest/model.py:263-316): query head j attends
    over the pages of its own top-k list + local window + new token.  Checked against a
    dense fp32 softmax over exactly those tokens, taken from the prompt by the page
    numbers the step selected; selection and LRU state still follow the oracle (the
    page cache works as in the default scope, only the attended set differs)."""
    from dram_attention_amd import DRAMAttention

    w = WORKLOADS["128k"].scaled(dram_tokens=16384, local_cache=1024, lru_tokens=8192,
                                 top_k_tokens=1024, steps=5)
    prompt = make_prompt(w, 8)
    m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                      w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
    m.attention_scope = "selected"
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    o = O.DecodeOracle(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    inputs = DecodeInputs(w, prompt.q0, 8)
    S, page, rep, kp = w.dram_tokens, w.page_size, w.rep, w.pages_per_q_head
    local_k = [prompt.k[0, S:].float()]
    local_v = [prompt.v[0, S:].float()]
    for t in range(w.steps):
        xq, xk, xv = inputs.next()
        out = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        check_step(m, o, xq, xk, xv, w.prompt_tokens + t, out, t, 2e-2, 1e-2, output=False)
        local_k.append(xk[0].float())
        local_v.append(xv[0].float())
        lk, lv = torch.cat(local_k), torch.cat(local_v)                 # (rows, Hkv, D)
        idx = m.lru_cache._topk_idx.cpu().view(w.n_kv_heads, rep, kp)
        want = torch.empty(w.n_q_heads, w.head_dim)
        for h in range(w.n_kv_heads):
            for r in range(rep):
                tok = (idx[h, r, :, None] * page + torch.arange(page)).reshape(-1)
                k_all = torch.cat([prompt.k[0, tok, h].float(), lk[:, h]])
                v_all = torch.cat([prompt.v[0, tok, h].float(), lv[:, h]])
                q = xq[0, 0, h * rep + r].float()
                p = torch.softmax(k_all @ q / math.sqrt(w.head_dim), 0)
                want[h * rep + r] = p @ v_all
        assert close(out[0, 0].cpu().float(), want, 2e-2, 1e-2), f"step {t}"
    with pytest.raises(RuntimeError, match="Unsupported attention scope"):
        m.attention_scope = "everything"
        x = inputs.next()
        m(x[0].to(DEV), x[1].to(DEV), x[2].to(DEV), start_pos=w.prompt_tokens + w.steps, stage="generate")


def test_token_max_selector_ranks_pages_by_their_best_token():
    """The page selector of the reference's accuracy ceiling
    (evaluation/quest-top-k-oracle/model.py:267-275): score = max over the page's tokens
    of q.k.  Checked against a brute-force fp32 computation from the prompt's keys and
    against the property that makes Quest's bound a bound (best token <= min/max score,
    page by page); ranking, LRU state and payload then follow the oracle fed with
    these scores, and the attended set is each query head's own list."""
    from dram_attention_amd import DRAMAttention
    from dram_attention_amd.topk_selector import TokenMaxTopKSelector

    w = WORKLOADS["128k"].scaled(dram_tokens=8192, local_cache=512, lru_tokens=4096,
                                 top_k_tokens=512, steps=4)
    prompt = make_prompt(w, 11)
    m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                      w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
    m.attention_scope = "selected"
    m.page_selector = "token_max"
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    assert isinstance(m.lru_cache.top_k_selector, TokenMaxTopKSelector)
    o = O.DecodeOracle(w.steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    inputs = DecodeInputs(w, prompt.q0, 11)
    S, page, rep = w.dram_tokens, w.page_size, w.rep
    keys = prompt.k[0, :S].float().view(S // page, page, w.n_kv_heads, w.head_dim)
    for t in range(w.steps):
        xq, xk, xv = inputs.next()
        out = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        q = xq[0, 0].float().view(w.n_kv_heads, rep, w.head_dim)
        best = torch.einsum("pthd,hrd->rhpt", keys, q).amax(-1)          # (rep, Hkv, P)
        bound = O.scores_for_selection(xq, o.min_max)
        assert torch.all(best <= bound + bound.abs() * 2.0 ** -6 + 1e-3), f"bound, step {t}"
        check_step(m, o, xq, xk, xv, w.prompt_tokens + t, out, t, 2e-2, 1e-2, output=False,
                   own_scores=best)
    m.page_selector = "best_guess"
    with pytest.raises(RuntimeError, match="Unsupported page selector"):
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))


def test_page_cache_path_at_32k_all_hits_matches_oracle():
    """configs[1] through the page-cache path: the prefix equals the cache capacity, so
    init_cache would pick the static cache; a page cache built directly over the same
    prefix holds every page from the start, every request hits, no page moves, and
    the step (scores, ordered top-k, LRU times, attention over all slots) matches the
    oracle at full size."""
    from dram_attention_amd import DRAMAttention, DummyCache, LRUCache

    w = WORKLOADS["32k"]
    steps = 6
    prompt = make_prompt(w, 3)
    m = DRAMAttention(steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                      w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    assert isinstance(m.lru_cache, DummyCache)
    S = m.dram_kv_cache_size
    m.lru_cache = LRUCache(prompt.k[0, :S].to(DEV).transpose(0, 1), prompt.v[0, :S].to(DEV).transpose(0, 1),
                           w.page_size, w.top_k_tokens // w.page_size, w.lru_tokens, device=DEV)
    m._workspace = None
    assert m.lru_cache.num_hbm_pages == m.lru_cache.num_dram_pages == 2048
    o = O.DecodeOracle(steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v, force_lru=True)
    inputs = DecodeInputs(w, prompt.q0, 3)
    for t in range(steps):
        xq, xk, xv = inputs.next()
        out = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        check_step(m, o, xq, xk, xv, w.prompt_tokens + t, out, t, 2e-2, 1e-2)
        assert o.last_hit.all() and m.lru_cache.last_miss_counts().sum().item() == 0


@pytest.mark.parametrize("full_size", [False, True])
def test_static_prefix_equals_full_attention(full_size):
    """Prefix within the HBM budget: the static cache path is dense attention over
    the whole sequence (the 32K configuration through init_cache, scaled down and
    at its full size, configs[1])."""
    from dram_attention_amd import DRAMAttention, DummyCache

    w = WORKLOADS["32k"]
    if not full_size:
        w = w.scaled(dram_tokens=4096, local_cache=512, lru_tokens=4096, steps=3)
    prompt = make_prompt(w, 3)
    m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, 16, w.top_k_tokens, w.n_kv_heads,
                      w.head_dim, device=DEV, dtype=w.dtype)
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    assert isinstance(m.lru_cache, DummyCache)
    inputs = DecodeInputs(w, prompt.q0, 3)
    ks, vs = [prompt.k[0]], [prompt.v[0]]
    for t in range(min(w.steps, 4)):
        xq, xk, xv = inputs.next()
        out = m(xq.to(DEV), xk.to(DEV), xv.to(DEV), start_pos=w.prompt_tokens + t, stage="generate")
        ks.append(xk[0]); vs.append(xv[0])
        want, _ = O.attention_partial(xq[0, 0], torch.cat(ks).transpose(0, 1),
                                      torch.cat(vs).transpose(0, 1))
        assert close(out[0, 0].cpu().float(), want, 2e-2, 1e-2)


# ------------------------------------------------------------ full size, by properties
@pytest.mark.parametrize("name,steps", [("128k", 6), ("1m", 64)])
def test_full_size_invariants(name, steps):
    """configs[2] (128K prefix, 8192 pages/head) and configs[4] (1M prefix, 65536
    pages/head, 64 query heads; all of its 64 steps, in which every slot is handed
    out several times over since a step requests as many pages as there are slots)
    at full size: invariants that need no CPU walk, plus attention against a dense
    fp32 computation on the GPU."""
    from dram_attention_amd import DRAMAttention

    w = WORKLOADS[name]
    prompt = make_prompt(w, 0)
    m = DRAMAttention(w.steps, w.lru_tokens, w.local_cache, 16, w.top_k_tokens, w.n_kv_heads,
                      w.head_dim, device=DEV, dtype=w.dtype)
    m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
    dram_dev = m.lru_cache.dram_kv_cache.to(DEV)
    inputs = DecodeInputs(w, prompt.q0, 0)
    for t in range(steps):
        xq, xk, xv = inputs.next()
        xq, xk, xv = xq.to(DEV), xk.to(DEV), xv.to(DEV)
        out = m(xq, xk, xv, start_pos=w.prompt_tokens + t, stage="generate")
        check_invariants(m, w, xq, xk, xv, out, t, dram_dev)
