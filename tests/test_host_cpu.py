"""CPU-side checks: the C-ABI library loads and exports every declared symbol,
host-side argument checking, synthetic workloads, and that nothing computes
without the GPU (the HIP kernels are the only implementation)."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "dram_attention_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(da_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dram_attention_amd import _lib

    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names        # the binding covers the header exactly
    assert lib.da_version() >= 100
    assert lib.da_last_error_string() is not None


def test_workspace_queries_need_no_gpu(lib):
    n = lib.da_decode_attention_workspace_bytes(32, 8, 128, 2, 32768, 4160, 0)
    assert n > 32 * 130 * 4
    assert lib.da_decode_attention_workspace_bytes(32, 8, 128, 2, 32768, 4160, 16384) > n
    assert lib.da_decode_attention_workspace_bytes(32, 8, 24, 2, 1024, 64, 0) == 0   # unsupported dim
    assert lib.da_lru_update_workspace_bytes(8, 1024, 8192, 2048) >= 4


def test_argument_checks_reject_before_any_launch(lib):
    # null pointers / bad geometry are refused on the host: no GPU is touched
    assert lib.da_page_score(None, 0, 0, None, 0, 0, 0, 4, 8, 16, 128, 2, None, 0, 0, 0, 1, None) == -1
    assert b"null" in lib.da_last_error_string()
    assert lib.da_page_score(None, 0, 0, None, 0, 0, 0, 4, 8, 16, 128, 9, None, 0, 0, 0, 1, None) == -1
    assert lib.da_topk_pages(None, 0, 0, 1, 1, 1, 10, 11, None, 0, 0, 0, 1, None, 0, None) == -1
    assert b"exceeds" in lib.da_last_error_string()
    assert lib.da_pages_gather(ctypes.c_void_p(16), 0, 0, ctypes.c_void_p(16), 0, 0, 24,
                               ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16),
                               1, 1, 0, None) == -1


def test_module_surface_and_errors_on_cpu():
    from dram_attention_amd import DRAMAttention

    m = DRAMAttention(max_output_length=64, lru_hbm_cache_size=32 * 1024,
                      local_cache_size=4096 + 512, page_size=16, top_k=4096, n_kv_heads=8,
                      head_dim=128, device="cpu")
    assert m.num_page == 2048 and m.dram_kv_cache_size is None
    assert m.cache_k.shape == (1, 4096 + 512 + 64, 8, 128) and m.cache_v.dtype == torch.bfloat16
    assert set(m.state_dict()) == {"cache_k", "cache_v"}
    x = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="Unsupported stage"):
        m(x, x, x, start_pos=0, stage="invalid")
    x2 = torch.zeros(2, 1, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="Only support batch size 1"):
        m(x2, x2, x2, start_pos=0, stage="prefill")


def test_no_cpu_fallback():
    from dram_attention_amd import LRUCache, max_inner_product

    with pytest.raises(RuntimeError, match="GPU"):
        max_inner_product(torch.zeros(2, 4, 64), torch.zeros(4, 16, 2, 64))
    with pytest.raises(RuntimeError, match="GPU"):
        LRUCache(torch.zeros(2, 64, 8), torch.zeros(2, 64, 8), page_size=16, top_k=2, device="cpu")
    with pytest.raises(AssertionError):
        LRUCache(torch.zeros(2, 60, 8), torch.zeros(2, 60, 8), page_size=16, top_k=2)


def test_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "dram_attention_amd")
    for name in os.listdir(pkg):
        if name.endswith(".py"):
            text = open(os.path.join(pkg, name)).read()
            # the reference's directory evaluation/quest-top-k-oracle and the model variant
            # named after it are the only places the word may appear
            text = text.replace("quest-top-k-oracle", "").replace("quest_oracle", "")
            assert "oracle" not in text, name


def test_max_ip_ref_formula():
    from dram_attention_amd import max_ip_ref
    from oracle import dram_attention_oracle as O

    g = torch.Generator().manual_seed(0)
    q, mm = torch.randn(2, 4, 64, generator=g), torch.randn(4, 16, 2, 64, generator=g)
    assert torch.allclose(max_ip_ref(q, mm), O.max_ip(q, mm), atol=1e-4)


def test_synthetic_workloads():
    from dram_attention_amd.synthetic import WORKLOADS, DecodeInputs, make_prompt
    from oracle import dram_attention_oracle as O

    w = WORKLOADS["128k"]
    assert (w.n_dram_pages, w.n_hbm_pages, w.pages_per_q_head, w.rep) == (8192, 2048, 256, 4)
    assert O.dram_split(w.prompt_tokens, w.local_cache, w.page_size) == w.dram_tokens
    w5 = WORKLOADS["1m"]
    assert (w5.n_dram_pages, w5.n_hbm_pages, w5.pages_per_q_head * w5.rep) == (65536, 4096, 4096)
    c = WORKLOADS["cpu"]
    p1, p2 = make_prompt(c, 0), make_prompt(c, 0)
    assert torch.equal(p1.k, p2.k) and p1.k.shape == (1, c.prompt_tokens, 2, 64)
    assert len(p1.planted) == 4 and all(pg < c.n_dram_pages - c.n_hbm_pages for _, pg in p1.planted)
    # planted pages top the oracle's ranking for their kv group at step 0
    xq, xk, xv = DecodeInputs(c, p1.q0, 0).next()
    mm = O.page_min_max(p1.k[0, : c.dram_tokens].transpose(0, 1), c.n_dram_pages)
    idx = O.lru_index_list(O.select_pages(O.scores_for_selection(xq, mm), 1, c.rep,
                                          c.pages_per_q_head))
    for h, page in p1.planted:
        assert (idx[h] == page).any()
    # ... also with outlier channels and 8 queries per kv head (the 1M layer shape, scaled)
    w8 = w5.scaled(dram_tokens=8192, local_cache=512, lru_tokens=2048, top_k_tokens=256,
                   planted_pages=8)
    p8 = make_prompt(w8, 2)
    xq8, _, _ = DecodeInputs(w8, p8.q0, 2).next()
    mm8 = O.page_min_max(p8.k[0, : w8.dram_tokens].transpose(0, 1), w8.n_dram_pages)
    idx8 = O.lru_index_list(O.select_pages(O.scores_for_selection(xq8, mm8), 1, w8.rep,
                                           w8.pages_per_q_head))
    for h, page in p8.planted:
        assert (idx8[h] == page).any()
    a, b = DecodeInputs(c, p1.q0, 0), DecodeInputs(c, p1.q0, 0)
    for _ in range(3):
        for x, y in zip(a.next(), b.next()):
            assert torch.equal(x, y)


def test_layer_cache_file_round_trip(tmp_path):
    """The chat example's per-layer file: name, keys, shapes and dtype survive a
    write / memory-mapped read, and malformed files are refused."""
    import torch

    from dram_attention_amd import layer_cache_path, load_layer_cache, save_layer_cache

    g = torch.Generator().manual_seed(0)
    k = torch.randn(1, 100, 2, 16, generator=g).bfloat16()
    v = torch.randn(1, 100, 2, 16, generator=g).bfloat16()
    path = save_layer_cache(str(tmp_path), 7, k, v)
    assert path == layer_cache_path(str(tmp_path), 7) and path.endswith("07_cache.pth")
    raw = torch.load(path, weights_only=True)
    assert set(raw) == {"cache_k", "cache_v"} and raw["cache_k"].device.type == "cpu"
    k2, v2 = load_layer_cache(str(tmp_path), 7, device="cpu")
    assert k2.dtype == torch.bfloat16 and torch.equal(k2, k) and torch.equal(v2, v)
    with pytest.raises(ValueError):
        save_layer_cache(str(tmp_path), 8, k[0], v[0])
    torch.save({"cache_k": k}, layer_cache_path(str(tmp_path), 9))
    with pytest.raises(KeyError):
        load_layer_cache(str(tmp_path), 9, device="cpu")


def test_bench_cpu_baseline_is_independent_of_staged_steps():
    """The CPU-baseline leg of bench.py draws its own inputs: it must work for any
    --steps/--warmup of the GPU legs (the driver runs --steps 20 --warmup 5 with the
    default 64 oracle steps) and must report value, cores and the CPU model."""
    import bench
    from dram_attention_amd.synthetic import WORKLOADS

    w = WORKLOADS["128k"].scaled(name="128k/32", dram_tokens=4096, local_cache=256,
                                 lru_tokens=1024, top_k_tokens=256)
    res = bench.cpu_baseline(w, seed=0, steps=64, cfg0_steps=2, cfg0_warmup=1)
    assert res["value"] > 0 and res["cores"] >= 1 and res["kind"] == "port"
    assert res["cpu_model"] and "error" not in res
    assert "64 decode steps" in res["sample"]
    assert res["cfg0"]["value"] > 0
    assert set(res["stage_ms_per_step"]) == {"score", "top_k", "lru", "attention"}


def test_bench_steps_per_graph_choice():
    """Equal graphs where the step count allows: 20 timed steps are one graph of 20,
    64 two of 32, 50 two of 25; 33 has no divisor between 16 and 32 and keeps 32 (+ 1
    single step); the limits hold."""
    import bench

    f = bench.steps_per_graph
    assert [f(n, 32, 32) for n in (20, 64, 256, 50, 48, 100, 33, 7, 1)] == [20, 32, 32, 25, 24, 25, 32, 7, 1]
    assert f(64, 8, 32) == 8 and f(20, 8, 32) == 5 and f(64, 100, 32) == 32 and f(5, 0, 32) == 1
    for n in range(1, 200):
        spg = f(n, 32, 32)
        assert 1 <= spg <= min(n, 32) and (n % spg == 0 or spg == min(n, 32))


def tile_scorer_listing(dot_regs=(1, 145, 142, 146, 143, 147, 144, 148), closing="s_nop 2",
                        mfma="v_mfma_f32_16x16x32_bf16 v[166:169], v[170:173], v[90:93], v[166:169]",
                        loop=False, stray_dot=False):
    """A listing in the shape hipcc -S gives the tile scorer: eight claimed registers, one
    block of eight hand-placed dot products, one MFMA; the arguments doctor it."""
    claimed = (1, 145, 142, 146, 143, 147, 144, 148)
    lines = ["_ZN2da22page_score_tile_kernelILi2ELi4ELi8ELb0EEEvPKcllS2_ilPfllii: ; @kernel",
             "\ts_load_dwordx4 s[0:3], s[4:5], 0x0"]
    lines += [f"\tv_mov_b32 v{r}, 0" for r in claimed]
    lines += [".LBB9_1:", "\tv_perm_b32 v140, v10, v11, s6"]
    lines += [f"\tv_dot2_f32_bf16 v{r}, v{178 + i}, v{157 + i}, 0" for i, r in enumerate(dot_regs)]
    lines += [f"\t{closing}", "\tv_cvt_pk_bf16_f32 v170, v1, v145"]
    if stray_dot:
        lines += ["\tv_dot2_f32_bf16 v1, v140, v157, 0"]
    lines += [f"\t{mfma}"]
    if loop:
        lines += ["\ts_cbranch_scc1 .LBB9_1"]
    lines += ["\tglobal_store_dword v[2:3], v166, off", "\ts_endpgm"]
    return "\n".join(lines) + "\n"


def test_tile_scorer_hazard_check_on_doctored_listings():
    """The build-time check of the tile scorer's hand-placed instructions accepts a
    well-formed listing and refuses each way the rule can break: an MFMA that names a
    hand-written register, a block that is not closed by its wait, a dot product that
    writes an unclaimed register or sits outside a block of eight, a kernel with no
    MFMA or no such kernel at all."""
    from dram_attention_amd.build import check_tile_scorer_listing as check

    assert check(tile_scorer_listing()) == 1
    assert check(tile_scorer_listing() + tile_scorer_listing().replace("ILi2E", "ILi4E")) == 2
    # an MFMA reads v142..v145 as its A operand ahead of a later hand-placed write (the loop)
    with pytest.raises(RuntimeError, match="v142 is written by a hand-placed instruction"):
        check(tile_scorer_listing(mfma="v_mfma_f32_16x16x32_bf16 v[166:169], v[142:145], v[90:93], v[166:169]",
                                  loop=True))
    # the same overlap as the MFMA's destination, straight-line but ahead of the last write
    with pytest.raises(RuntimeError, match="v1 is written by a hand-placed instruction"):
        check(tile_scorer_listing(mfma="v_mfma_f32_16x16x32_bf16 v[0:3], v[170:173], v[90:93], v[0:3]")
              .replace("\tv_perm_b32 v140, v10, v11, s6",
                       "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[170:173], v[90:93], v[0:3]"))
    with pytest.raises(RuntimeError, match="not closed by s_nop 2"):
        check(tile_scorer_listing(closing="s_nop 1"))
    with pytest.raises(RuntimeError, match="never claimed"):
        check(tile_scorer_listing(dot_regs=(1, 145, 142, 146, 143, 147, 144, 149)))
    with pytest.raises(RuntimeError, match="writes a register twice"):
        check(tile_scorer_listing(dot_regs=(1, 145, 142, 146, 143, 147, 144, 144)))
    with pytest.raises(RuntimeError, match="not blocks of eight"):
        check(tile_scorer_listing(stray_dot=True))
    with pytest.raises(RuntimeError, match="no MFMA"):
        check(tile_scorer_listing(mfma="v_add_f32 v166, v170, v171"))
    with pytest.raises(RuntimeError, match="no page_score_tile_kernel"):
        check("_ZN2da21page_score_vec_kernelIfLi4EEEvv:\n\ts_endpgm\n")
    # a claimed register may serve an MFMA once the hand-placed writes are over (no loop)
    assert check(tile_scorer_listing(
        mfma="v_mfma_f32_16x16x32_bf16 v[166:169], v[142:145], v[90:93], v[166:169]")) == 1


def test_bench_roofline_traffic_constant_matches_the_committed_counter_summary():
    """bench.py reports the roofline kernel's HBM bytes per launch from the committed
    counter summary and keeps the same figure as a constant for when the file is not
    beside it: the two must agree, so a refreshed profile cannot leave a stale constant."""
    import bench

    path = os.path.join(ROOT, bench.TRAFFIC_PROFILE)
    assert os.path.exists(path)
    parsed = bench.roofline_traffic_from_profile(path)
    assert parsed is not None and parsed == bench.ROOFLINE_TRAFFIC_BYTES["128k"]
    assert 151.26e6 <= parsed < 1.1 * 151.26e6      # at least the algorithmic bytes, little more
    assert bench.roofline_traffic_from_profile(os.path.join(ROOT, "profiles", "no_such_file.md")) is None


def test_blocked_prefill_fallback_on_cpu_matches_dense_causal_softmax():
    """The torch fallback of the prefill stage (what fp32 or an odd head_dim takes) against
    a dense causal softmax, with a block size small enough to cross several blocks."""
    import math

    import torch

    from dram_attention_amd.dram_attention import causal_prefill_attention

    torch.manual_seed(0)
    S, Hq, Hkv, D = 2500, 4, 2, 16
    q, k, v = torch.randn(1, S, Hq, D), torch.randn(1, S, Hkv, D), torch.randn(1, S, Hkv, D)
    got = causal_prefill_attention(q, k, v, "blocked")
    kk, vv = k.repeat_interleave(Hq // Hkv, 2), v.repeat_interleave(Hq // Hkv, 2)
    sc = torch.einsum("bqhd,bkhd->bhqk", q, kk) / math.sqrt(D)
    sc = sc.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
    want = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(sc, -1), vv)
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
