"""The Llama-shaped model around the attention path on the GPU against its CPU
restatement, and graph-captured decoding against eager decoding."""

import pytest
import torch

from dram_attention_amd import llama as L
from oracle import llama_oracle as M

pytestmark = pytest.mark.gpu


def small_args(dtype, **kw):
    base = dict(dim=256, n_layers=3, n_heads=8, n_kv_heads=2, vocab_size=257, multiple_of=32,
                ffn_dim_multiplier=1.3, rope_theta=500000.0, use_scaled_rope=True,
                lru_hbm_cache_size=256, local_cache_size=128, cache_page_size=16,
                cache_top_k=128, max_output_length=16, max_seq_len=1100, dtype=dtype)
    base.update(kw)
    return L.ModelArgs(**base)


def build(args, seed):
    torch.manual_seed(seed)
    model = L.Transformer(args, device="cuda")
    # norms away from their all-ones start, so that a dropped weight shows
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm.weight"):
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
    return model


def test_fp32_model_matches_cpu_restatement():
    args = small_args(torch.float32)
    model = build(args, 0)
    oracle = M.LlamaOracle(args, model.state_dict())
    g = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, args.vocab_size, (1, 1000), generator=g)
    got = model(prompt.cuda(), 0).cpu()
    want = oracle.forward(prompt, 0)
    assert got.shape == want.shape == (1, 1, args.vocab_size)
    scale = want.abs().max().item()
    assert torch.allclose(got, want, atol=2e-4 * scale, rtol=1e-3), (got - want).abs().max()
    for layer, o in zip(model.layers, oracle.layers):
        assert o.uses_lru and layer.attention.dram_attention.dram_kv_cache_size == 880
    pos = prompt.shape[1]
    for t in range(args.max_output_length - 1):
        token = want.argmax(-1)                      # both sides are fed the same token
        got = model(token.cuda(), pos).cpu()
        want = oracle.forward(token, pos)
        for i, (layer, o) in enumerate(zip(model.layers, oracle.layers)):
            sel = layer.attention.dram_attention.lru_cache._topk_idx.cpu()
            assert torch.equal(sel, o.last_idx), f"page selection, layer {i}, step {t}"
        assert torch.allclose(got, want, atol=2e-4 * scale, rtol=1e-3), \
            (t, (got - want).abs().max().item())
        assert got.argmax(-1).item() == want.argmax(-1).item()
        pos += 1


def test_device_position_equals_host_position():
    args = small_args(torch.bfloat16)
    a, b = build(args, 2), build(args, 2)
    g = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, args.vocab_size, (1, 700), generator=g).cuda()
    la, lb = a(prompt, 0), b(prompt, 0)
    assert torch.equal(la, lb)
    pos = torch.tensor([700], dtype=torch.int32, device="cuda")
    for t in range(6):
        token = la.argmax(-1)
        la = a(token, 700 + t)
        lb = b(token, pos)
        pos += 1
        assert torch.equal(la, lb), f"step {t}"


def test_graphed_greedy_decoding_equals_eager():
    args = small_args(torch.bfloat16)
    a, b = build(args, 4), build(args, 4)
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, args.vocab_size, (1, 900), generator=g).cuda()
    first = a(prompt, 0).argmax(-1).item()
    assert b(prompt, 0).argmax(-1).item() == first
    dec = L.GraphedDecoder(b, 900, first)
    token = torch.tensor([[first]], device="cuda")
    for t in range(10):
        want = a(token, 900 + t)
        got = dec.step()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"step {t}"
        token = want.argmax(-1)
        assert torch.equal(dec.token, token)
    assert dec.graph is not None and dec.pos.item() == 910


def test_layer_files_feed_the_model(tmp_path):
    from dram_attention_amd import save_layer_cache

    args = small_args(torch.bfloat16)
    a, b = build(args, 6), build(args, 6)
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, args.vocab_size, (1, 640), generator=g).cuda()
    la = a(prompt, 0)
    # capture every layer's prompt K/V the way the chat example's prefill phase does
    kv = []
    hooks = [layer.attention.dram_attention.register_forward_pre_hook(
        lambda mod, inp, store=kv: store.append((inp[1].cpu(), inp[2].cpu())))
        for layer in b.layers]
    b(prompt, 0)
    for h in hooks:
        h.remove()
    for i, (k, v) in enumerate(kv):
        save_layer_cache(str(tmp_path), i, k, v)
    c = build(args, 6)
    assert c.init_cache_from_files(str(tmp_path)) == 640
    token = la.argmax(-1)
    assert torch.equal(c(token, 640), a(token, 640))


def test_model_variants_full_quest_and_quest_oracle():
    """The reference's comparison models on the same kernels.  "full" keeps the whole
    prefix in HBM behind the static cache (evaluation/full-attention/model.py:201-215):
    its logits follow the CPU restatement of the model with a cache budget that holds
    everything.  "quest" attends over the selected pages only
    (evaluation/quest/model.py:263-316; the attention itself is checked against a dense
    computation in test_gpu_module.py): here, that the model runs it in every layer and
    that it sees fewer tokens than "dram" does.  "quest_oracle" is "quest" with pages
    ranked by their best token (evaluation/quest-top-k-oracle/model.py:267-275; the
    selector is checked in test_gpu_module.py)."""
    from dram_attention_amd import DummyCache, LRUCache
    from dram_attention_amd.topk_selector import TokenMaxTopKSelector

    g = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, 257, (1, 1000), generator=g)
    args = small_args(torch.float32, attention_variant="full")
    model = build(args, 0)
    oracle = M.LlamaOracle(small_args(torch.float32, lru_hbm_cache_size=1100), model.state_dict())
    got, want = model(prompt.cuda(), 0).cpu(), oracle.forward(prompt, 0)
    scale = want.abs().max().item()
    pos = 1000
    for t in range(5):
        assert torch.allclose(got, want, atol=2e-4 * scale, rtol=1e-3), (t, (got - want).abs().max())
        token = want.argmax(-1)
        got, want = model(token.cuda(), pos).cpu(), oracle.forward(token, pos)
        pos += 1
    for layer, o in zip(model.layers, oracle.layers):
        assert isinstance(layer.attention.dram_attention.lru_cache, DummyCache) and not o.uses_lru
    # 8 pages per query head, 32 requests per kv head, 32 slots
    outs = {}
    for variant in ("dram", "quest", "quest_oracle"):
        model = build(small_args(torch.float32, attention_variant=variant, lru_hbm_cache_size=512), 0)
        out = model(prompt.cuda(), 0)
        for layer in model.layers:
            a = layer.attention.dram_attention
            assert isinstance(a.lru_cache, LRUCache)
            assert a.attention_scope == ("resident" if variant == "dram" else "selected")
            assert isinstance(a.lru_cache.top_k_selector, TokenMaxTopKSelector) == (variant == "quest_oracle")
        outs[variant] = model(out.argmax(-1), 1000).cpu()
        assert torch.isfinite(outs[variant]).all()
    assert (outs["dram"] - outs["quest"]).abs().max().item() > 1e-4 * scale
    with pytest.raises(AssertionError):
        small_args(torch.float32, attention_variant="sparse")


def test_recall_harness_on_a_checkpoint_directory(tmp_path):
    """The evaluation driver end to end on a small random checkpoint written the way
    the Llama-3 download lays it out (params.json + consolidated.00.pth): the loaded
    model decodes the token sequence the CPU restatement of the driver decodes from
    the same weights (page-aligned prefill of 992 of 1003 prefix tokens, 11 + 9 forced
    prompt tokens, then free running), for the paged model and, against the restatement
    with a cache that holds everything, for the full-attention variant; then two
    generated key-value items through tokenizer, model, answer extraction and results
    file."""
    import json

    from dram_attention_amd import LRUCache
    from dram_attention_amd import evaluate as E

    tok = E.ByteTokenizer()
    params = dict(dim=256, n_layers=2, n_heads=8, n_kv_heads=2, vocab_size=tok.n_words,
                  multiple_of=32, ffn_dim_multiplier=1.3, norm_eps=1e-5, rope_theta=500000.0,
                  use_scaled_rope=True)
    cache = dict(lru_hbm_cache_size=256, cache_top_k=128, cache_page_size=16,
                 local_cache_size=128 + 64, max_output_length=64, max_seq_len=1100)
    donor = build(L.ModelArgs(dtype=torch.float32, **params, **cache), 7)
    (tmp_path / "params.json").write_text(json.dumps(params))
    weights = {k: v.detach().cpu() for k, v in donor.named_parameters()}
    weights["rope.freqs"] = torch.zeros(16)         # older checkpoints carry the rope table
    torch.save(weights, tmp_path / "consolidated.00.pth")

    g = torch.Generator().manual_seed(11)
    prefix = torch.randint(0, 256, (1003,), generator=g).tolist()
    suffix = torch.randint(0, 256, (9,), generator=g).tolist()
    for variant, oracle_cache in (("dram", 256), ("full", 1100)):
        model = E.load_model(str(tmp_path), 1100, variant=variant, top_k=128, page_size=16,
                             local_attn_window=128, local_margin=64, lru_hbm_cache_size=256,
                             max_output_length=64, dtype=torch.float32)
        assert model.params.local_cache_size == 128 + 64 and model.params.cache_top_k == 128
        for (name, p), (_, q) in zip(model.named_parameters(), donor.named_parameters()):
            assert torch.equal(p, q), name
        got = E.generate(model, prefix, suffix, 24, page_size=16, stop_tokens=tok.stop_tokens,
                         special_start=tok.special_start)
        args = L.ModelArgs(dtype=torch.float32, **params, **dict(cache, lru_hbm_cache_size=oracle_cache))
        want = M.greedy_generate(M.LlamaOracle(args, donor.state_dict()), prefix, suffix, 24, 16,
                                 tok.stop_tokens, tok.special_start)
        assert got == want and 1 <= len(got) <= 23, (variant, got, want)
        a = model.layers[0].attention.dram_attention
        assert a.dram_kv_cache_size == 816 and isinstance(a.lru_cache, LRUCache) == (variant == "dram")

    # the question line is ~100 byte tokens: they, the completion and the tokens behind the
    # last whole page of the prefix all land in the local cache's room for new rows
    model = E.load_model(str(tmp_path), 1100, top_k=128, page_size=16, local_attn_window=128,
                         local_margin=64, lru_hbm_cache_size=256, max_output_length=192,
                         dtype=torch.float32)
    items = E.synthetic_niah(2, 14, seed=3)
    path = tmp_path / E.results_file_name(1100, "smoke")
    recall = E.evaluate_items(model, tok, items, page_size=16, results_path=str(path), max_gen_len=8)
    rows = [json.loads(line) for line in path.read_text().splitlines()]
    assert [r["index"] for r in rows] == [0, 1] and all(r["recall"] in (0, 1) for r in rows)
    assert recall == sum(r["recall"] for r in rows) / 2
    assert "1100 |" in E.report(str(tmp_path))
    del weights["norm.weight"]
    torch.save(weights, tmp_path / "consolidated.00.pth")
    with pytest.raises(KeyError, match="norm.weight"):
        E.load_model(str(tmp_path), 1100, dtype=torch.float32)
    (tmp_path / "params.json").write_text(json.dumps(dict(params, hidden=3)))
    with pytest.raises(ValueError, match="hidden"):
        E.load_model(str(tmp_path), 1100)
