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
