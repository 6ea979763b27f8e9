"""The prefill stage: causal attention over the prompt (reference
dram_attention/dram_attention.py:136, flash_attn_func(causal=True)).

The reference's own test of this stage checks the output's shape only
(dram_attention_test.py:31-60), and flash-attn is a third-party library that is not
here, so the values are held against the closed form: a dense fp32 causal softmax
over the same bf16/fp16 inputs, within atol 2e-2 / rtol 1e-2 (the tolerance of the
attention contract), through the C ABI (da_prefill_attention) and through
DRAMAttention.forward(stage="prefill") with each of its backends."""

import math

import pytest
import torch

from tests.util import close, same

pytestmark = pytest.mark.gpu
DEV = "cuda"
ATOL, RTOL = 2e-2, 1e-2


def dense_causal(xq, xk, xv, scale=None):
    """fp32 softmax(q k^T * scale + causal mask) v per kv head; returns (out (1,S,Hq,D) fp32,
    lse (Hq,S) fp32)."""
    _, S, Hq, D = xq.shape
    Hkv = xk.shape[2]
    rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    out = torch.empty(1, S, Hq, D, dtype=torch.float32, device=xq.device)
    lse = torch.empty(Hq, S, dtype=torch.float32, device=xq.device)
    mask = torch.ones(S, S, dtype=torch.bool, device=xq.device).tril_()
    for h in range(Hkv):
        q = xq[0, :, h * rep:(h + 1) * rep].float().transpose(0, 1)          # (rep, S, D)
        s = torch.matmul(q, xk[0, :, h].float().t()) * scale                  # (rep, S, S)
        s.masked_fill_(~mask, float("-inf"))
        lse[h * rep:(h + 1) * rep] = torch.logsumexp(s, dim=-1)
        o = torch.matmul(torch.softmax(s, dim=-1), xv[0, :, h].float())       # (rep, S, D)
        out[0, :, h * rep:(h + 1) * rep] = o.transpose(0, 1)
    return out, lse


def draw(S, Hq, Hkv, D, dtype, seed, spread=1.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    xq = (torch.randn(1, S, Hq, D, device=DEV, generator=g) * spread).to(dtype)
    xk = (torch.randn(1, S, Hkv, D, device=DEV, generator=g) * spread).to(dtype)
    xv = torch.randn(1, S, Hkv, D, device=DEV, generator=g).to(dtype)
    return xq, xk, xv


@pytest.mark.parametrize("S,Hq,Hkv,D,dtype", [
    (4096 + 517, 32, 8, 128, torch.bfloat16),     # the layer shape, a ragged length
    (1, 4, 1, 128, torch.bfloat16),
    (5, 8, 2, 128, torch.bfloat16),
    (31, 4, 4, 64, torch.bfloat16),
    (33, 4, 2, 128, torch.float16),
    (63, 2, 2, 128, torch.bfloat16),
    (64, 4, 1, 128, torch.bfloat16),
    (65, 8, 8, 64, torch.float16),
    (127, 3, 1, 128, torch.bfloat16),             # rep 3: one head per workgroup
    (129, 6, 3, 128, torch.bfloat16),             # rep 2
    (200, 8, 1, 64, torch.bfloat16),              # rep 8: two workgroups per row block
    (1000, 16, 2, 128, torch.float16),
    (2048, 8, 2, 64, torch.bfloat16),
])
def test_prefill_attention_matches_dense_causal_softmax(S, Hq, Hkv, D, dtype):
    from dram_attention_amd.dram_attention import prefill_attention

    xq, xk, xv = draw(S, Hq, Hkv, D, dtype, S + Hq)
    lse = torch.empty(Hq, S, dtype=torch.float32, device=DEV)
    out = prefill_attention(xq, xk, xv, lse=lse)
    want, want_lse = dense_causal(xq, xk, xv)
    assert out.shape == xq.shape and out.dtype == dtype
    assert close(out.float(), want, ATOL, RTOL)
    assert close(lse, want_lse, 1e-3, 1e-4)


def test_prefill_attention_takes_strided_views_and_peaked_scores():
    """Rows taken out of a fused (S, Hq + 2 Hkv, D) projection, and scores spread widely
    enough that the running maximum moves many times."""
    from dram_attention_amd.dram_attention import prefill_attention

    S, Hq, Hkv, D = 777, 8, 2, 128
    g = torch.Generator(device=DEV).manual_seed(3)
    qkv = (torch.randn(1, S, Hq + 2 * Hkv, D, device=DEV, generator=g) * 3.0).bfloat16()
    xq, xk, xv = qkv[:, :, :Hq], qkv[:, :, Hq:Hq + Hkv], qkv[:, :, Hq + Hkv:]
    out = prefill_attention(xq, xk, xv, scale=0.5)
    want, _ = dense_causal(xq, xk, xv, scale=0.5)
    assert close(out.float(), want, ATOL, RTOL)
    # the first row attends to itself only: its output is its value row, exactly
    assert same(out[0, 0].view(Hkv, Hq // Hkv, D), xv[0, 0][:, None].expand(-1, Hq // Hkv, -1))


def test_prefill_attention_at_the_headline_prompt_length_on_sampled_rows():
    """configs[2]'s prompt (135 152 tokens, 32 q / 8 kv heads, D 128, bf16) through the
    kernel once; rows sampled from the first, a middle and the last blocks, and around
    tile boundaries, are held against a dense fp32 causal softmax over all their keys."""
    from dram_attention_amd.dram_attention import prefill_attention

    S, Hq, Hkv, D = 131072 + 4096 - 16, 32, 8, 128
    rep = Hq // Hkv
    xq, xk, xv = draw(S, Hq, Hkv, D, torch.bfloat16, 5)
    lse = torch.empty(Hq, S, dtype=torch.float32, device=DEV)
    out = prefill_attention(xq, xk, xv, lse=lse)
    rows = torch.tensor(sorted(set(
        list(range(0, 70)) + list(range(65500, 65570)) + [4095, 4096, 4097, 100000, 100063, 100064, 131071, 131072]
        + list(range(S - 40, S)))), device=DEV)
    scale = 1.0 / math.sqrt(D)
    for h in range(Hkv):
        q = xq[0, rows, h * rep:(h + 1) * rep].float().transpose(0, 1)       # (rep, R, D)
        s_ = torch.matmul(q, xk[0, :, h].float().t()) * scale                 # (rep, R, S)
        keys = torch.arange(S, device=DEV)
        s_.masked_fill_(keys[None, None, :] > rows[None, :, None], float("-inf"))
        want = torch.matmul(torch.softmax(s_, dim=-1), xv[0, :, h].float()).transpose(0, 1)   # (R, rep, D)
        assert close(out[0, rows, h * rep:(h + 1) * rep].float(), want, ATOL, RTOL)
        assert close(lse[h * rep:(h + 1) * rep][:, rows], torch.logsumexp(s_, dim=-1), 1e-3, 1e-4)
    assert torch.isfinite(out.float()).all()


def test_prefill_attention_rejects_what_the_kernel_does_not_cover():
    from dram_attention_amd.dram_attention import (causal_prefill_attention, prefill_attention,
                                                   prefill_attention_supported)

    xq, xk, xv = draw(16, 4, 2, 128, torch.float32, 0)
    assert not prefill_attention_supported(xq)
    with pytest.raises(RuntimeError, match="head_dim 64 or 128"):
        prefill_attention(xq, xk, xv)
    xq, xk, xv = draw(16, 4, 2, 32, torch.bfloat16, 0)
    with pytest.raises(RuntimeError, match="head_dim 64 or 128"):
        prefill_attention(xq, xk, xv)
    with pytest.raises(RuntimeError, match="Unsupported prefill backend"):
        causal_prefill_attention(xq, xk, xv, backend="triton")
    # "auto" still answers for such shapes, through torch
    xq, xk, xv = draw(100, 4, 2, 32, torch.float32, 1)
    want, _ = dense_causal(xq, xk, xv)
    assert close(causal_prefill_attention(xq, xk, xv), want, 1e-4, 1e-4)


@pytest.mark.parametrize("backend", ["native", "sdpa", "blocked", "auto"])
def test_module_prefill_stage_values_at_the_layer_shape(backend):
    """DRAMAttention.forward(stage="prefill") at bf16, 32 q / 8 kv heads, D 128, a length
    that is no multiple of the block sizes: the returned output against the dense fp32
    causal softmax, with every backend the module can attend with."""
    from dram_attention_amd import DRAMAttention, LRUCache

    S = 4096 + 517
    xq, xk, xv = draw(S, 32, 8, 128, torch.bfloat16, 11)
    m = DRAMAttention(max_output_length=4, lru_hbm_cache_size=1024, local_cache_size=512,
                      page_size=16, top_k=256, n_kv_heads=8, head_dim=128, device=DEV)
    m.prefill_backend = backend
    try:
        out = m(xq, xk, xv, start_pos=0, stage="prefill")
    except RuntimeError as exc:
        if backend == "sdpa":
            pytest.skip(f"torch's fused attention refuses this shape here: {exc}")
        raise
    want, _ = dense_causal(xq, xk, xv)
    assert out.shape == xq.shape and out.dtype == torch.bfloat16
    assert close(out.float(), want, ATOL, RTOL)
    assert isinstance(m.lru_cache, LRUCache) and m.dram_kv_cache_size == (S - 512 + 16) // 16 * 16
