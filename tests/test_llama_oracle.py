"""Pins the CPU restatement of the Llama-shaped model around the attention path
(closed forms, invariants, published widths), and checks the package's host-side
tables against it.  No GPU needed."""

import math

import torch

from dram_attention_amd import llama as L
from oracle import llama_oracle as M


# ------------------------------------------------------------- rotary embedding
def test_rotary_identity_norm_and_relative_position():
    g = torch.Generator().manual_seed(0)
    D, S = 16, 40
    cis = M.freqs_cis(D, S, 10000.0, False)
    x = torch.randn(1, S, 3, D, generator=g)
    y = M.rotary(x, cis)
    assert torch.equal(y[:, 0], x[:, 0])                      # angle 0 at position 0
    pair_norm = lambda t: t.reshape(1, S, 3, D // 2, 2).norm(dim=-1)
    assert torch.allclose(pair_norm(y), pair_norm(x), atol=1e-5)
    # the same vector placed at positions (i, j) and (i + s, j + s): equal dot products
    q = torch.randn(D, generator=g)
    k = torch.randn(D, generator=g)
    qs = M.rotary(q.expand(1, S, 1, D).contiguous(), cis)[0, :, 0]
    ks = M.rotary(k.expand(1, S, 1, D).contiguous(), cis)[0, :, 0]
    dots = qs @ ks.t()
    for shift in (1, 7, 19):
        assert torch.allclose(dots[5, 2], dots[5 + shift, 2 + shift], atol=1e-4)
        assert torch.allclose(dots[0, 11], dots[shift, 11 + shift], atol=1e-4)
    assert not torch.allclose(dots[5, 2], dots[6, 2], atol=1e-4)


def test_rotary_first_pair_is_a_plane_rotation_by_the_position():
    # frequency 0 is theta**0 = 1: pair 0 at position p turns by p radians
    cis = M.freqs_cis(8, 6, 10000.0, False)
    x = torch.zeros(1, 6, 1, 8)
    x[..., 0] = 1.0
    y = M.rotary(x, cis)
    for p in range(6):
        assert math.isclose(y[0, p, 0, 0].item(), math.cos(p), abs_tol=1e-6)
        assert math.isclose(y[0, p, 0, 1].item(), math.sin(p), abs_tol=1e-6)


def test_scaled_frequencies_three_cases():
    two_pi = 2 * math.pi
    f = torch.tensor([two_pi / 100.0, two_pi / 4096.0, two_pi / 100000.0])
    out = M.scaled_frequencies(f)
    assert out[0].item() == f[0].item()                       # short wavelength: kept
    # wavelength 4096: smooth = (8192/4096 - 1) / 3 = 1/3 -> f * (2/3 / 8 + 1/3) = f * 5/12
    assert math.isclose(out[1].item(), f[1].item() * 5 / 12, rel_tol=1e-5)
    assert math.isclose(out[2].item(), f[2].item() / 8, rel_tol=1e-6)   # long: slowed 8x


def test_swiglu_width_published():
    assert M.swiglu_width(4096, 1024, 1.3) == 14336           # Llama-3 8B
    assert M.swiglu_width(8192, 4096, 1.3) == 28672           # Llama-3 70B
    assert M.swiglu_width(4096, 256, None) == 11008           # Llama-2 7B


def test_rms_norm_closed_form():
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]])                 # mean square 25/4
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    y = M.rms_norm(x, w, 0.0)
    assert torch.allclose(y, torch.tensor([[1.2, -3.2, 0.0, 0.0]]), atol=1e-6)


def test_causal_attention_first_row_and_uniform_case():
    g = torch.Generator().manual_seed(1)
    S, Hq, Hkv, D = 6, 4, 2, 8
    q = torch.randn(1, S, Hq, D, generator=g)
    k = torch.randn(1, S, Hkv, D, generator=g)
    v = torch.randn(1, S, Hkv, D, generator=g)
    out = M.causal_attention(q, k, v)
    # row 0 sees only key 0: the output is v[0] of the query head's kv head
    for h in range(Hq):
        assert torch.allclose(out[0, 0, h], v[0, 0, h // 2], atol=1e-6)
    # zero queries: uniform weights, row i is the mean of v[0..i]
    out0 = M.causal_attention(torch.zeros_like(q), k, v)
    for i in range(S):
        assert torch.allclose(out0[0, i, 3], v[0, : i + 1, 1].mean(0), atol=1e-6)


# ------------------------------------------------- the package's host-side tables
def test_package_rope_matches_the_complex_form():
    g = torch.Generator().manual_seed(2)
    for scaled in (False, True):
        D, S = 64, 300
        table = L.rope_table(D, S, 500000.0, scaled)
        cis = M.freqs_cis(D, S, 500000.0, scaled)
        assert torch.allclose(table[..., 0], cis.real, atol=1e-6)
        assert torch.allclose(table[..., 1], cis.imag, atol=1e-6)
        x = torch.randn(1, 9, 5, D, generator=g)
        assert torch.allclose(L.apply_rope(x, table[100:109]), M.rotary(x, cis[100:109]), atol=1e-6)
        xb = x.bfloat16()
        assert torch.equal(L.apply_rope(xb, table[100:109]), M.rotary(xb, cis[100:109]))


def test_package_scaled_frequencies_cover_all_three_branches():
    # head_dim 128 at theta 5e5 spans wavelengths from 6 to ~3e6 tokens
    f = L.rope_frequencies(128, 500000.0, False)
    want = M.scaled_frequencies(f)
    got = L.rope_frequencies(128, 500000.0, True)
    wl = 2 * math.pi / f
    assert (wl < 2048).any() and (wl > 8192).any() and ((wl >= 2048) & (wl <= 8192)).any()
    assert torch.allclose(got, want, rtol=1e-6, atol=0)


def test_package_widths_and_norm():
    assert L.ffn_hidden_dim(4096, 1024, 1.3) == M.swiglu_width(4096, 1024, 1.3) == 14336
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, 32, generator=g).bfloat16()
    n = L.RMSNorm(32, eps=1e-5)
    with torch.no_grad():
        n.weight.copy_(torch.randn(32, generator=g))
    n = n.bfloat16()
    assert torch.equal(n(x), M.rms_norm(x, n.weight.detach(), 1e-5))
