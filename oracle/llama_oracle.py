"""CPU restatement of the Llama-3 shaped model the reference wraps around
DRAMAttention (evaluation/dram-attention/model.py).  TEST INFRASTRUCTURE ONLY:
imported by tests/ as the checker of dram_attention_amd/llama.py, never by the
package.

It follows the reference's formulation, not the package's: rotary embedding
as a complex product (model.py:108-136), the frequency scaling as the
reference's per-frequency branches (:81-105), RMSNorm (:66-78), SwiGLU
(:233-234), blocks and logits (:265-274, :305-317).  The attention layer is
``DecodeOracle`` plus a direct causal softmax for the prefill (what
``flash_attn_func(causal=True)`` computes, dram_attention.py:136).

What pins it (tests/test_llama_oracle.py): rotary embedding is the identity at
position 0, preserves norms, and makes q.k a function of the position difference
only; the scaled frequencies against the three hand-computed cases of the rule;
the SwiGLU width against the published Llama-3 widths (8B: 14336, 70B: 28672);
RMSNorm against the formula on a vector whose answer is known in closed form.
``greedy_generate`` (the evaluation driver's loop, evaluate.py:75-121) against a
scripted model whose next token is a known function of the last one: the
page-aligned prefill length, the forced prompt tokens, both stop rules and the
returned slice are then fixed by hand.
"""
import math
from typing import Dict, List, Optional

import torch

from .dram_attention_oracle import DecodeOracle


def scaled_frequencies(freqs: torch.Tensor) -> torch.Tensor:
    """model.py:81-105: per frequency, by wavelength against 8192/1 and 8192/4."""
    out = []
    for f in freqs:  # 0-d tensors: the arithmetic stays in the tensor's precision
        wavelen = 2 * math.pi / f
        if wavelen < 8192 / 4:
            out.append(f)
        elif wavelen > 8192 / 1:
            out.append(f / 8)
        else:
            smooth = (8192 / wavelen - 1) / (4 - 1)
            out.append((1 - smooth) * f / 8 + smooth * f)
    return torch.stack(out).to(freqs.dtype)


def freqs_cis(head_dim: int, end: int, theta: float, use_scaled: bool) -> torch.Tensor:
    """model.py:108-117: complex64 (end, head_dim/2), unit modulus, angle = pos*freq."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    if use_scaled:
        freqs = scaled_frequencies(freqs)
    angle = torch.outer(torch.arange(end, dtype=torch.float32), freqs)
    return torch.polar(torch.ones_like(angle), angle)


def rotary(x: torch.Tensor, cis: torch.Tensor) -> torch.Tensor:
    """model.py:126-136: x (1,S,H,D) as D/2 complex numbers times cis (S,D/2)."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    return torch.view_as_real(xc * cis[None, :, None, :]).flatten(3).type_as(x)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """model.py:66-78."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x) * weight


def swiglu_width(dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float]) -> int:
    """model.py:207-220 with hidden_dim = 4*dim (:255)."""
    hidden = int(2 * (4 * dim) / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


def causal_attention(xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor) -> torch.Tensor:
    """(1,S,Hq,D), (1,S,Hkv,D) x2 -> (1,S,Hq,D): softmax over keys j <= i, scale D**-0.5,
    query head j on kv head j // rep; fp32 arithmetic, result in xq's dtype."""
    _, S, Hq, D = xq.shape
    Hkv = xk.shape[2]
    rep = Hq // Hkv
    q = xq[0].float().transpose(0, 1).reshape(Hkv, rep, S, D)
    k = xk[0].float().transpose(0, 1)
    v = xv[0].float().transpose(0, 1)
    s = torch.einsum("hrid,hjd->hrij", q, k) / math.sqrt(D)
    s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
    out = torch.einsum("hrij,hjd->hrid", torch.softmax(s, dim=-1), v)
    return out.reshape(Hq, S, D).transpose(0, 1)[None].to(xq.dtype)


class LlamaOracle:
    """Runs a state dict with the reference's parameter names on the CPU."""

    def __init__(self, args, state: Dict[str, torch.Tensor]):
        self.a = args
        self.w = {k: v.detach().cpu() for k, v in state.items()}
        self.head_dim = args.dim // args.n_heads
        self.cis = freqs_cis(self.head_dim, args.max_seq_len * 2, args.rope_theta,
                             args.use_scaled_rope)
        self.layers = [
            DecodeOracle(args.max_output_length, args.lru_hbm_cache_size, args.local_cache_size,
                         args.cache_page_size, args.cache_top_k, args.n_kv_heads, self.head_dim,
                         dtype=args.dtype)
            for _ in range(args.n_layers)
        ]

    def _linear(self, x, name):
        return x @ self.w[name].t()

    def _attention(self, i, x, start_pos, cis):
        a, D = self.a, self.head_dim
        p = f"layers.{i}.attention."
        S = x.shape[1]
        xq = self._linear(x, p + "wq.weight").view(1, S, a.n_heads, D)
        xk = self._linear(x, p + "wk.weight").view(1, S, a.n_kv_heads, D)
        xv = self._linear(x, p + "wv.weight").view(1, S, a.n_kv_heads, D)
        xq, xk = rotary(xq, cis), rotary(xk, cis)
        if S > 1 and start_pos == 0:
            out = causal_attention(xq, xk, xv)
            self.layers[i].init_cache(xk, xv)
        else:
            out = self.layers[i].generate(xq, xk, xv, start_pos)
        return self._linear(out.reshape(1, S, -1), p + "wo.weight")

    def forward(self, tokens: torch.Tensor, start_pos: int) -> torch.Tensor:
        a = self.a
        S = tokens.shape[1]
        h = self.w["tok_embeddings.weight"][tokens]
        cis = self.cis[start_pos: start_pos + S]
        for i in range(a.n_layers):
            p = f"layers.{i}."
            h = h + self._attention(i, rms_norm(h, self.w[p + "attention_norm.weight"], a.norm_eps),
                                    start_pos, cis)
            g = rms_norm(h, self.w[p + "ffn_norm.weight"], a.norm_eps)
            gate = torch.nn.functional.silu(self._linear(g, p + "feed_forward.w1.weight"))
            h = h + self._linear(gate * self._linear(g, p + "feed_forward.w3.weight"),
                                 p + "feed_forward.w2.weight")
        h = rms_norm(h[:, -1:, :], self.w["norm.weight"], a.norm_eps)
        return self._linear(h, "output.weight").float()


def greedy_generate(oracle: "LlamaOracle", prefix: List[int], suffix: List[int], max_gen_len: int,
                    page_size: int, stop_tokens, special_start: int) -> List[int]:
    """The evaluation driver's decoding loop on the CPU model
    (evaluation/dram-attention/evaluate.py:75-121): the prefix cut to whole pages is
    the prefill; from there on one token per call, where position p + 1 takes the
    prompt's token if the prompt reaches that far and the argmax of the logits at p
    otherwise; the loop ends after writing a stop token or a token of the special
    range, and the result is what lies between the end of the prompt and the last
    position fed to the model."""
    prompt = list(prefix) + list(suffix)
    total = min(oracle.a.max_seq_len, len(prompt) + max_gen_len)
    seq = torch.full((total,), -1, dtype=torch.long)
    seq[: len(prompt)] = torch.tensor(prompt, dtype=torch.long)
    given = seq >= 0
    start = len(prefix) // page_size * page_size
    logits = oracle.forward(seq[None, :start], 0)
    if not given[start]:
        seq[start] = logits[0, -1].argmax()
    last_fed = start
    for p in range(start, total - 1):
        last_fed = p
        logits = oracle.forward(seq[None, p: p + 1], p)
        if not given[p + 1]:
            seq[p + 1] = logits[0, -1].argmax()
        t = int(seq[p + 1])
        if t in stop_tokens or t >= special_start:
            break
    return seq[len(prompt): last_fed + 1].tolist()
