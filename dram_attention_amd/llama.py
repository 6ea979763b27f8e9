"""Llama-3 shaped decoder whose attention layers are ``DRAMAttention``.

Counterpart of the model the reference evaluates with
(evaluation/dram-attention/model.py:28-317): same ``ModelArgs`` fields, same
module and parameter names (``tok_embeddings``, ``layers.N.attention.wq`` …
``norm``, ``output``), so a Llama-3 checkpoint's state dict loads unchanged,
and the same ``forward(tokens, start_pos)`` contract: a call with more than one
token at position 0 is the prefill (it builds every layer's page cache), any
other call decodes one token.  ``start_pos`` of a decode call may be an int32
device tensor, which keeps the step free of host reads so that it can be
captured in a HIP graph the way examples/long-qa-chat/chat.py:238-249 does.

Everything here is plumbing around the attention path (projections, rotary
embedding, norms, SwiGLU): plain torch ops on the GPU.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .dram_attention import DRAMAttention


@dataclass
class ModelArgs:
    """Model and cache geometry; defaults are Llama-3.1-8B with the reference's
    cache settings (evaluation/dram-attention/model.py:28-63)."""

    dim: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: Optional[int] = None
    vocab_size: int = -1
    multiple_of: int = 256
    ffn_dim_multiplier: Optional[float] = None
    norm_eps: float = 1e-5
    rope_theta: float = 500000
    use_scaled_rope: bool = False
    lru_hbm_cache_size: int = 32 * 1024
    local_cache_size: int = 4 * 1024 + 1024
    cache_page_size: int = 16
    cache_top_k: int = 4 * 1024
    max_output_length: int = 128
    max_batch_size: int = 1
    max_seq_len: int = 2048
    dtype: torch.dtype = torch.bfloat16
    # which of the reference's evaluated models the attention layers form:
    #   "dram"  DRAM Attention (evaluation/dram-attention/model.py)
    #   "quest" attention over the selected pages only (evaluation/quest/model.py:263-316)
    #   "quest_oracle" the same with pages ranked by their best token instead of the
    #           min/max bound (evaluation/quest-top-k-oracle/model.py:267-275)
    #   "full"  dense attention over the whole cache (evaluation/full-attention/model.py:201-215)
    attention_variant: str = "dram"

    def __post_init__(self):
        if self.n_kv_heads is None:
            self.n_kv_heads = self.n_heads
        assert self.n_kv_heads <= self.n_heads
        assert self.n_heads % self.n_kv_heads == 0
        assert self.dim % self.n_heads == 0
        assert self.attention_variant in ("dram", "quest", "quest_oracle", "full")

    @property
    def head_dim(self) -> int:
        return self.dim // self.n_heads


def ffn_hidden_dim(dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float]) -> int:
    """Width of the SwiGLU layer: 2/3 of 4*dim, scaled, rounded up to ``multiple_of``
    (evaluation/dram-attention/model.py:216-220)."""
    hidden = int(2 * (4 * dim) / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


def rope_frequencies(head_dim: int, theta: float, use_scaled: bool) -> torch.Tensor:
    """The head_dim/2 rotation frequencies; with ``use_scaled`` the Llama-3.1
    long-context rule: wavelengths above 8192 slowed 8x, below 2048 kept, a linear
    blend between (evaluation/dram-attention/model.py:81-105)."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    if not use_scaled:
        return freqs
    scale, low, high, old_len = 8.0, 1.0, 4.0, 8192.0
    wavelen = 2 * math.pi / freqs
    smooth = ((old_len / wavelen - low) / (high - low)).clamp(0.0, 1.0)
    # smooth is 0 for wavelengths above old_len/low and 1 below old_len/high
    return (1 - smooth) * freqs / scale + smooth * freqs


def rope_table(head_dim: int, end: int, theta: float, use_scaled: bool,
               device=None) -> torch.Tensor:
    """(end, head_dim/2, 2) fp32: cos and sin of position * frequency."""
    angle = torch.outer(torch.arange(end, dtype=torch.float32),
                        rope_frequencies(head_dim, theta, use_scaled))
    return torch.stack((angle.cos(), angle.sin()), dim=-1).to(device)


def apply_rope(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """Rotate adjacent channel pairs of x (1, S, H, D) by the table rows (S, D/2, 2);
    arithmetic in fp32, result in x's dtype (the complex product of
    evaluation/dram-attention/model.py:126-136 written out)."""
    pairs = x.float().unflatten(-1, (-1, 2))
    even, odd = pairs[..., 0], pairs[..., 1]
    cos, sin = rows[None, :, None, :, 0], rows[None, :, None, :, 1]
    out = torch.stack((even * cos - odd * sin, even * sin + odd * cos), dim=-1)
    return out.flatten(-2).to(x.dtype)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        x32 = x.float()
        normed = x32 * torch.rsqrt(x32.square().mean(-1, keepdim=True) + self.eps)
        return normed.to(x.dtype) * self.weight


class Attention(nn.Module):
    """Projections and rotary embedding around DRAMAttention
    (evaluation/dram-attention/model.py:138-205)."""

    def __init__(self, args: ModelArgs, device="cuda"):
        super().__init__()
        self.n_heads, self.n_kv_heads, self.head_dim = args.n_heads, args.n_kv_heads, args.head_dim
        self.wq = nn.Linear(args.dim, args.n_heads * self.head_dim, bias=False)
        self.wk = nn.Linear(args.dim, args.n_kv_heads * self.head_dim, bias=False)
        self.wv = nn.Linear(args.dim, args.n_kv_heads * self.head_dim, bias=False)
        self.wo = nn.Linear(args.n_heads * self.head_dim, args.dim, bias=False)
        # "full": a page cache as large as the longest sequence keeps the whole prefix
        # in HBM (init_cache then picks the static cache: plain dense attention)
        budget = (max(args.lru_hbm_cache_size, args.max_seq_len)
                  if args.attention_variant == "full" else args.lru_hbm_cache_size)
        self.dram_attention = DRAMAttention(
            max_output_length=args.max_output_length,
            lru_hbm_cache_size=budget,
            local_cache_size=args.local_cache_size,
            page_size=args.cache_page_size,
            top_k=args.cache_top_k,
            n_kv_heads=args.n_kv_heads,
            head_dim=self.head_dim,
            device=device,
            dtype=args.dtype,
        )
        if args.attention_variant in ("quest", "quest_oracle"):
            self.dram_attention.attention_scope = "selected"
        if args.attention_variant == "quest_oracle":
            self.dram_attention.page_selector = "token_max"

    def forward(self, x: torch.Tensor, start_pos, rope_rows: torch.Tensor):
        bsz, seqlen, _ = x.shape
        xq = self.wq(x).view(bsz, seqlen, self.n_heads, self.head_dim)
        xk = self.wk(x).view(bsz, seqlen, self.n_kv_heads, self.head_dim)
        xv = self.wv(x).view(bsz, seqlen, self.n_kv_heads, self.head_dim)
        xq, xk = apply_rope(xq, rope_rows), apply_rope(xk, rope_rows)
        prefill = seqlen > 1 and not isinstance(start_pos, torch.Tensor) and start_pos == 0
        out = self.dram_attention(xq, xk, xv, start_pos=start_pos,
                                  stage="prefill" if prefill else "generate")
        return self.wo(out.reshape(bsz, seqlen, -1))


class FeedForward(nn.Module):
    ROWS_PER_PASS = 8192  # a long prompt goes through in slices (model.py:236-245)

    def __init__(self, dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float]):
        super().__init__()
        hidden = ffn_hidden_dim(dim, multiple_of, ffn_dim_multiplier)
        self.w1 = nn.Linear(dim, hidden, bias=False)
        self.w2 = nn.Linear(hidden, dim, bias=False)
        self.w3 = nn.Linear(dim, hidden, bias=False)

    def forward(self, x):
        if x.shape[1] <= self.ROWS_PER_PASS:
            return self.w2(F.silu(self.w1(x)) * self.w3(x))
        return torch.cat([self.w2(F.silu(self.w1(c)) * self.w3(c))
                          for c in x.split(self.ROWS_PER_PASS, dim=1)], dim=1)


class TransformerBlock(nn.Module):
    def __init__(self, layer_id: int, args: ModelArgs, device="cuda"):
        super().__init__()
        self.layer_id = layer_id
        self.attention = Attention(args, device)
        self.feed_forward = FeedForward(args.dim, args.multiple_of, args.ffn_dim_multiplier)
        self.attention_norm = RMSNorm(args.dim, eps=args.norm_eps)
        self.ffn_norm = RMSNorm(args.dim, eps=args.norm_eps)

    def forward(self, x, start_pos, rope_rows):
        h = x + self.attention(self.attention_norm(x), start_pos, rope_rows)
        return h + self.feed_forward(self.ffn_norm(h))


class Transformer(nn.Module):
    """``forward(tokens (1, S), start_pos) -> logits (1, 1, vocab)`` fp32 of the last
    position (evaluation/dram-attention/model.py:276-317)."""

    def __init__(self, params: ModelArgs, device="cuda"):
        super().__init__()
        self.params = params
        with torch.device(device):  # parameters are born on the device
            self.tok_embeddings = nn.Embedding(params.vocab_size, params.dim)
            self.layers = nn.ModuleList(TransformerBlock(i, params, device)
                                        for i in range(params.n_layers))
            self.norm = RMSNorm(params.dim, eps=params.norm_eps)
            self.output = nn.Linear(params.dim, params.vocab_size, bias=False)
        with torch.device("cpu"):   # one table for every device: built on the host
            rope = rope_table(params.head_dim, params.max_seq_len * 2, params.rope_theta,
                              params.use_scaled_rope)
        self.rope = rope.to(device)
        self.to(dtype=params.dtype)

    @torch.no_grad()
    def forward(self, tokens: torch.Tensor, start_pos):
        _bsz, seqlen = tokens.shape
        h = self.tok_embeddings(tokens)
        if isinstance(start_pos, torch.Tensor):
            assert seqlen == 1, "a device-resident position is for single-token decode steps"
            rows = self.rope.index_select(0, start_pos.reshape(1).long())
        else:
            rows = self.rope[start_pos: start_pos + seqlen]
        for layer in self.layers:
            h = layer(h, start_pos, rows)
        return self.output(self.norm(h[:, -1:, :])).float()

    def init_cache_from_files(self, cache_dir: str) -> int:
        """Load every layer's ``NN_cache.pth`` (examples/long-qa-chat/chat.py:214-233);
        returns the prompt length."""
        n = 0
        for i, layer in enumerate(self.layers):
            n = layer.attention.dram_attention.init_cache_from_file(cache_dir, i)
        return n


class GraphedDecoder:
    """Greedy decoding with the whole model step in one HIP graph, position and
    token resident on the device (examples/long-qa-chat/chat.py:238-273).

    The first step after the prompt runs eagerly: it sizes every layer's
    workspace, which a capture must not do.
    """

    def __init__(self, model: Transformer, prompt_len: int, first_token: int):
        dev = model.tok_embeddings.weight.device
        self.model = model
        self.token = torch.tensor([[first_token]], dtype=torch.long, device=dev)
        self.pos = torch.tensor([prompt_len], dtype=torch.int32, device=dev)
        self.graph = None
        self.logits = None

    def _step(self):
        logits = self.model(self.token, self.pos)
        self.token.copy_(logits.argmax(-1))
        self.pos.add_(1)
        return logits

    def step(self) -> torch.Tensor:
        """Feed the current token, advance; returns the logits (1, 1, vocab), valid
        until the next call."""
        if self.graph is None and self.logits is None:
            self.logits = self._step()
            return self.logits
        if self.graph is None:
            torch.cuda.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.logits = self._step()
        self.graph.replay()
        return self.logits
