"""Seeded synthetic decode workloads (the five benchmark configurations).

All draws come from a CPU ``torch.Generator`` in fp32 and are cast afterwards,
so a CPU checker and the GPU path see bit-identical inputs.

  K ~ N(0,1) * s_d, s_d = exp(N(0, 0.5)) per (kv head, channel)   [outlier channels]
  V ~ N(0,1)
  q_0 ~ N(0,1);  q_t = 0.9 q_{t-1} + 0.44 N(0,1)                  [drift => page reuse]
  planted pages (configs "cpu" and "1m"): every token of the page has
  key = 3 * q_dir + N(0, 0.3), q_dir = the initial query of one member of the
  owning kv group rescaled to norm sqrt(D) (page j: kv head j % Hkv, member
  (j // Hkv) % rep); they sit outside the initially resident tail.
Config "cpu" draws K without the channel scale (plain N(0,1)).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, replace

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    n_q_heads: int
    n_kv_heads: int
    head_dim: int
    dram_tokens: int        # prefix tokens that end up in the paged store
    local_cache: int
    lru_tokens: int         # HBM page-cache capacity in tokens
    top_k_tokens: int
    steps: int
    page_size: int = 16
    planted_pages: int = 0
    channel_scale: bool = True
    layers: int = 1

    @property
    def prompt_tokens(self) -> int:
        # init_cache pages (S - local + page)//page*page tokens: this S gives dram_tokens
        return self.dram_tokens + self.local_cache - self.page_size

    @property
    def n_dram_pages(self) -> int:
        return self.dram_tokens // self.page_size

    @property
    def n_hbm_pages(self) -> int:
        return self.lru_tokens // self.page_size

    @property
    def pages_per_q_head(self) -> int:
        return self.top_k_tokens // self.page_size

    @property
    def rep(self) -> int:
        return self.n_q_heads // self.n_kv_heads

    def scaled(self, **kw) -> "Workload":
        return replace(self, **kw)


WORKLOADS = {
    # configs[0]: the CPU-runnable reference case
    "cpu": Workload("cpu", torch.float32, 8, 2, 64, 8192, 1024, 2048, 512, 16,
                    planted_pages=4, channel_scale=False),
    # configs[1]: Llama-3-8B layer shape, 32K prefix (prefix == LRU capacity)
    "32k": Workload("32k", torch.bfloat16, 32, 8, 128, 32768, 4096, 32768, 4096, 64),
    # configs[2]: the headline, 128K prefix
    "128k": Workload("128k", torch.bfloat16, 32, 8, 128, 131072, 4096, 32768, 4096, 64),
    # configs[3]: 32 such layers
    "128k-x32": Workload("128k-x32", torch.bfloat16, 32, 8, 128, 131072, 4096, 32768, 4096, 64,
                         layers=32),
    # configs[4]: Llama-3-70B layer shape, 1M prefix
    "1m": Workload("1m", torch.bfloat16, 64, 8, 128, 1048576, 8192, 65536, 8192, 64,
                   planted_pages=16),
}


@dataclass
class Prompt:
    k: torch.Tensor          # (1, S, Hkv, D)
    v: torch.Tensor          # (1, S, Hkv, D)
    q0: torch.Tensor         # (Hq, D) fp32, the initial query state
    planted: list            # [(kv_head, page)]


def make_prompt(w: Workload, seed: int = 0) -> Prompt:
    g = torch.Generator().manual_seed(seed)
    S, H, D = w.prompt_tokens, w.n_kv_heads, w.head_dim
    q0 = torch.randn(w.n_q_heads, D, generator=g)
    k = torch.randn(S, H, D, generator=g)
    if w.channel_scale:
        k *= torch.exp(0.5 * torch.randn(H, D, generator=g))
    v = torch.randn(S, H, D, generator=g)
    planted = []
    if w.planted_pages:
        free = w.n_dram_pages - w.n_hbm_pages  # pages not resident at start
        members = q0.view(H, w.rep, D)
        for j in range(w.planted_pages):
            h = j % H
            q_dir = members[h, (j // H) % w.rep]
            q_dir = q_dir / q_dir.norm() * math.sqrt(D)
            page = (j + 1) * free // (w.planted_pages + 1)
            t0 = page * w.page_size
            noise = 0.3 * torch.randn(w.page_size, D, generator=g)
            k[t0:t0 + w.page_size, h] = 3.0 * q_dir + noise
            planted.append((h, page))
    return Prompt(k.to(w.dtype)[None], v.to(w.dtype)[None], q0, planted)


class DecodeInputs:
    """Iterator over the per-step (xq, xk, xv) of a workload, each shaped like the
    module's generate inputs: (1,1,Hq,D), (1,1,Hkv,D), (1,1,Hkv,D)."""

    def __init__(self, w: Workload, q0: torch.Tensor, seed: int = 0):
        self.w = w
        self.g = torch.Generator().manual_seed(seed + 7919)
        self.q = q0.clone()
        self.t = 0

    def next(self):
        w = self.w
        if self.t > 0:
            self.q = 0.9 * self.q + 0.44 * torch.randn(self.q.shape, generator=self.g)
        self.t += 1
        xk = torch.randn(w.n_kv_heads, w.head_dim, generator=self.g)
        xv = torch.randn(w.n_kv_heads, w.head_dim, generator=self.g)
        return (self.q.to(w.dtype)[None, None].clone(), xk.to(w.dtype)[None, None],
                xv.to(w.dtype)[None, None])
