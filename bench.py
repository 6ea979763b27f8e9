#!/usr/bin/env python3
"""Decode-step benchmark of the DRAM Attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 128k] [--eager] [--no-overlap]

A step is one `generate` call of one attention layer: page scoring, ordered
top-k, LRU update, streaming of missed pages from pinned host DRAM, and decode
attention over the resident pages + local window + new token.  Inputs of all
steps are staged in HBM before the clock starts.  By default the step is
captured once into a HIP graph (position and LRU step live on the device) and
replayed (--steps-per-graph consecutive steps per graph, as a model step of
several layers would be, with one input fetch and one counter increment per
graph); --eager issues the launches from Python every step;
--no-overlap runs the page stream to completion before attention starts.

Prints ONE JSON line: the headline metric plus `roofline` (the dominant HBM
kernel, timed live with events on the launch stream) and `cpu_baseline` (the CPU
oracle timed on this box's host cores on a bounded sample of the same workload).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0          # dense bf16 / fp16
# HBM bytes per launch of the roofline kernel (first attention pass) from the committed
# counter runs, by workload: the fallback when the summary file is not next to this script;
# a CPU test holds it equal to what the file says.
TRAFFIC_PROFILE = os.path.join("profiles", "bench_128k_hbm_traffic_pmc.md")
ROOFLINE_TRAFFIC_BYTES = {"128k": 152.8e6}


def roofline_traffic_from_profile(path=None):
    """The 'HBM traffic of the roofline kernel per launch = ... = N MB' figure of the
    committed counter summary, in bytes; None if the file is not there."""
    import re

    path = path or os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        with open(path) as f:
            text = f.read()
    except OSError:
        return None
    m = re.search(r"HBM traffic of the roofline kernel per launch\s*=[^\n]*?=\s*([0-9.]+)\s*MB", text)
    return float(m.group(1)) * 1e6 if m else None
WORKLOAD_INDEX = {"cpu": 0, "32k": 1, "128k": 2, "1m": 4}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="128k", choices=sorted(WORKLOAD_INDEX))
    ap.add_argument("--eager", action="store_true", help="no HIP graph: launch from Python each step")
    ap.add_argument("--steps-per-graph", type=int, default=32,
                    help="decode steps captured into one HIP graph, at most 32 (the reference's "
                         "example captures a whole model step, i.e. 32 attention layers, per graph); "
                         "if --steps is not a multiple, the largest divisor of --steps between half "
                         "of this and this is taken, else single-step graphs make up the rest")
    ap.add_argument("--no-overlap", action="store_true",
                    help="page stream and attention serialised on one stream")
    ap.add_argument("--force-lru", action="store_true",
                    help="workload 32k: run the page-cache path although the prefix fits the cache "
                         "(every request hits; the reference's init_cache would pick the static cache)")
    ap.add_argument("--plain-scorer", action="store_true",
                    help="score pages with the plain vector kernel (both products and their maximum) "
                         "instead of the sign-select / matrix-core form: same scores, for comparison")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-steps", type=int, default=64, help="steps of the CPU oracle to time (0 = skip)")
    ap.add_argument("--reference-shaped-steps", type=int, default=24,
                    help="steps of the reference-shaped stand-in pipeline to time (0 = skip)")
    ap.add_argument("--profile-steps", type=int, default=16, help="extra steps timed per kernel with events")
    ap.add_argument("--model-decode-steps", type=int, default=0,
                    help="also time greedy decoding of a Llama-3.1-8B-shaped model (random weights, "
                         "random K/V of the workload's prompt length in every layer's page cache), "
                         "whole model step per HIP graph; 0 = skip")
    ap.add_argument("--stack-layers", type=int, default=32,
                    help="also time an attention-only stack of this many layers of the workload "
                         "(configs[3] at 32 with workload 128k), pipelined and serial; 0 = skip")
    ap.add_argument("--stack-steps", type=int, default=6, help="timed model steps of that stack")
    ap.add_argument("--prefill-reps", type=int, default=2,
                    help="also time causal prefill attention at the workload's prompt length, this "
                         "library's kernel and torch's fused op; 0 = skip")
    ap.add_argument("--no-value-64", action="store_true",
                    help="skip the second timed run at the configuration's own 64 steps (warm-up 8) that "
                         "is made when --steps/--warmup differ from it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 128 MiB device copy (reference point for HBM traffic counters)")
    return ap.parse_args()


class Layer:
    """One attention layer set up on the workload, plus the staged step inputs."""

    def __init__(self, w, seed, total_steps, dev, overlap, force_lru=False, device_prompt=False,
                 prompt=None):
        from dram_attention_amd import DRAMAttention, DummyCache, LRUCache
        from dram_attention_amd.synthetic import DecodeInputs, make_prompt

        self.w = w
        self.m = DRAMAttention(max_output_length=total_steps, lru_hbm_cache_size=w.lru_tokens,
                               local_cache_size=w.local_cache, page_size=w.page_size,
                               top_k=w.top_k_tokens, n_kv_heads=w.n_kv_heads, head_dim=w.head_dim,
                               device=dev, dtype=w.dtype)
        self.m.overlap_page_stream = overlap
        if device_prompt:
            # the workload's distributions drawn on the GPU (a 32-layer stack would spend a
            # minute in the host generator); no CPU checker reads these layers
            prompt = device_prompt_like(w, seed, dev)
            self.m.init_cache(prompt.k, prompt.v)
            prompt.k = prompt.v = None
        else:
            if prompt is None:
                prompt = make_prompt(w, seed)
            self.m.init_cache(prompt.k.to(dev), prompt.v.to(dev))
        self.prompt = prompt
        if force_lru and isinstance(self.m.lru_cache, DummyCache):
            # the prefix fits the page cache, so init_cache chose the static cache; a page
            # cache built directly over the same prefix is the all-hits point of the LRU path
            S = self.m.dram_kv_cache_size
            self.m.lru_cache = LRUCache(prompt.k[0, :S].to(dev).transpose(0, 1),
                                        prompt.v[0, :S].to(dev).transpose(0, 1), w.page_size,
                                        w.top_k_tokens // w.page_size, w.lru_tokens, device=dev)
            self.m._workspace = None
        inputs = DecodeInputs(w, prompt.q0, seed)
        qs, ks, vs = zip(*(inputs.next() for _ in range(total_steps)))
        self.qs = torch.cat(qs).to(dev)   # (T, 1, Hq, D)
        self.ks = torch.cat(ks).to(dev)
        self.vs = torch.cat(vs).to(dev)
        # What the rest of a model would hand to the layer each step, staged as one
        # row per step: [q heads | k heads | v heads], fetched by one index_select.
        Hq, Hkv, D = w.n_q_heads, w.n_kv_heads, w.head_dim
        self.qkv = torch.cat([self.qs.view(total_steps, Hq * D), self.ks.view(total_steps, Hkv * D),
                              self.vs.view(total_steps, Hkv * D)], dim=1).contiguous()
        # Row 0: step index, row 1: position, each for this step and the next few
        # (column j = j steps ahead); all advance with a single increment kernel.
        ahead = torch.arange(self.MAX_STEPS_PER_GRAPH, dtype=torch.int32)
        self.cnt = torch.stack([ahead, ahead + w.prompt_tokens]).to(dev)
        self.t_dev, self.pos_dev = self.cnt[0, 0:1], self.cnt[1, 0:1]
        self.out = None

    MAX_STEPS_PER_GRAPH = 32

    def _step(self, row, pos):
        w = self.w
        Hq, Hkv, D = w.n_q_heads, w.n_kv_heads, w.head_dim
        xq = row[: Hq * D].view(1, 1, Hq, D)
        xk = row[Hq * D:(Hq + Hkv) * D].view(1, 1, Hkv, D)
        xv = row[(Hq + Hkv) * D:].view(1, 1, Hkv, D)
        self.out = self.m(xq, xk, xv, start_pos=pos, stage="generate")
        return self.out

    def step_from_device_state(self):
        """One decode step driven entirely by device-resident counters."""
        self._step(self.qkv.index_select(0, self.t_dev)[0], self.pos_dev)
        self.cnt += 1
        return self.out

    def steps_from_device_state(self, n):
        """n consecutive decode steps: their inputs arrive by one fetch and the
        counters advance once, the way a serving loop hands a model step its
        inputs and bumps the position once per token, not once per layer."""
        rows = self.qkv.index_select(0, self.cnt[0, :n])
        for j in range(n):
            self._step(rows[j], self.cnt[1, j:j + 1])
        self.cnt += n
        return self.out


def device_prompt_like(w, seed, dev):
    """make_prompt's distributions (K ~ N(0,1) x per-channel lognormal(0, 0.5), V ~ N(0,1),
    q0 ~ N(0,1)) drawn by the GPU's generator; planted pages are left out."""
    from dram_attention_amd.synthetic import Prompt

    g = torch.Generator(device=dev).manual_seed(seed)
    S, H, D = w.prompt_tokens, w.n_kv_heads, w.head_dim
    q0 = torch.randn(w.n_q_heads, D, generator=g, device=dev)
    k = torch.randn(S, H, D, generator=g, device=dev)
    if w.channel_scale:
        k *= torch.exp(0.5 * torch.randn(H, D, generator=g, device=dev))
    v = torch.randn(S, H, D, generator=g, device=dev)
    return Prompt(k.to(w.dtype)[None], v.to(w.dtype)[None], q0.cpu(), [])


def stack_leg(w, n_layers, steps, warmup, seed, dev):
    """configs[3]: `n_layers` independent attention layers of workload `w` stepped as one
    model step per HIP graph, once with layer i's page stream overlapping the
    selection (scores, top-k, LRU update) of the layers after it and once with the
    layers strictly one after the other, on the same caches."""
    from dram_attention_amd import AttentionStack

    settle, rounds = 16, 2
    total = settle + 2 * rounds * (steps + 1) + 6
    layers = []
    for li in range(n_layers):
        layers.append(Layer(w, seed + 100 + li, total, dev, overlap=True, device_prompt=True))
        if (li + 1) % 8 == 0:
            print(f"bench.py: stack layer {li + 1}/{n_layers} built", file=sys.stderr, flush=True)
    Hq, Hkv, D = w.n_q_heads, w.n_kv_heads, w.head_dim
    qkv = torch.stack([l_.qkv for l_ in layers], dim=1).contiguous()      # (T, layers, width)
    for l_ in layers:
        l_.qs = l_.ks = l_.vs = l_.qkv = None
    cnt = torch.tensor([0, w.prompt_tokens], dtype=torch.int32, device=dev)   # step, position

    def model_step(stack):
        rows = qkv.index_select(0, cnt[0:1])[0]                               # (layers, width)
        xq = [rows[i, : Hq * D].view(1, 1, Hq, D) for i in range(n_layers)]
        xk = [rows[i, Hq * D:(Hq + Hkv) * D].view(1, 1, Hkv, D) for i in range(n_layers)]
        xv = [rows[i, (Hq + Hkv) * D:].view(1, 1, Hkv, D) for i in range(n_layers)]
        out = stack.generate(xq, xk, xv, cnt[1:2])
        cnt.add_(1)
        return out

    # Both orders run on the same caches, so they are timed in alternating rounds after
    # the page caches have settled (the first steps after a prefill miss several
    # times as many pages as the steady state).
    graphs = {}
    for name, pipelined in (("pipelined", True), ("serial", False)):
        stack = AttentionStack([l_.m for l_ in layers], pipelined=pipelined)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model_step(stack)                     # eager: pinned mappings, workspaces
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graphs[name] = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graphs[name]):
            model_step(stack)
    for _ in range(settle):
        graphs["serial"].replay()
    torch.cuda.synchronize()
    spent = {"pipelined": 0.0, "serial": 0.0}
    for _ in range(rounds):
        for name in ("pipelined", "serial"):
            graphs[name].replay()                 # warm-up of the round
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                graphs[name].replay()
            torch.cuda.synchronize()
            spent[name] += time.perf_counter() - t0
    res = {}
    for name, dt in spent.items():
        n = rounds * steps
        res[name] = {"layer_steps_per_s": n * n_layers / dt, "model_steps_per_s": n / dt,
                     "ms_per_model_step": dt / n * 1e3, "us_per_layer_step": dt / n / n_layers * 1e6}
    misses = sum(int(l_.m.lru_cache.last_miss_counts().sum().item()) for l_ in layers) / n_layers
    page_bytes = w.page_size * 2 * D * torch.empty(0, dtype=w.dtype).element_size()
    return {"value": res["pipelined"]["layer_steps_per_s"], "unit": "decode steps/s per layer",
            "layers": n_layers, "steps": rounds * steps, "settling_steps": settle,
            "workload": f"configs[3] shape: {n_layers} independent layers of workload {w.name}, one page "
                        f"cache each ({n_layers * w.n_kv_heads * w.n_dram_pages * page_bytes / 1e9:.1f} GB "
                        "of pinned pages), one model step per HIP graph",
            "pipelined": res["pipelined"], "serial": res["serial"],
            "speedup_of_overlap": res["pipelined"]["layer_steps_per_s"] / res["serial"]["layer_steps_per_s"],
            "distinct_misses_per_layer_last_step": misses,
            "h2d_bytes_per_model_step": misses * n_layers * page_bytes,
            "what": "pipelined: selection of layer i+1.. on a side stream while layer i's pages cross "
                    "the host link; serial: the same launches on one stream"}


def algorithmic_bytes(w, local_rows):
    e = torch.empty(0, dtype=w.dtype).element_size()
    score = w.n_kv_heads * w.n_dram_pages * 2 * w.head_dim * e
    attn = (w.n_hbm_pages * w.page_size + local_rows + 1) * w.n_kv_heads * 2 * w.head_dim * e
    return score, attn


def time_kernels(layer, steps):
    """Per-kernel GPU time over `steps` further decode steps, issued one launch at a
    time on the current stream with an event on either side.  A short busy kernel
    goes first so that both events and the launch are queued before the GPU gets
    to them: the interval is the kernel, not the host's launch latency.  The page
    stream runs to completion before attention here (no overlap), so each kernel
    is seen alone."""
    from dram_attention_amd.dram_attention import PagedPrefix, decode_attention
    from dram_attention_amd.lru_kernel import GATHER_BLOCKS, gather_attend_supported

    from dram_attention_amd import LRUCache

    m, lru, w = layer.m, layer.m.lru_cache, layer.w
    names = ("page_score", "topk_pages", "lru_update", "pages_gather", "decode_attention_split",
             "split+merge", "decode_attention_first_merge", "decode_attention_tail+merge")
    acc = {n: 0.0 for n in names}
    misses, local_rows = 0, []
    if not isinstance(lru, LRUCache):
        # prefix within the HBM budget: no paging, the step is one attention pass
        for _ in range(steps):
            t = int(layer.t_dev.item())
            xq, xk, xv = layer.qs[t:t + 1], layer.ks[t:t + 1], layer.vs[t:t + 1]
            pk, pv = lru.get_kv_cache_(xq)
            c_len = int(layer.pos_dev.item()) - m.dram_kv_cache_size
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda._sleep(2_000_000)
            e0.record()
            decode_attention(xq[0, 0], pk, pv, m.cache_k[0], m.cache_v[0], c_len, xk[0, 0],
                             xv[0, 0], workspace=m._workspace)
            e1.record()
            torch.cuda.synchronize()
            acc["decode_attention_split"] += e0.elapsed_time(e1)   # includes its merge launch
            local_rows.append(c_len)
            layer.cnt += 1
        return ({"decode_attention_split": acc["decode_attention_split"] / steps * 1e3}, 0.0,
                sum(local_rows) / len(local_rows))

    def timed(name, fn, repeat=8):
        """`repeat` back-to-back launches between one pair of events (the kernels
        timed this way are idempotent); the interval / repeat is one launch."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda._sleep(2_000_000)  # GPU busy time: the whole batch is queued behind it
        e0.record()
        for _ in range(repeat):
            r = fn()
        e1.record()
        pending.append((name, e0, e1, repeat))
        return r

    for _ in range(steps):
        pending = []
        t = int(layer.t_dev.item())
        xq, xk, xv = layer.qs[t:t + 1], layer.ks[t:t + 1], layer.vs[t:t + 1]
        sel = lru.top_k_selector
        k = min(lru.top_k, lru.num_dram_pages)
        from dram_attention_amd.topk_selector import topk_pages
        scores = timed("page_score", lambda: sel.scores(xq))
        idx = lru._topk_idx
        cand = lru._scratch_for(idx.shape[1]).candidates   # least recent slots, listed by the same launch
        timed("topk_pages", lambda: topk_pages(scores, w.rep, k, idx, w.rep * k, idx.shape[1], k,
                                               lru=(lru.page_access_time, cand, lru.current_step)))
        scratch = timed("lru_update", lambda: lru.update_(idx), repeat=1)   # mutates its state
        pk, pv = lru.views()
        c_len = int(layer.pos_dev.item()) - m.dram_kv_cache_size
        args = (xq[0, 0], pk, pv, m.cache_k[0], m.cache_v[0], c_len, xk[0, 0], xv[0, 0])
        out = torch.empty(w.n_q_heads, w.head_dim, dtype=w.dtype, device=xq.device)
        fused = m.attend_on_page_stream and gather_attend_supported(
            w.n_q_heads, w.n_kv_heads, w.head_dim, w.page_size, w.dtype)
        blocks = max(1, min(GATHER_BLOCKS // w.n_kv_heads, idx.shape[1])) if fused else 0
        if fused:   # the page stream that also attends over the pages it moves
            timed("pages_gather", lambda: lru.gather_attend_(
                idx.shape[1], xq[0, 0], 1.0 / math.sqrt(w.head_dim), m.cache_k.shape[1],
                m._workspace, blocks))
        else:
            timed("pages_gather", lambda: lru.gather_(idx.shape[1]))
        P = PagedPrefix
        # fused stream: the step merges once, after the combined launch; its cost is
        # (first pass + merge) - (first pass).  Otherwise: first-pass merge, then
        # tail pass + final merge after the stream.
        phases = ((("decode_attention_split", P.FIRST), ("split+merge", P.FIRST | P.SECOND))
                  if fused else
                  (("decode_attention_split", P.FIRST),
                   ("decode_attention_first_merge", P.FIRST_MERGE),
                   ("decode_attention_tail+merge", P.SECOND)))
        for name, phase in phases:
            timed(name, lambda phase=phase: decode_attention(
                *args, workspace=m._workspace, out=out,
                paged=PagedPrefix(w.page_size, scratch, lru.current_step, phase, blocks)))
        torch.cuda.synchronize()
        for name, e0, e1, repeat in pending:
            acc[name] += e0.elapsed_time(e1) / repeat
        misses += int(lru.last_miss_counts().sum().item())
        local_rows.append(c_len)
        layer.cnt += 1
    us = {n: v / steps * 1e3 for n, v in acc.items() if v > 0.0}  # microseconds
    if "split+merge" in us:
        us["decode_attention_merge"] = us.pop("split+merge") - us["decode_attention_split"]
    return us, misses / steps, sum(local_rows) / len(local_rows)


def time_step_launch(layer, steps):
    """The launch that dominates a step, timed where it runs: `steps` further decode steps
    issued as the module issues them (selection, then page stream + first attention pass
    as ONE launch, then the merge), with an event on either side of the stream + attention
    launch and a busy kernel ahead so that the launches are queued when the GPU gets to
    them.  Returns (average us of that launch, average distinct misses per step)."""
    m = layer.m
    spent, misses = 0.0, 0
    for _ in range(steps):
        t = int(layer.t_dev.item())
        xq, xk, xv = layer.qs[t:t + 1], layer.ks[t:t + 1], layer.vs[t:t + 1]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda._sleep(2_000_000)
        selected = m.select_(xq)
        e0.record()
        out, merge = m.attend_(xq, xk, xv, layer.pos_dev, selected, defer_merge=True)
        e1.record()
        if merge is None:
            return None, None          # this shape does not take the one-launch form
        merge()
        torch.cuda.synchronize()
        spent += e0.elapsed_time(e1)
        misses += int(m.lru_cache.last_miss_counts().sum().item())
        layer.cnt += 1
    return spent / steps * 1e3, misses / steps


def timed_replays(layer, steps, warmup, wanted_spg):
    """`warmup` untimed + `steps` timed decode steps of a freshly built layer, captured and
    replayed as the main leg does; returns (steps/s, steps per graph)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            layer.step_from_device_state()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    single = torch.cuda.CUDAGraph()
    with torch.cuda.graph(single):
        layer.step_from_device_state()
    spg = steps_per_graph(steps, wanted_spg, Layer.MAX_STEPS_PER_GRAPH)
    many = None
    if spg > 1:
        many = torch.cuda.CUDAGraph()
        with torch.cuda.graph(many):
            layer.steps_from_device_state(spg)
    for _ in range(max(warmup - 2, 0)):
        single.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps // spg if many is not None else 0):
        many.replay()
    for _ in range(steps % spg if many is not None else steps):
        single.replay()
    torch.cuda.synchronize()
    return steps / (time.perf_counter() - t0), spg


def prefill_leg(w, dev, reps, seed):
    """stage="prefill" attention at the workload's prompt length: the library's kernel
    (da_prefill_attention) and torch's fused op beside it, events on the launch stream;
    flops = the causal half of two S x S x D products per query head."""
    from dram_attention_amd.dram_attention import causal_prefill_attention, prefill_attention_supported

    S, Hq, Hkv, D = w.prompt_tokens, w.n_q_heads, w.n_kv_heads, w.head_dim
    g = torch.Generator(device=dev).manual_seed(seed)
    xq = torch.randn(1, S, Hq, D, device=dev, generator=g).to(w.dtype)
    xk = torch.randn(1, S, Hkv, D, device=dev, generator=g).to(w.dtype)
    xv = torch.randn(1, S, Hkv, D, device=dev, generator=g).to(w.dtype)
    flops = 4.0 * S * S * D * Hq / 2
    res = {"prompt_tokens": S, "flops": flops, "reps": reps,
           "what": "causal attention of stage=prefill (reference dram_attention.py:136), outside the "
                   "decode-step metric; flops = 4*S*S*D*Hq/2"}
    backends = (["native"] if prefill_attention_supported(xq) else []) + ["sdpa"]
    for b in backends:
        try:
            causal_prefill_attention(xq, xk, xv, b)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                causal_prefill_attention(xq, xk, xv, b)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            tf = flops / (ms * 1e-3) / 1e12
            res[b] = {"ms": ms, "TFLOPs": tf}
            if b == "native":
                res[b]["roofline"] = {"bound": "mfma", "kernel": "prefill_attention_kernel", "achieved": tf,
                                      "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                                      "frac": tf / MFMA_PEAK_TFLOPS}
        except RuntimeError as exc:
            res[b] = {"error": str(exc)[:200]}
    if "native" in res and "sdpa" in res and "ms" in res["native"] and "ms" in res["sdpa"]:
        res["native_over_sdpa"] = res["sdpa"]["ms"] / res["native"]["ms"]
    return res


def host_link_gbps(dev, mb=64, reps=5):
    """Pinned host -> HBM copy rate of the box (hipMemcpyAsync through torch)."""
    src = torch.empty(mb << 20, dtype=torch.uint8).pin_memory()
    dst = torch.empty(mb << 20, dtype=torch.uint8, device=dev)
    dst.copy_(src, non_blocking=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        dst.copy_(src, non_blocking=True)
    torch.cuda.synchronize()
    return reps * (mb << 20) / (time.perf_counter() - t0) / 1e9


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            return next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")),
                        "unknown")
    except OSError:
        return "unknown"


def time_oracle(w, seed, steps, warmup=0, prompt=None):
    """Wall-clock of the CPU oracle on `warmup` untimed + `steps` timed decode steps
    of workload `w`.  Draws its own prompt and step inputs from the workload's
    seeded generators (the first steps the GPU run sees), so it depends on
    nothing the GPU legs staged.  Returns (steps/s, per-stage ms per step)."""
    from dram_attention_amd.synthetic import DecodeInputs, make_prompt
    from oracle import dram_attention_oracle as O

    if prompt is None:
        prompt = make_prompt(w, seed)
    o = O.DecodeOracle(warmup + steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                       w.n_kv_heads, w.head_dim, dtype=w.dtype)
    o.init_cache(prompt.k, prompt.v)
    inputs = DecodeInputs(w, prompt.q0, seed)
    for t in range(warmup):
        o.generate(*inputs.next(), w.prompt_tokens + t)
    stages = {}
    staged = [inputs.next() for _ in range(steps)]
    t0 = time.perf_counter()
    for t, (q, k, v) in enumerate(staged):
        o.generate(q, k, v, w.prompt_tokens + warmup + t, timings=stages)
    dt = time.perf_counter() - t0
    return steps / dt, {k: v / steps * 1e3 for k, v in stages.items()}, dt


def cpu_baseline(w, seed, steps, prompt=None, cfg0_steps=16, cfg0_warmup=3):
    """The CPU oracle (a restatement of the reference's torch/Triton path; the
    reference has no CPU path of its own for the LRU walk or for attention) on
    all host cores: `value` on the first `steps` decode steps of the benchmarked
    workload, `cfg0` on configs[0] exactly as stated (fp32, 3 warm-up + 16 timed)."""
    from dram_attention_amd.synthetic import WORKLOADS

    cores = torch.get_num_threads()
    value, stages, dt = time_oracle(w, seed, steps, prompt=prompt)
    res = {"value": value, "unit": "decode steps/s per layer", "cores": cores, "kind": "port",
           "cpu_model": cpu_model_name(), "os_cpu_count": os.cpu_count(),
           "same_workload": True, "stage_ms_per_step": stages,
           "sample": f"first {steps} decode steps of workload {w.name}, torch-CPU oracle, "
                     f"{dt / steps * 1e3:.1f} ms/step, {dt:.1f} s in all"}
    if cfg0_steps > 0:
        w0 = WORKLOADS["cpu"]
        v0, st0, dt0 = time_oracle(w0, seed, cfg0_steps, warmup=cfg0_warmup)
        res["cfg0"] = {"value": v0, "unit": "decode steps/s per layer", "cores": cores,
                       "stage_ms_per_step": st0,
                       "sample": f"configs[0] as stated: fp32, 8q/2kv heads, D 64, 8192-token prefix, "
                                 f"{cfg0_warmup} warm-up + {cfg0_steps} timed steps, "
                                 f"{dt0 / cfg0_steps * 1e3:.2f} ms/step"}
    return res


def time_cache_build(layer, dev):
    """One-time set-up kernels at the size of the workload, timed with events: the page
    summaries, and the kernel that packs the prompt's K/V into the pinned page store
    and the initial slots (writes cross the host link once)."""
    from dram_attention_amd import LRUCache, _lib
    from dram_attention_amd.topk_selector import page_min_max

    lru, w = layer.m.lru_cache, layer.w
    if not isinstance(lru, LRUCache) or layer.prompt is None:
        return None
    S = w.dram_tokens
    k = layer.prompt.k[0, :S].to(dev).transpose(0, 1)      # (Hkv, S, D) views, as init_cache passes
    v = layer.prompt.v[0, :S].to(dev).transpose(0, 1)
    esz = k.element_size()
    dram, dram_ptr, hbm = lru.page_stores()
    scratch_hbm = torch.empty_like(hbm)                    # the live slots must stay as they are
    lib = _lib.load()

    def build():
        _lib.check(lib.da_pages_build(
            k.data_ptr(), v.data_ptr(), k.stride(1), k.stride(0), w.n_kv_heads, w.n_dram_pages,
            w.page_size, w.head_dim, _lib.dtype_code(w.dtype), dram_ptr, dram.stride(0) * esz,
            dram.stride(1) * esz, scratch_hbm.data_ptr(), hbm.stride(0) * esz, hbm.stride(1) * esz,
            w.n_dram_pages - w.n_hbm_pages, w.n_hbm_pages, _lib.stream_ptr(dev)), "da_pages_build")

    res = {}
    for name, fn in (("page_minmax", lambda: page_min_max(k, w.n_dram_pages)), ("pages_build", build)):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            fn()
        e1.record()
        torch.cuda.synchronize()
        res[name + "_ms"] = e0.elapsed_time(e1) / 3
    res["host_store_bytes"] = dram.numel() * esz
    res["pages_build_to_host_GBps"] = res["host_store_bytes"] / (res["pages_build_ms"] * 1e-3) / 1e9
    return res


def reference_shaped(w, seed, steps, dev):
    """Stand-in for the reference's own GPU decode step (its Triton and flash-attn
    kernels cannot run here): the same sequence of stages in the same shape,
    from stock torch-ROCm ops where the reference uses torch or flash-attn, and
    from the serial form of this library's kernels where it uses Triton
    (dram_attention/lru_cache.py:211-265, lru_triton_kernel.py:140-194,
    dram_attention.py:179-238):
      scores by the torch statement max_ip_ref; full descending argsort; index
      shuffle; step += 1; touch of the hit slots; full stable argsort of the
      access times; a serial walk, one lane per kv head, then one workgroup per
      kv head copying that head's missed pages; attention as two passes (slots,
      local window) with log-sum-exp, combined by the reference's formula.
    Returns steps/s over `steps` replays and the average misses per step."""
    from dram_attention_amd import DRAMAttention
    from dram_attention_amd.lru_kernel import lru_update, pages_gather
    from dram_attention_amd.synthetic import DecodeInputs, make_prompt

    prompt = make_prompt(w, seed)
    total = (steps + 4 + 63) // 64 * 64      # local cache rows divisible into equal key ranges
    m = DRAMAttention(max_output_length=total, lru_hbm_cache_size=w.lru_tokens,
                      local_cache_size=w.local_cache, page_size=w.page_size, top_k=w.top_k_tokens,
                      n_kv_heads=w.n_kv_heads, head_dim=w.head_dim, device=dev, dtype=w.dtype)
    m.init_cache(prompt.k.to(dev), prompt.v.to(dev))
    lru = m.lru_cache
    inputs = DecodeInputs(w, prompt.q0, seed)
    qs, ks, vs = zip(*(inputs.next() for _ in range(total)))
    Hq, Hkv, D, rep = w.n_q_heads, w.n_kv_heads, w.head_dim, w.rep
    qkv = torch.cat([torch.cat(qs).view(total, Hq * D), torch.cat(ks).view(total, Hkv * D),
                     torch.cat(vs).view(total, Hkv * D)], dim=1).to(dev)
    ctr = torch.tensor([0, w.prompt_tokens - m.dram_kv_cache_size], dtype=torch.int64, device=dev)
    kp = min(lru.top_k, lru.num_dram_pages)
    K = rep * kp
    mm = lru.top_k_selector.chunk_min_max
    cap = m.cache_k.shape[1]
    rows = torch.arange(cap, device=dev)
    scale = 1.0 / math.sqrt(D)
    out = torch.empty(Hq, D, dtype=w.dtype, device=dev)
    from dram_attention_amd.lru_kernel import LruScratch
    scratch = LruScratch.allocate(Hkv, K, dev, lru.num_hbm_pages)
    misses = torch.zeros(1, dtype=torch.int64, device=dev)

    # Attention passes: flash-attn's decode kernel splits the keys over many workgroups
    # (flash_attn_with_kvcache).  torch-ROCm's fused attention ops do not (one call
    # over the 32K-token prefix takes ~1.16 ms on this part, a bmm + softmax pair
    # ~0.21 ms), so the stand-in splits the keys itself: the sequence is cut into
    # `parts` batch entries, one fused call returns every part's output and
    # log-sum-exp, and the parts are combined by their log-sum-exp (~0.09 ms).
    fused_ok = w.dtype in (torch.bfloat16, torch.float16)
    used = set()

    def split_attend(q, k, v, parts, bias=None):
        """q (Hkv, rep, D); k, v (Hkv, T, D) views; bias (T,) additive or None."""
        T = k.shape[1]
        kb = k.reshape(Hkv, parts, T // parts, D).transpose(0, 1)
        vb = v.reshape(Hkv, parts, T // parts, D).transpose(0, 1)
        qb = q[None].expand(parts, Hkv, rep, D)
        if bias is None:
            r = torch.ops.aten._scaled_dot_product_flash_attention(qb, kb, vb, 0.0, False, False,
                                                                   scale=scale)
            o, lse = r[0], r[1]
        else:
            bb = bias.view(parts, 1, 1, T // parts).expand(parts, Hkv, rep, T // parts).contiguous()
            r = torch.ops.aten._scaled_dot_product_efficient_attention(qb, kb, vb, bb, True,
                                                                       scale=scale)
            o, lse = r[0], r[1][..., :rep]
        lse = lse.float()
        total = torch.logsumexp(lse, 0)
        return (o.float() * torch.exp(lse - total)[..., None]).sum(0), total

    def bmm_attend(q, k, v, mask=None):
        s_ = torch.bmm(q, k.transpose(1, 2)).float() * scale          # (Hkv, rep, T)
        if mask is not None:
            s_ = s_.masked_fill(mask, float("-inf"))
        lse = torch.logsumexp(s_, dim=-1)
        p = torch.exp(s_ - lse[..., None]).to(q.dtype)
        return torch.bmm(p, v).float(), lse

    def parts_of(T, want):
        while want > 1 and (T % want or (T // want) % 8):
            want //= 2
        return want

    def attend(q, k, v, want_parts, beyond=None):
        """`beyond`: bool (T,), True for rows past the valid length (device side)."""
        if fused_ok:
            try:
                bias = None
                if beyond is not None:
                    bias = torch.zeros(k.shape[1], dtype=q.dtype, device=dev).masked_fill_(
                        beyond, float("-inf"))
                parts = parts_of(k.shape[1], want_parts)
                res = split_attend(q, k, v, parts, bias)
                used.add(f"fused op over {parts} key ranges" + (" with a length mask" if bias is not None else ""))
                return res
            except RuntimeError:
                pass
        used.add("bmm + softmax")
        return bmm_attend(q, k, v, None if beyond is None else beyond[None, None, :])

    def step():
        row = qkv.index_select(0, ctr[0:1])[0]
        xq = row[: Hq * D].view(Hkv, rep, D)
        xk = row[Hq * D:(Hq + Hkv) * D].view(Hkv, D)
        xv = row[(Hq + Hkv) * D:].view(Hkv, D)
        # scores: sum_d max(q*min, q*max), one query row of the group at a time
        scores = torch.stack([(xq[:, r, None, None, :] * mm).amax(dim=2).sum(dim=-1)
                              for r in range(rep)], dim=1)            # (Hkv, rep, P)
        top = torch.argsort(scores, dim=-1, descending=True, stable=True)[..., :kp]
        idx = top.reshape(Hkv, K).contiguous().clamp_(0, lru.num_dram_pages - 1)
        lru.current_step.add_(1)
        slots = torch.gather(lru.dram_page_to_hbm_page_mapping, 1, idx)
        now = lru.current_step.to(lru.page_access_time.dtype)
        touched = torch.where(slots >= 0, now, torch.full_like(now, float("-inf")))
        lru.page_access_time.scatter_reduce_(1, slots.clamp(min=0), touched.expand_as(slots),
                                             reduce="amax")
        torch.argsort(lru.page_access_time, dim=-1, stable=True)      # the reference's eviction order
        lru_update(lru.dram_kv_cache, lru.page_access_time, lru.dram_page_to_hbm_page_mapping,
                   lru.hbm_page_to_dram_page_mapping, idx, lru.current_step, lru.hbm_kv_cache,
                   scratch, bump_step=False, serial_walk=True)
        pages_gather(lru.dram_kv_cache, lru.hbm_kv_cache, scratch, K, lru.page_stores()[1],
                     max_blocks=Hkv)
        misses.add_(scratch.miss_count.sum())
        pk, pv = lru.views()
        o_p, lse_p = attend(xq, pk, pv, 32)
        c = ctr[1:2]
        m.cache_k[0].index_copy_(0, c, xk[None])
        m.cache_v[0].index_copy_(0, c, xv[None])
        ck = m.cache_k[0].transpose(0, 1)                              # (Hkv, cap, D)
        cv = m.cache_v[0].transpose(0, 1)
        o_s, lse_s = attend(xq, ck, cv, 8, rows > c)
        lse = torch.logaddexp(lse_p, lse_s)
        o = o_p * torch.exp(lse_p - lse)[..., None] + o_s * torch.exp(lse_s - lse)[..., None]
        out.copy_(o.view(Hq, D))
        ctr.add_(1)

    # Issued eagerly, not from a HIP graph: replaying a capture of this step ended in
    # an out-of-range address; the library sorts in it record memset nodes, which
    # are not reliable in replayed graphs here.  The step is GPU-bound (about 50 launches against more
    # than a millisecond of GPU work), so launches queue ahead and eager issue
    # costs the stand-in nothing.
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    misses.zero_()
    t0 = time.perf_counter()
    for _ in range(steps - 3):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    n = steps - 3
    return {"value": n / dt, "unit": "decode steps/s per layer", "ms_per_step": dt / n * 1e3,
            "steps": n, "distinct_misses_per_step": misses.item() / n,
            "attention_op": "aten._scaled_dot_product_flash_attention (prefix) / _efficient_attention "
                            "(local window), keys split over the batch axis, + log-sum-exp combine; "
                            "paths taken: " + "; ".join(sorted(used)),
            "what": "stand-in for the reference's GPU step, not the reference: torch-ROCm ops for its "
                    "torch/flash-attn stages (max_ip_ref scores, full argsorts, two attention passes by "
                    "torch's fused attention op with the keys split over the batch axis as flash-attn's "
                    "decode kernel splits them, + the reference's log-sum-exp combine), this library's "
                    "serial one-lane-per-head LRU walk and one-workgroup-per-head page copy for its "
                    "Triton stages; launched eagerly (GPU-bound)"}


def model_decode(w, steps, seed, dev):
    """Tokens per second of a Llama-3.1-8B-shaped decoder (32 layers, random bf16
    weights) whose every layer holds a page cache over a random prompt of the
    workload's length: the figure the reference's chat example prints, with the
    model step captured in one graph as it does."""
    from dram_attention_amd.llama import GraphedDecoder, ModelArgs, Transformer

    torch.manual_seed(seed)
    a = ModelArgs(dim=w.n_q_heads * w.head_dim, n_layers=32, n_heads=w.n_q_heads,
                  n_kv_heads=w.n_kv_heads, vocab_size=128256, multiple_of=1024,
                  ffn_dim_multiplier=1.3, rope_theta=500000.0, use_scaled_rope=True,
                  lru_hbm_cache_size=w.lru_tokens, local_cache_size=w.local_cache,
                  cache_page_size=w.page_size, cache_top_k=w.top_k_tokens,
                  max_output_length=steps + 8, max_seq_len=w.prompt_tokens + steps + 8,
                  dtype=w.dtype)
    model = Transformer(a, device=dev)
    shape = (1, w.prompt_tokens, w.n_kv_heads, w.head_dim)
    for layer in model.layers:
        k = torch.randn(shape, device=dev, dtype=w.dtype)
        v = torch.randn(shape, device=dev, dtype=w.dtype)
        layer.attention.dram_attention.init_cache(k, v)
        del k, v
    dec = GraphedDecoder(model, w.prompt_tokens, first_token=1)
    dec.step()                       # eager: sizes the workspaces
    dec.step()                       # captures the graph and replays it once
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dec.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    misses = sum(l_.attention.dram_attention.lru_cache.last_miss_counts().sum().item()
                 for l_ in model.layers) / a.n_layers
    params = sum(p.numel() for p in model.parameters())
    return {"value": steps / dt, "unit": "tokens/s", "ms_per_token": dt / steps * 1e3,
            "steps": steps, "model": "Llama-3.1-8B shape, random weights", "parameters": params,
            "prompt_tokens": w.prompt_tokens, "distinct_misses_per_layer_last_step": misses,
            "launch": "one HIP graph per token (32 layers)"}


def steps_per_graph(steps: int, wanted: int, limit: int) -> int:
    """How many decode steps one captured graph holds: `wanted`, capped by `limit` and by
    the number of timed steps; if that does not divide `steps`, the largest divisor of
    `steps` between half of it and it (equal graphs, no single-step graphs at the end)."""
    spg = max(1, min(wanted, steps, limit))
    if steps % spg:
        spg = next((d for d in range(spg, (spg + 1) // 2 - 1, -1) if steps % d == 0), spg)
    return spg


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this hot path is a single-device decode step "
              "(run with --gpus 1)", file=sys.stderr)
        return 2
    if args.profile_steps <= 0:
        print("bench.py: --profile-steps must be at least 1 (the roofline figures come from that pass)",
              file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HIP kernels are the only implementation", file=sys.stderr)
        return 2
    from dram_attention_amd import LRUCache, _lib
    from dram_attention_amd.synthetic import WORKLOADS

    _lib.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    w = WORKLOADS[args.workload]
    step_launch_steps = 8
    total = args.warmup + args.steps + args.profile_steps + step_launch_steps + 4
    layer = Layer(w, args.seed, total, dev, overlap=not args.no_overlap, force_lru=args.force_lru)
    if args.plain_scorer and isinstance(layer.m.lru_cache, LRUCache):
        layer.m.lru_cache.top_k_selector.bounds_are_ordered = False
    n_layers = 1

    def model_step():
        layer.step_from_device_state()

    torch.cuda.synchronize()

    # -- warm-up (also resolves the pinned-host device address before any capture)
    graph, graph_many, spg = None, None, 1
    if args.eager:
        for _ in range(args.warmup):
            model_step()
    else:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                model_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            model_step()
        spg = steps_per_graph(args.steps, args.steps_per_graph, Layer.MAX_STEPS_PER_GRAPH)
        if spg > 1:
            graph_many = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph_many):
                layer.steps_from_device_state(spg)
        # the captures themselves executed nothing; replay for the remaining warm-up steps
        for _ in range(max(args.warmup - 2, 0)):
            graph.replay()
    torch.cuda.synchronize()

    # -- timed region: exactly args.steps decode steps
    t0 = time.perf_counter()
    if graph is not None:
        for _ in range(args.steps // spg if graph_many is not None else 0):
            graph_many.replay()
        for _ in range(args.steps % spg if graph_many is not None else args.steps):
            graph.replay()
    else:
        for _ in range(args.steps):
            model_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / (args.steps * n_layers) * 1e3

    # -- the step's dominant launch where it runs, then every kernel alone, and traffic counters
    paged = isinstance(layer.m.lru_cache, LRUCache)
    step_launch_us, step_launch_misses = (time_step_launch(layer, step_launch_steps)
                                          if paged and not args.no_overlap else (None, None))
    kernel_us, miss_per_step, local_rows = time_kernels(layer, args.profile_steps)
    score_b, attn_b = algorithmic_bytes(w, local_rows)
    attn_us = kernel_us["decode_attention_split"]
    achieved = attn_b / (attn_us * 1e-6) / 1e9
    requests = w.n_kv_heads * w.rep * w.pages_per_q_head
    page_bytes = w.page_size * 2 * w.head_dim * torch.empty(0, dtype=w.dtype).element_size()
    link = host_link_gbps(dev)
    if args.calibrate_copy:
        # a plain elementwise kernel of known traffic: reads 128 MiB, writes 128 MiB
        src = torch.ones(32 << 20, dtype=torch.float32, device=dev)
        dst = torch.add(src, 1.0)
        torch.cuda.synchronize()
        del src, dst
    stream_gbps = (miss_per_step * page_bytes / (kernel_us["pages_gather"] * 1e-6) / 1e9
                   if miss_per_step else 0.0)
    score_gbps = (score_b / (kernel_us["page_score"] * 1e-6) / 1e9
                  if "page_score" in kernel_us else None)

    # HBM bytes per launch of the roofline kernel from the committed counter runs
    # (profiles/bench_128k_hbm_traffic_pmc.md: FETCH_SIZE x 2.0 + WRITE_SIZE); only
    # known for the workload those runs used
    traffic = None
    if w.name in ROOFLINE_TRAFFIC_BYTES:
        traffic = roofline_traffic_from_profile() or ROOFLINE_TRAFFIC_BYTES[w.name]
    result = {
        "metric": "decode steps/sec per layer at 128K ctx; scorer+attn HBM GB/s vs peak",
        "value": args.steps * n_layers / dt,
        "unit": "decode steps/s per layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[w.dtype],
        "data": "synthetic",
        "config": {
            "workload": f"configs[{WORKLOAD_INDEX[w.name]}] {w.name}: 1 layer, "
                        f"{w.n_q_heads}q/{w.n_kv_heads}kv heads, D {w.head_dim}, "
                        f"{w.dram_tokens}-token prefix in pinned host DRAM ({w.n_dram_pages} pages/head), "
                        f"local {w.local_cache}, LRU {w.lru_tokens} tokens, top-k {w.top_k_tokens} tokens",
            "launch": ("eager" if args.eager else
                       f"hip-graph replay, {spg} decode steps per graph (one input fetch and one counter "
                       f"increment per graph)"),
            "page_stream": "serialised" if args.no_overlap else "in the launch of the first attention pass",
            "seed": args.seed,
            "cache": type(layer.m.lru_cache).__name__,
            "scorer": "plain vector kernel" if args.plain_scorer else "sign-select + matrix-core sum",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": ("decode_attention_tile_kernel (first pass: prefix + local segments, matrix cores)"
                       if paged else
                       "decode_attention_tile_kernel + merge launch (static prefix: the two launches "
                       "of one call are timed together, so frac is a lower bound for the first)")
                      if w.dtype != torch.float32 else "decode_attention_split_kernel (fp32, vector units)",
            "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
            "traffic_source": ("not measured by this run: FETCH_SIZE x 2.0 + WRITE_SIZE per launch of this kernel "
                               "from the committed counter runs, profiles/bench_128k_hbm_traffic_pmc.md"
                               if traffic is not None else None),
            "algorithmic_bytes": attn_b, "avg_us": attn_us,
        },
        "roofline_step": None,
        "kernels_us": kernel_us,
        "kernels_us_note": "each kernel alone, after the timed region: 8 launches back to back between two "
                           "events, except lru_update, which changes its state and is one launch between "
                           "two events, so that its figure holds ~4 us of event and launch latency (a "
                           "kernel trace shows 6.3-6.6 us at the 128K shape)",
        "page_score_GBps": score_gbps,
        "page_stream": {"requests_per_step": requests, "distinct_misses_per_step": miss_per_step,
                        "h2d_bytes_per_step": miss_per_step * page_bytes,
                        "gather_GBps": stream_gbps, "host_link_memcpy_GBps": link,
                        "frac_of_link": stream_gbps / link if link else None,
                        "hit_rate": 1.0 - miss_per_step / requests},
    }
    if step_launch_us:
        step_bytes = step_launch_misses * page_bytes
        step_gbps = step_bytes / (step_launch_us * 1e-6) / 1e9
        result["roofline_step"] = {
            "kernel": "decode_stream_attend_tile_kernel (page stream + first attention pass, the launch "
                      "that dominates the timed step)" if w.dtype != torch.float32 else
                      "decode_stream_attend_kernel (page stream + first attention pass)",
            "bound": "host link", "bytes": step_bytes, "distinct_misses_per_step": step_launch_misses,
            "avg_us": step_launch_us, "achieved": step_gbps, "peak": link, "unit": "GB/s",
            "frac": step_gbps / link if link else None,
            "peak_source": "pinned hipMemcpyAsync rate measured in this run",
            "note": "events around the launch inside eagerly issued steps (selection before it, merge "
                    "after it), 8 steps after the timed region",
        }
    else:
        del result["roofline_step"]
    # The auxiliary legs below must never cost the headline line: a failure in one of
    # them is reported in its place.
    def leg(name, fn):
        try:
            value = fn()
            if value is not None:
                result[name] = value
        except Exception as exc:  # noqa: BLE001 - reported, not swallowed
            result[name] = {"error": f"{type(exc).__name__}: {exc}"}
            print(f"bench.py: leg {name} failed: {type(exc).__name__}: {exc}", file=sys.stderr, flush=True)

    leg("cache_build", lambda: time_cache_build(layer, dev))
    config_steps, config_warmup = w.steps, 8
    if (args.steps, args.warmup) == (config_steps, config_warmup) or args.eager:
        if not args.eager:
            result["value_64"] = {"value": result["value"], "steps": config_steps, "warmup": config_warmup,
                                  "note": "the timed region of this run"}
    elif not args.no_value_64:
        def value_64():
            prompt = layer.prompt
            l2 = Layer(w, args.seed, config_warmup + config_steps + 4, dev, overlap=not args.no_overlap,
                       force_lru=args.force_lru, prompt=prompt)
            if args.plain_scorer and isinstance(l2.m.lru_cache, LRUCache):
                l2.m.lru_cache.top_k_selector.bounds_are_ordered = False
            v, spg2 = timed_replays(l2, config_steps, config_warmup, args.steps_per_graph)
            return {"value": v, "unit": "decode steps/s per layer", "steps": config_steps,
                    "warmup": config_warmup, "ms_per_step": 1e3 / v, "steps_per_graph": spg2,
                    "note": f"the configuration's own {config_steps} decode steps after {config_warmup} "
                            "warm-up steps, same prompt and seed, a second layer built for it"}
        leg("value_64", value_64)
    if args.prefill_reps > 0 and w.dtype != torch.float32:
        leg("prefill", lambda: prefill_leg(w, dev, args.prefill_reps, args.seed))
    if args.cpu_steps > 0:
        leg("cpu_baseline", lambda: cpu_baseline(w, args.seed, args.cpu_steps, prompt=layer.prompt))
    if args.reference_shaped_steps > 3 and isinstance(layer.m.lru_cache, LRUCache):
        del layer, model_step
        torch.cuda.empty_cache()

        def ref_leg():
            ref = reference_shaped(w, args.seed, args.reference_shaped_steps, dev)
            ref["speedup_of_value"] = result["value"] / ref["value"]
            return ref

        leg("reference_shaped_gpu", ref_leg)
    if args.stack_layers > 1 and paged:
        layer = model_step = None
        torch.cuda.empty_cache()
        leg("stack", lambda: stack_leg(w, args.stack_layers, args.stack_steps, 2, args.seed, dev))
    if args.model_decode_steps > 0:
        layer = model_step = None
        torch.cuda.empty_cache()
        leg("model_decode", lambda: model_decode(w, args.model_decode_steps, args.seed, dev))
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
