"""configs[3] in small: several attention layers of the 128K shape stepped as one model
step, with layer i's page stream overlapping the selection of the layers after it.

Every layer is compared with its own CPU oracle at every step (request list, maps,
access times, hit mask, slot payload bit for bit; output within the bf16 tolerance),
and the pipelined order must give the same bits as stepping the layers one by one.
The pipelined model step is captured into one HIP graph and replayed, with the
position on the device, as a serving loop would run it."""

import pytest
import torch

from dram_attention_amd.synthetic import WORKLOADS, DecodeInputs, make_prompt
from oracle import dram_attention_oracle as O
from tests.parity import check_invariants, check_step
from tests.util import same

pytestmark = pytest.mark.gpu
DEV = "cuda"


def build(w, n_layers, seed0, max_out):
    from dram_attention_amd import DRAMAttention

    layers, oracles, feeds = [], [], []
    for li in range(n_layers):
        prompt = make_prompt(w, seed0 + li)
        m = DRAMAttention(max_out, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        o = O.DecodeOracle(max_out, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                           w.n_kv_heads, w.head_dim, dtype=w.dtype)
        o.init_cache(prompt.k, prompt.v)
        layers.append(m)
        oracles.append(o)
        feeds.append(DecodeInputs(w, prompt.q0, seed0 + li))
        print(f"stack test: layer {li} built", flush=True)
    return layers, oracles, feeds


@pytest.mark.parametrize("shape", ["scaled", "128k"])
def test_pipelined_stack_matches_oracles_and_serial_order(shape):
    from dram_attention_amd import AttentionStack, DRAMAttention

    if shape == "128k":
        w, n_layers, steps = WORKLOADS["128k"], 4, 3       # configs[3]'s layer, four of them
    else:
        w = WORKLOADS["128k"].scaled(dram_tokens=16384, local_cache=1024, lru_tokens=4096,
                                     top_k_tokens=1024)
        n_layers, steps = 6, 5
    layers, oracles, feeds = build(w, n_layers, 40, steps)
    stack = AttentionStack(layers, pipelined=True)
    # the same layers again, stepped one by one on one stream
    serial = []
    for li in range(n_layers):
        prompt = make_prompt(w, 40 + li)
        m = DRAMAttention(steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                          w.n_kv_heads, w.head_dim, device=DEV, dtype=w.dtype)
        m.init_cache(prompt.k.to(DEV), prompt.v.to(DEV))
        serial.append(m)
    serial_stack = AttentionStack(serial, pipelined=False)

    host = [[f.next() for f in feeds] for _ in range(steps)]           # [step][layer] -> (q, k, v)
    bufs = [tuple(torch.empty_like(x, device=DEV) for x in host[0][li]) for li in range(n_layers)]
    pos = torch.tensor([w.prompt_tokens], dtype=torch.int32, device=DEV)

    def feed(t):
        for li in range(n_layers):
            for dst, src in zip(bufs[li], host[t][li]):
                dst.copy_(src)

    def model_step():
        return stack.generate([b[0] for b in bufs], [b[1] for b in bufs], [b[2] for b in bufs], pos)

    def check(t, outs):
        want_serial = serial_stack.generate(*[[x[i].to(DEV) for x in host[t]] for i in range(3)],
                                            w.prompt_tokens + t)
        torch.cuda.synchronize()
        for li in range(n_layers):
            q, k, v = host[t][li]
            check_step(layers[li], oracles[li], q, k, v, w.prompt_tokens + t, outs[li], t, 2e-2, 1e-2)
            assert same(outs[li], want_serial[li]), f"layer {li} step {t}: pipelined vs serial order"
            assert same(layers[li].lru_cache.hbm_kv_cache, serial[li].lru_cache.hbm_kv_cache)
            assert same(layers[li].lru_cache.page_access_time, serial[li].lru_cache.page_access_time)
            assert layers[li].lru_cache.last_miss_counts().sum().item() > 0

    # step 0 eagerly (resolves the pinned mappings, sizes the workspaces)
    feed(0)
    outs = model_step()
    check(0, outs)
    pos += 1
    torch.cuda.synchronize()
    # the rest as one captured model step, replayed
    graph = torch.cuda.CUDAGraph()
    feed(1)
    with torch.cuda.graph(graph):
        outs = model_step()
        pos += 1
    for t in range(1, steps):
        feed(t)
        graph.replay()
        torch.cuda.synchronize()
        assert pos.item() == w.prompt_tokens + t + 1
        check(t, outs)


def test_stack_of_32_full_size_layers_by_properties():
    """configs[3] at its stated depth: 32 layers of the 128K shape (17 GB of pinned pages),
    one model step per HIP graph, 9 decode steps.  No CPU walk: every layer of the
    pipelined stack is held to the size-independent properties of a step (selection
    ordered and maximal, maps mutually inverse, slot payload = mapped page, attention
    against a dense fp32 softmax on the GPU), and to the bits of a second stack over the
    same prompts whose layers are stepped one after the other on one stream."""
    from dram_attention_amd import AttentionStack, DRAMAttention

    w, n_layers, steps = WORKLOADS["128k"], 32, 9
    Hq, Hkv, D = w.n_q_heads, w.n_kv_heads, w.head_dim
    g = torch.Generator(device=DEV).manual_seed(77)
    piped, serial, stores = [], [], []
    for li in range(n_layers):
        # the workload's distributions drawn on the GPU: K ~ N(0,1) x per-channel lognormal(0, 0.5)
        k = torch.randn(w.prompt_tokens, Hkv, D, generator=g, device=DEV)
        k *= torch.exp(0.5 * torch.randn(Hkv, D, generator=g, device=DEV))
        k = k.to(w.dtype)[None]
        v = torch.randn(w.prompt_tokens, Hkv, D, generator=g, device=DEV).to(w.dtype)[None]
        for group in (piped, serial):
            m = DRAMAttention(steps, w.lru_tokens, w.local_cache, w.page_size, w.top_k_tokens,
                              Hkv, D, device=DEV, dtype=w.dtype)
            m.init_cache(k, v)
            group.append(m)
        stores.append(piped[-1].lru_cache.dram_kv_cache.to(DEV))
        del k, v
        if (li + 1) % 8 == 0:
            print(f"stack test: {li + 1} of {n_layers} layer pairs built", flush=True)
    stack, serial_stack = AttentionStack(piped, pipelined=True), AttentionStack(serial, pipelined=False)
    # drifting queries as in the workload: q_t = 0.9 q_{t-1} + 0.44 N(0,1), per layer
    q = torch.randn(n_layers, Hq, D, generator=g, device=DEV)
    feeds = []
    for t in range(steps):
        if t:
            q = 0.9 * q + 0.44 * torch.randn(n_layers, Hq, D, generator=g, device=DEV)
        feeds.append((q.to(w.dtype), torch.randn(n_layers, Hkv, D, generator=g, device=DEV).to(w.dtype),
                      torch.randn(n_layers, Hkv, D, generator=g, device=DEV).to(w.dtype)))
    bufs = tuple(torch.empty_like(x) for x in feeds[0])
    pos = torch.tensor([w.prompt_tokens], dtype=torch.int32, device=DEV)

    def split(x):
        return [x[li][None, None] for li in range(n_layers)]

    def model_step():
        return stack.generate(split(bufs[0]), split(bufs[1]), split(bufs[2]), pos)

    def check(t, outs):
        want = serial_stack.generate(*[split(x) for x in feeds[t]], w.prompt_tokens + t)
        torch.cuda.synchronize()
        missed = 0
        for li in range(n_layers):
            check_invariants(piped[li], w, *[x[li][None, None] for x in feeds[t]], outs[li], t,
                             stores[li])
            assert same(outs[li], want[li]), f"layer {li} step {t}: pipelined vs serial order"
            assert same(piped[li].lru_cache.hbm_kv_cache, serial[li].lru_cache.hbm_kv_cache)
            assert same(piped[li].lru_cache.page_access_time, serial[li].lru_cache.page_access_time)
            missed += piped[li].lru_cache.last_miss_counts().sum().item()
        assert missed > n_layers * 100          # the steps really paged

    for dst, src in zip(bufs, feeds[0]):
        dst.copy_(src)
    outs = model_step()                         # step 0 eagerly: pinned mappings, workspaces
    check(0, outs)
    pos += 1
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = model_step()
        pos += 1
    for t in range(1, steps):
        for dst, src in zip(bufs, feeds[t]):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        assert pos.item() == w.prompt_tokens + t + 1
        check(t, outs)
        print(f"stack test: step {t} of {steps - 1} checked", flush=True)


def test_stack_argument_checks_and_short_stacks():
    from dram_attention_amd import AttentionStack

    w = WORKLOADS["128k"].scaled(dram_tokens=4096, local_cache=256, lru_tokens=1024, top_k_tokens=256)
    layers, oracles, feeds = build(w, 1, 60, 2)
    stack = AttentionStack(layers)
    q, k, v = feeds[0].next()
    with pytest.raises(ValueError):
        stack.generate([q.to(DEV)], [k.to(DEV)], [], w.prompt_tokens)
    (out,) = stack.generate([q.to(DEV)], [k.to(DEV)], [v.to(DEV)], w.prompt_tokens)
    check_step(layers[0], oracles[0], q, k, v, w.prompt_tokens, out, 0, 2e-2, 1e-2)
