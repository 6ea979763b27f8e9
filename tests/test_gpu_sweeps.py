"""Seeded sweeps over many small, odd shapes: every kernel against the CPU oracle.
The fixed cases of test_gpu_kernels.py pin the sizes that matter; these look for
the shapes nobody thought of."""

import numpy as np
import pytest
import torch

from oracle import dram_attention_oracle as O
from tests.test_gpu_kernels import dense_reference, lru_trace, run_topk
from tests.util import close, same

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
TOL = {torch.float32: (2e-5, 1e-4), torch.bfloat16: (2e-2, 1e-2), torch.float16: (4e-3, 1e-2)}


@pytest.mark.parametrize("seed", range(40))
def test_decode_attention_random_shapes(seed):
    from dram_attention_amd import decode_attention

    rng = np.random.default_rng(2000 + seed)
    dtype = DTYPES[rng.integers(0, 3)]
    Hkv = int(rng.integers(1, 5))
    rep = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16]))
    D = int(rng.choice([64, 128, 256] if dtype != torch.float32 else [16, 32, 64, 128]))
    p_len = int(rng.choice([0, 1, 7, 64, 333, 1024, 2500]))
    cap = int(rng.integers(1, 300))
    c_len = int(rng.integers(0, cap))
    append = bool(rng.integers(0, 2)) or (p_len == 0 and c_len == 0)
    Hq = Hkv * rep
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(Hq, D, generator=g).to(dtype)
    inter = torch.randn(Hkv, max(p_len, 1), 2, D, generator=g).to(dtype)[:, :p_len]
    ck = torch.randn(cap, Hkv, D, generator=g).to(dtype)
    cv = torch.randn(cap, Hkv, D, generator=g).to(dtype)
    nk = torch.randn(Hkv, D, generator=g).to(dtype)
    nv = torch.randn(Hkv, D, generator=g).to(dtype)
    segs = [(inter[:, :, 0], inter[:, :, 1]),
            (ck[:c_len].transpose(0, 1), cv[:c_len].transpose(0, 1))]
    if append:
        segs.append((nk[:, None], nv[:, None]))
    want, want_lse = dense_reference(q, segs)
    inter_d, ckd, cvd = inter.to(DEV), ck.to(DEV), cv.to(DEV)
    lse = torch.empty(Hq, dtype=torch.float32, device=DEV)
    out = decode_attention(q.to(DEV), inter_d[:, :, 0], inter_d[:, :, 1], ckd, cvd, c_len,
                           nk.to(DEV) if append else None, nv.to(DEV) if append else None, lse=lse)
    atol, rtol = TOL[dtype]
    assert close(out.cpu().float(), want, atol, rtol)
    assert torch.allclose(lse.cpu(), want_lse, atol=2e-3 if dtype != torch.float32 else 1e-4)
    if append:
        assert same(ckd[c_len].cpu(), nk) and same(cvd[c_len].cpu(), nv)


@pytest.mark.parametrize("seed", range(24))
def test_lru_update_random_shapes(seed):
    rng = np.random.default_rng(3000 + seed)
    H = int(rng.integers(1, 6))
    P = int(rng.integers(12, 700))
    N = int(rng.integers(2, P))
    K = int(rng.integers(1, min(2 * N, 600) + 1))
    itype = [torch.int32, torch.int64][rng.integers(0, 2)]
    ttype = [torch.float32, torch.int32][rng.integers(0, 2)]
    mode = int(rng.integers(0, 3))        # plain / list of least recent slots / forced serial walk
    hot = None if rng.integers(0, 2) else int(rng.integers(2, max(3, P // 4)))
    lru_trace(H, P, N, K, 6, 3100 + seed, itype, ttype, bool(rng.integers(0, 2)),
              dtype=torch.float32, page_dim=32, hot=hot, candidates=mode == 1,
              serial_walk=mode == 2)


@pytest.mark.parametrize("seed", range(24))
def test_topk_pages_random_shapes(seed):
    rng = np.random.default_rng(4000 + seed)
    rep = int(rng.choice([1, 2, 4, 7]))
    H = int(rng.integers(1, 4))
    seq = int(rng.integers(1, 3))
    L = int(rng.choice([1, 3, 64, 257, 1000, 4097, 9000, 17000, 40000]))
    k = int(rng.integers(1, min(L, 700) + 1))
    levels = int(rng.choice([0, 0, 3, 50]))   # 0: continuous scores, else that many distinct values
    g = torch.Generator().manual_seed(seed)
    if levels:
        scores = torch.randint(0, levels, (seq * rep, H, L), generator=g).float()
    else:
        scores = torch.randn(seq * rep, H, L, generator=g)
        if rng.integers(0, 2):
            scores = scores.bfloat16().float()
    got = run_topk(scores, rep, k)
    assert same(got, O.select_pages(scores, seq, rep, k))


@pytest.mark.parametrize("seed", range(24))
def test_page_score_and_minmax_random_shapes(seed):
    from dram_attention_amd import max_inner_product
    from dram_attention_amd.topk_selector import page_min_max

    rng = np.random.default_rng(5000 + seed)
    dtype = DTYPES[rng.integers(0, 3)]
    H = int(rng.integers(1, 5))
    N = int(rng.integers(1, 10))
    D = int(rng.choice([8, 24, 40, 64, 128, 256]))
    page = int(rng.choice([1, 4, 16, 24]))
    L = int(rng.integers(1, 300))
    g = torch.Generator().manual_seed(seed)
    keys = torch.randn(H, L * page, D, generator=g).to(dtype)
    mm = page_min_max(keys.to(DEV), L).cpu()
    assert same(mm, O.page_min_max(keys, L))
    q = torch.randn(N, H, D, generator=g).to(dtype)
    got = max_inner_product(q.to(DEV), mm.to(DEV)).cpu()
    want = O.max_ip(q, mm)
    assert got.dtype == dtype
    if dtype == torch.float32:
        assert close(got, want, 1e-3, 1e-3)
    else:
        # same rounding points; the fp32 summation order may move a sum across one rounding step
        step = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert torch.all((got.float() - want.float()).abs() <= want.float().abs() * step + 1e-6)
