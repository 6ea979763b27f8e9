"""da_decode_attention_static: decode attention whose partial results live in a
device array built into the library (for callers that cannot allocate).  Called
through the C ABI and compared with da_decode_attention on the same inputs, to
the bar of the integer/byte work around it: the two run the same kernels with
the same chunk geometry, so outputs, log-sum-exp and the appended rows must
have the same bits.  Two calls in a row, the second on a smaller input, then a
shape beyond the built-in buffer (refused, nothing launched)."""

import math

import pytest
import torch

from dram_attention_amd import _lib
from tests.util import close, same

pytestmark = pytest.mark.gpu


def _case(seed, Hq, Hkv, D, p_len, capacity, c_len, dtype, dev):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g).to(dtype).to(dev)
    return dict(q=r(Hq, D), pk=r(Hkv, p_len, D), pv=r(Hkv, p_len, D), ck=r(capacity, Hkv, D),
                cv=r(capacity, Hkv, D), nk=r(Hkv, D), nv=r(Hkv, D), c_len=c_len)


def _call(lib, c, static, workspace=None):
    q, pk, pv = c["q"], c["pk"], c["pv"]
    ck, cv = c["ck"].clone(), c["cv"].clone()
    Hq, D = q.shape
    Hkv, p_len = pk.shape[0], pk.shape[1]
    out = torch.full((Hq, D), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((Hq,), float("nan"), dtype=torch.float32, device=q.device)
    head = (q.data_ptr(), q.stride(0), Hq, Hkv, D, _lib.dtype_code(q.dtype), pk.data_ptr(),
            pv.data_ptr(), pk.stride(1), pk.stride(0), p_len, ck.data_ptr(), cv.data_ptr(),
            ck.stride(0), ck.stride(1), ck.shape[0], c["c_len"], None, c["nk"].data_ptr(),
            c["nv"].data_ptr(), c["nk"].stride(0), 1.0 / math.sqrt(D), out.data_ptr(),
            out.stride(0), lse.data_ptr())
    stream = _lib.stream_ptr(q.device)
    if static:
        rc = lib.da_decode_attention_static(*head, stream)
    else:
        rc = lib.da_decode_attention(*head, workspace.data_ptr(), workspace.numel() * 4, stream)
    torch.cuda.synchronize()
    return rc, out, lse, ck, cv


def _dense(c):
    """fp64 softmax attention over prefix ++ local rows ++ the new token."""
    q = c["q"].double().cpu()
    Hq, D = q.shape
    Hkv = c["pk"].shape[0]
    rep = Hq // Hkv
    n = c["c_len"]
    k = torch.cat([c["pk"].cpu(), c["ck"][:n].transpose(0, 1).cpu(), c["nk"][:, None].cpu()], 1).double()
    v = torch.cat([c["pv"].cpu(), c["cv"][:n].transpose(0, 1).cpu(), c["nv"][:, None].cpu()], 1).double()
    s = torch.einsum("hrd,htd->hrt", q.view(Hkv, rep, D), k) / math.sqrt(D)
    return torch.einsum("hrt,htd->hrd", torch.softmax(s, -1), v).reshape(Hq, D)


def test_static_scratch_entry_matches_workspace_entry(lib):
    dev = torch.device("cuda", 0)
    cap_bytes = lib.da_decode_attention_static_capacity()
    assert cap_bytes == 8 << 20
    # the decode shape of the headline workload first, then a smaller, ragged one:
    # the second call must not see anything the first left in the shared array
    cases = [_case(1, 32, 8, 128, 32768, 4160, 4100, torch.bfloat16, dev),
             _case(2, 8, 2, 64, 1000 * 16, 300, 37, torch.float32, dev),
             _case(3, 32, 8, 128, 4096, 512, 0, torch.bfloat16, dev)]
    for n, c in enumerate(cases):
        Hq, D = c["q"].shape
        Hkv, p_len = c["pk"].shape[0], c["pk"].shape[1]
        need = lib.da_decode_attention_workspace_bytes(Hq, Hkv, D, _lib.dtype_code(c["q"].dtype),
                                                       p_len, c["ck"].shape[0], 0)
        assert 0 < need <= cap_bytes
        ws = torch.zeros((need + 3) // 4, dtype=torch.float32, device=dev)
        print(f"no-alloc case {n}: Hq {Hq} Hkv {Hkv} D {D} p_len {p_len} need {need}", flush=True)
        rc0, out0, lse0, ck0, cv0 = _call(lib, c, static=False, workspace=ws)
        assert rc0 == 0, lib.da_last_error_string()
        rc1, out1, lse1, ck1, cv1 = _call(lib, c, static=True)
        assert rc1 == 0, lib.da_last_error_string()
        assert not torch.isnan(out1.float()).any() and not torch.isnan(lse1).any()
        assert same(out1, out0) and same(lse1, lse0)          # bit for bit
        assert same(ck1, ck0) and same(cv1, cv0)              # the in-place append
        assert same(ck1[c["c_len"]], c["nk"]) and same(cv1[c["c_len"]], c["nv"])
        tol = (2e-2, 1e-2) if c["q"].dtype != torch.float32 else (1e-4, 1e-4)
        assert close(out1, _dense(c), *tol)


def test_static_scratch_entry_rejects_oversize(lib):
    dev = torch.device("cuda", 0)
    # a static 8M-token prefix needs more partial results than the built-in array holds
    Hq, Hkv, D = 128, 8, 128
    p_len = 8 << 20
    need = lib.da_decode_attention_workspace_bytes(Hq, Hkv, D, _lib.DA_BF16, p_len, 64, 0)
    assert need > lib.da_decode_attention_static_capacity()
    t = torch.zeros(Hq, D, dtype=torch.bfloat16, device=dev)     # stands in for every operand
    rc = lib.da_decode_attention_static(
        t.data_ptr(), D, Hq, Hkv, D, _lib.DA_BF16, t.data_ptr(), t.data_ptr(), D, p_len * D, p_len,
        t.data_ptr(), t.data_ptr(), Hkv * D, D, 64, 0, None, None, None, 0, 1.0, t.data_ptr(), D,
        None, _lib.stream_ptr(dev))
    assert rc == -2
    assert b"built-in buffer" in lib.da_last_error_string()
    torch.cuda.synchronize()
