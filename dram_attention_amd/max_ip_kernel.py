"""Quest upper-bound page scorer on the HIP kernel.

Mirrors dram_attention/max_ip_triton_kernel.py of the reference:
``max_inner_product`` (:95-124) launches the gfx950 kernel, ``max_ip_ref``
(:127-133) is the plain-torch statement of the same formula that the
reference ships next to its kernel for tests.
"""

from __future__ import annotations

import torch

from . import _lib


DA_SCORE_ROUND, DA_SCORE_ORDERED_BOUNDS = 1, 2


def page_scores(q: torch.Tensor, min_max: torch.Tensor, out: torch.Tensor,
                round_to_input: bool, ordered_bounds: bool = False) -> torch.Tensor:
    """score[n,h,l] into ``out`` (fp32 or q.dtype; any strides, last axis dense).
    ``ordered_bounds``: the caller vouches that min_max[...,0,:] <= min_max[...,1,:]
    (summaries made by page_min_max are); the kernel may then pick the bound by the
    sign of q instead of forming both products."""
    N, H, D = q.shape
    H1, L, R, D1 = min_max.shape
    assert H1 == H and D1 == D and R == 2
    _lib.require_gpu(q, "q")
    _lib.require_gpu(min_max, "min_max")
    if min_max.dtype != q.dtype:
        raise TypeError(f"q is {q.dtype} but min_max is {min_max.dtype}")
    if q.stride(-1) != 1:
        q = q.contiguous()
    if min_max.stride(-1) != 1:
        min_max = min_max.contiguous()
    assert out.shape == (N, H, L) and (L <= 1 or out.stride(-1) == 1)
    lib = _lib.load()
    _lib.check(
        lib.da_page_score(
            q.data_ptr(), q.stride(0), q.stride(1),
            min_max.data_ptr(), min_max.stride(0), min_max.stride(1), min_max.stride(2),
            N, H, L, D, _lib.dtype_code(q.dtype),
            out.data_ptr(), out.stride(0), out.stride(1), _lib.dtype_code(out.dtype),
            (DA_SCORE_ROUND if round_to_input else 0)
            | (DA_SCORE_ORDERED_BOUNDS if ordered_bounds else 0),
            _lib.stream_ptr(q.device),
        ),
        "da_page_score",
    )
    return out


def max_inner_product(q: torch.Tensor, min_max: torch.Tensor) -> torch.Tensor:
    """(N,H,D) x (H,L,2,D) -> (N,H,L) in q.dtype, like the reference wrapper."""
    N, H, D = q.shape
    H1, L, R, D1 = min_max.shape
    assert H1 == H and D1 == D and R == 2
    out = torch.empty(N, H, L, dtype=q.dtype, device=q.device)
    return page_scores(q, min_max, out, round_to_input=True)


def max_ip_ref(q: torch.Tensor, min_max: torch.Tensor) -> torch.Tensor:
    """Torch statement of the score: sum over channels of the larger of the two
    products with the page's per-channel min and max."""
    N, H, D = q.shape
    H1, L, R, D1 = min_max.shape
    assert H1 == H and D1 == D
    qe = q.reshape(N, H, 1, 1, D)
    return (qe * min_max.unsqueeze(0)).amax(dim=3).sum(dim=-1)
