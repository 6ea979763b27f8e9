"""Compact tensor comparisons for the test-suite (short failure messages)."""

import torch


def same(a, b) -> bool:
    """torch.equal with a one-line report of where two tensors first differ."""
    a, b = torch.as_tensor(a), torch.as_tensor(b)
    if a.shape != b.shape:
        print(f"shape mismatch: {tuple(a.shape)} vs {tuple(b.shape)}")
        return False
    a, b = a.cpu(), b.cpu()
    if torch.equal(a, b):
        return True
    neq = (a != b) & ~((a != a) & (b != b)) if a.is_floating_point() else (a != b)
    where = neq.nonzero()
    if where.numel() == 0:      # only NaNs at matching places
        return True
    first = tuple(where[0].tolist())
    print(f"{int(neq.sum())} of {a.numel()} entries differ; first at {first}: "
          f"{a[first].item()} vs {b[first].item()}")
    return False


def close(a, b, atol, rtol) -> bool:
    a, b = torch.as_tensor(a).cpu().float(), torch.as_tensor(b).cpu().float()
    if a.shape != b.shape:
        print(f"shape mismatch: {tuple(a.shape)} vs {tuple(b.shape)}")
        return False
    bad = ~((a - b).abs() <= atol + rtol * b.abs())
    if not bad.any():
        return True
    first = tuple(bad.nonzero()[0].tolist())
    print(f"{int(bad.sum())} of {a.numel()} entries out of tolerance (atol {atol}, rtol {rtol}); "
          f"max abs err {float((a - b).abs().max()):.4g}; first at {first}: "
          f"{a[first].item()} vs {b[first].item()}")
    return False
