"""Oracle: reward / advantage normalisation (CPU, test-only).

Restates ``areal/utils/data.py:1382-1637`` (class Normalization: group slices :1399-1430,
__call__ :1432-1538, masked mean with leave-one-out :1540-1597, masked std :1599-1637) and
``areal/utils/functional/functional.py:16-53`` (masked_normalization).  dtypes are kept as the
reference has them: group-level mean and std are written into fp32 tensors, batch-level ones
stay fp64 until the final ``.float()``.

Pinned by (tests/test_oracle_norm.py) the reference tests' literals: leave-one-out
[-2,-2/3,2/3,2], masked batch mean 5.0 / std sqrt(52/6), [-0.9258,-0.4629,0,1.3887], the
unbiased/biased ratio sqrt(3/2), variable group sizes against per-group mean/std, zero-variance
group -> 0, singleton leave-one-out -> 0, and the error cases.
"""

from __future__ import annotations

import numpy as np
import torch


def _mean(x, mask, leave_one_out):
    x = x.to(torch.float64)
    dims = tuple(range(x.ndim))
    if mask is None:
        factor = torch.tensor(np.prod(x.shape), dtype=torch.float64)
        xm = x
    else:
        mask = mask.to(torch.float64)
        xm = x * mask
        factor = mask.sum(dims, keepdim=True)
    total = xm.sum(dim=dims, keepdim=True)
    if leave_one_out:
        if factor.item() <= 1:
            return torch.zeros_like(total)
        if mask is None:
            return (total.expand_as(x) - x) / (factor - 1)
        loo = (total.expand_as(x) - xm) / torch.clamp(factor - mask, min=1.0)
        return torch.where(mask > 0, loo, (total / factor).expand_as(x))
    if factor.item() == 0:
        return torch.zeros_like(total)
    return total / factor


def _std(x, mask, mean, unbiased):
    x = x.to(torch.float64)
    mean = mean.to(torch.float64)
    dims = tuple(range(x.ndim))
    if mask is None:
        factor = torch.tensor(np.prod(x.shape), dtype=torch.float64)
        dev = x - mean
    else:
        mask = mask.to(torch.float64)
        factor = mask.sum(dims, keepdim=True)
        dev = x * mask - mean * mask
    ss = (dev**2).sum(dim=dims, keepdim=True)
    if unbiased:
        if factor.item() <= 1:
            return torch.ones_like(ss)
        return (ss / (factor - 1)).sqrt()
    if factor.item() == 0:
        return torch.ones_like(ss)
    return (ss / factor).sqrt()


def _slices(bs, group_size, group_sizes):
    if group_sizes is not None:
        if any(s <= 0 for s in group_sizes):
            raise ValueError(f"group_sizes must be all positive, got {group_sizes}")
        if sum(group_sizes) != bs:
            raise ValueError(f"group_sizes sum ({sum(group_sizes)}) must equal batch size ({bs}), got {group_sizes}")
        out, off = [], 0
        for s in group_sizes:
            out.append(slice(off, off + s))
            off += s
        return out
    return [slice(i * group_size, (i + 1) * group_size) for i in range(bs // group_size)]


def normalization(
    x, loss_mask=None, *, mean_level="batch", mean_leave1out=False, std_level="batch",
    std_unbiased=True, eps=1e-5, group_size=1, group_sizes=None,
):
    """Normalization(config)(x, loss_mask, group_sizes=...) (data.py:1432-1538)."""
    bs = x.size(0)
    if loss_mask is not None and loss_mask.sum().item() == 0:
        return x.float()
    sl = None
    if mean_level == "group" or std_level == "group":
        sl = _slices(bs, group_size, group_sizes)
    if mean_level == "batch":
        mean = _mean(x, loss_mask, mean_leave1out).expand_as(x)
    elif mean_level == "group":
        mean = torch.zeros_like(x)
        for s in sl:
            xs = x[s]
            ms = loss_mask[s] if loss_mask is not None else None
            if s.stop - s.start == 1 and mean_leave1out:
                gm = xs.to(torch.float64)
            else:
                gm = _mean(xs, ms, mean_leave1out)
            mean[s] = gm.expand_as(xs)
    else:
        mean = torch.zeros_like(x)
    centred = x - mean
    if loss_mask is not None:
        centred = centred * loss_mask
    if std_level == "batch":
        std = _std(x, loss_mask, mean, std_unbiased).expand_as(x)
    elif std_level == "group":
        std = torch.zeros_like(x)
        for s in sl:
            xs = x[s]
            ms = loss_mask[s] if loss_mask is not None else None
            if s.stop - s.start == 1 and std_unbiased:
                gs = torch.ones((1, *xs.shape[1:]), dtype=torch.float64)
            else:
                gs = _std(xs, ms, mean[s], std_unbiased)
            std[s] = gs.expand_as(xs)
    else:
        std = torch.ones_like(x)
        eps = 0.0
    return (centred / (std + eps)).float()


def masked_normalization(x, mask=None, unbiased=False, eps=1e-5, dim=None):
    """masked_normalization, fp64 sums (functional.py:16-53); dim=None reduces over everything."""
    x = x.to(torch.float64)
    dims = tuple(range(x.ndim)) if dim is None else ((dim,) if isinstance(dim, int) else tuple(dim))
    if mask is None:
        factor = torch.tensor(np.prod([x.shape[d] for d in dims]), dtype=torch.float64)
    else:
        mask = mask.to(torch.float64)
        x = x * mask
        factor = mask.sum(dims, keepdim=True)
    mean = x.sum(dim=dims, keepdim=True) / factor
    var = x.square().sum(dim=dims, keepdim=True) / factor - mean**2
    if unbiased:
        var = var * (factor / (factor - 1))
    return ((x - mean) / (var.sqrt() + eps)).float()
