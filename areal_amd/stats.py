"""Masked statistics of the per-token stat tensors of a loss call on MI355X.

The reference logs about 25 ``[T]`` tensors per micro-batch through ``stats_tracker.stat`` and
reduces each with ``torch.where(denominator, value, fill).sum() / .min() / .max()``
(``areal/utils/stats_tracker.py:455-560``): about 75 small reductions.  ``masked_stats`` computes
the sum, count, minimum and maximum of up to 32 tensors under their denominator masks in one
launch and one device-to-host copy.
"""

from __future__ import annotations

import ctypes

import torch

from areal_amd import _lib

MAX_TENSORS = 32


class DeferredStats:
    """Result of ``masked_stats(..., defer=True)``: the reductions are queued and their results
    on their way to pinned host memory; ``results`` waits for them when first read."""

    def __init__(self, pending):
        self._pending = pending  # [(keys, pinned host tensor, event)]
        self._results = None

    @property
    def results(self) -> dict[str, dict[str, float | None]]:
        if self._results is None:
            out = {}
            for keys, host, event in self._pending:
                event.synchronize()
                _unpack(out, keys, host)
            self._results, self._pending = out, None
        return self._results


def _unpack(out, keys, host) -> None:
    for j, k in enumerate(keys):
        s, c, mn, mx = host[j].tolist()
        empty = c == 0
        out[k] = dict(sum=s, count=c, avg=None if empty else s / c,
                      min=None if empty else mn, max=None if empty else mx)


def masked_stats(
    values: dict[str, torch.Tensor],
    denominators: dict[str, torch.Tensor | None],
    defer: bool = False,
):
    """``{key: {"sum", "count", "avg", "min", "max"}}`` of ``values[key]`` where
    ``denominators[key]`` is true (``None``: everywhere).  ``avg`` / ``min`` / ``max`` are ``None``
    for an empty mask, as ``_avg_of`` / ``_min_of`` / ``_max_of`` return.  ``defer=True`` returns
    a ``DeferredStats`` without waiting for the GPU."""
    lib = _lib.load()
    keys = list(values)
    out: dict[str, dict[str, float | None]] = {}
    pending = []
    for i in range(0, len(keys), MAX_TENSORS):
        chunk = keys[i : i + MAX_TENSORS]
        vals, masks = [], []
        n = None
        for k in chunk:
            v = values[k].detach().to(torch.float32).contiguous().view(-1)
            d = denominators.get(k)
            m = d.detach().bool().contiguous().view(-1) if d is not None else None
            if n is None:
                n = v.numel()
            if v.numel() != n or (m is not None and m.numel() != n):
                raise ValueError(f"stat `{k}` has {v.numel()} elements, expected {n}")
            vals.append(v)
            masks.append(m)
        dev = _lib.require_gpu(*vals, *[m for m in masks if m is not None])
        K = len(chunk)
        vptr = (ctypes.c_void_p * K)(*[v.data_ptr() for v in vals])
        mptr = (ctypes.c_void_p * K)(*[(m.data_ptr() if m is not None else None) for m in masks])
        res = torch.empty((K, 4), dtype=torch.float64, device=dev)
        nbytes = lib.areal_masked_stats_workspace_bytes(K)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_masked_stats(vptr, mptr, K, n, _lib.ptr(res), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev))
        _lib.check(rc, "areal_masked_stats")
        if defer:
            host = torch.empty(res.shape, dtype=res.dtype, pin_memory=True)
            host.copy_(res, non_blocking=True)
            event = torch.cuda.Event()
            event.record(torch.cuda.current_stream(dev))
            pending.append((chunk, host, event))
        else:
            _unpack(out, chunk, res.cpu())
    return DeferredStats(pending) if defer else out
