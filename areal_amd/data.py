"""``Normalization`` and ``KLEstimator`` with the reference's interfaces
(``areal/utils/data.py:1382-1637`` and ``:1640-1698``).

``Normalization.__call__`` runs the three-pass kernel of ``csrc/gae_norm.hip``: fp64 sums,
group-level statistics rounded to fp32 exactly where the reference stores them in fp32
tensors.  Multi-rank reduction of batch statistics is outside the one-GPU scope.
"""

from __future__ import annotations

import functools

import torch
import torch.distributed as dist

from areal_amd import _lib
from areal_amd.config import NormConfig

_LEVEL_ID = {None: 0, "none": 0, "batch": 1, "group": 2}


@functools.lru_cache(maxsize=64)
def _group_tables(groups: tuple, tail_rows: int, row_len: int, device_str: str):
    offsets, rows = [0], []
    for g in groups:
        offsets.append(offsets[-1] + g * row_len)
        rows.append(g)
    tail_group = -1
    if tail_rows > 0:
        tail_group = len(rows)
        offsets.append(offsets[-1] + tail_rows * row_len)
        rows.append(tail_rows)
    dev = torch.device(device_str)
    max_len = max(b - a for a, b in zip(offsets[:-1], offsets[1:]))
    return (
        torch.tensor(offsets, dtype=torch.int64, device=dev),
        torch.tensor(rows, dtype=torch.int64, device=dev),
        tail_group,
        max_len,
    )


class Normalization:
    """Adaptive normalisation with independent levels for mean and std:
    ``"batch"``, ``"group"`` (fixed ``group_size`` or explicit ``group_sizes``) or ``None``."""

    def __init__(self, config: NormConfig):
        self.mean_level = config.mean_level
        self.mean_leave1out = config.mean_leave1out
        self.std_level = config.std_level
        self.std_unbiased = config.std_unbiased
        self.group_size = config.group_size
        self.eps = config.eps

    def _group_rows(self, bs: int, group_sizes: list[int] | None) -> tuple[tuple, int]:
        """Row counts of the groups and the number of trailing rows in no group."""
        if group_sizes is not None:
            if any(sz <= 0 for sz in group_sizes):
                raise ValueError(f"group_sizes must be all positive, got {group_sizes}")
            if sum(group_sizes) != bs:
                raise ValueError(
                    f"group_sizes sum ({sum(group_sizes)}) must equal "
                    f"batch size ({bs}), got {group_sizes}"
                )
            return tuple(int(s) for s in group_sizes), 0
        n_groups = bs // self.group_size
        return (self.group_size,) * n_groups, bs - n_groups * self.group_size

    @torch.no_grad()
    def __call__(
        self,
        x: torch.Tensor,
        loss_mask: torch.Tensor | None = None,
        high_precision: bool = True,
        reduce_group=None,
        group_sizes: list[int] | None = None,
    ) -> torch.Tensor:
        del high_precision  # sums are always fp64
        if dist.is_initialized() and dist.get_world_size(reduce_group) > 1 and "batch" in (
            self.mean_level, self.std_level,
        ):
            raise NotImplementedError("batch-level normalisation over several ranks is not built")
        lib = _lib.load()
        dev = _lib.require_gpu(x, loss_mask)
        bs = x.size(0)
        xf = x.to(torch.float32).contiguous()
        n = xf.numel()
        out = torch.empty_like(xf)
        if n == 0:
            return out
        if loss_mask is not None and loss_mask.shape != x.shape:
            loss_mask = loss_mask.expand_as(x)
        mf = loss_mask.to(torch.float32).contiguous() if loss_mask is not None else None
        row_len = n // bs
        if self.mean_level == "group" or self.std_level == "group":
            groups, tail = self._group_rows(bs, group_sizes)
        else:
            groups, tail = (bs,), 0
        if not groups and tail == 0:
            return xf
        offsets, rows, tail_group, max_len = _group_tables(groups, tail, row_len, str(dev))
        n_groups = rows.numel()
        nbytes = lib.areal_group_norm_workspace_bytes(n_groups, max_len)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_group_norm(
            _lib.ptr(xf), _lib.ptr(mf), n, _lib.ptr(offsets), _lib.ptr(rows), n_groups, max_len,
            tail_group, _LEVEL_ID[self.mean_level], _LEVEL_ID[self.std_level],
            int(bool(self.mean_leave1out)), int(bool(self.std_unbiased)), float(self.eps),
            _lib.ptr(out), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_group_norm")
        return out


    def needs_one_statistics_pass(self) -> bool:
        """True when the sums of one pass over the data determine the result: no leave-one-out
        mean, and not a group-level mean under a batch-level deviation."""
        return not self.mean_leave1out and not (self.mean_level == "group" and self.std_level == "batch")

    @torch.no_grad()
    def from_row_stats(self, x: torch.Tensor, mask_f32: torch.Tensor, row_stats: torch.Tensor,
                       group_sizes: list[int] | None = None) -> torch.Tensor | None:
        """``self(x, mask)`` for a 2-D fp32 ``x`` whose per-row masked sums are already known
        (``row_stats`` ``[5, bs]`` fp64 as the GAE kernel leaves them): one launch. Returns
        ``None`` when this configuration needs a second statistics pass."""
        if not self.needs_one_statistics_pass() or x.ndim != 2:
            return None
        lib = _lib.load()
        dev = _lib.require_gpu(x, mask_f32, row_stats)
        bs, row_len = x.shape
        if self.mean_level == "group" or self.std_level == "group":
            groups, tail = self._group_rows(bs, group_sizes)
        else:
            groups, tail = (bs,), 0
        if not groups and tail == 0:
            return x
        offsets, rows, tail_group, max_len = _group_tables(groups, tail, row_len, str(dev))
        out = torch.empty_like(x)
        rc = lib.areal_group_norm_from_row_stats(
            _lib.ptr(x), _lib.ptr(mask_f32), bs, row_len, _lib.ptr(offsets), _lib.ptr(rows), rows.numel(),
            max_len, tail_group, _LEVEL_ID[self.mean_level], _LEVEL_ID[self.std_level],
            int(bool(self.std_unbiased)), float(self.eps), _lib.ptr(row_stats), _lib.ptr(out),
            _lib.stream_ptr(dev),
        )
        if rc == _lib.ERR_UNSUPPORTED:
            return None
        _lib.check(rc, "areal_group_norm_from_row_stats")
        return out


    @torch.no_grad()
    def packed(self, x: torch.Tensor, mask_f32: torch.Tensor | None, cu_seqlens: torch.Tensor,
               group_sizes: list[int] | None = None, max_group_tokens: int | None = None,
               segment_stats: torch.Tensor | None = None) -> torch.Tensor:
        """``self`` over a packed 1-D fp32 ``x``: sequence ``i`` is ``[cu_seqlens[i],
        cu_seqlens[i+1])`` and plays the part of row ``i`` of the padded form, so groups are runs
        of ``group_size`` (or ``group_sizes``) whole sequences.  ``segment_stats``: the sums the
        packed GAE kernel left for these groups (``_packed_gae_with_segment_stats``), which make
        this one launch; the configuration must satisfy ``needs_one_statistics_pass``.
        ``max_group_tokens``: an upper bound of a group's token count (read back from
        ``cu_seqlens`` when not given, which waits for the GPU)."""
        lib = _lib.load()
        dev = _lib.require_gpu(x, mask_f32, cu_seqlens)
        if x.ndim != 1:
            raise ValueError(f"packed normalisation expects a 1D tensor, got ndim={x.ndim}")
        n, n_seqs = x.numel(), cu_seqlens.numel() - 1
        if n == 0:
            return x.clone()
        index, rows, tail_group = self._packed_groups(n_seqs, group_sizes, dev)
        offsets = cu_seqlens.to(torch.int64)[index]
        if max_group_tokens is None:
            max_group_tokens = int((offsets[1:] - offsets[:-1]).max())
        out = torch.empty_like(x)
        levels = (_LEVEL_ID[self.mean_level], _LEVEL_ID[self.std_level])
        if segment_stats is not None:
            rc = lib.areal_group_norm_from_segment_stats(
                _lib.ptr(x), _lib.ptr(mask_f32), n, _lib.ptr(offsets), _lib.ptr(rows), rows.numel(),
                max_group_tokens, tail_group, *levels, int(bool(self.std_unbiased)), float(self.eps),
                _lib.ptr(segment_stats), _lib.ptr(out), _lib.stream_ptr(dev),
            )
            _lib.check(rc, "areal_group_norm_from_segment_stats")
            return out
        nbytes = lib.areal_group_norm_workspace_bytes(rows.numel(), max_group_tokens)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_group_norm(
            _lib.ptr(x), _lib.ptr(mask_f32), n, _lib.ptr(offsets), _lib.ptr(rows), rows.numel(),
            max_group_tokens, tail_group, *levels, int(bool(self.mean_leave1out)),
            int(bool(self.std_unbiased)), float(self.eps), _lib.ptr(out), _lib.ptr(ws), nbytes,
            _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_group_norm")
        return out

    def _packed_groups(self, n_seqs: int, group_sizes, dev):
        """(index of each group's first sequence plus ``n_seqs`` [G+1], sequences per group [G],
        tail group) as device tensors, for groups of whole sequences."""
        if self.mean_level == "group" or self.std_level == "group":
            groups, tail = self._group_rows(n_seqs, group_sizes)
        else:
            groups, tail = (n_seqs,), 0
        return _group_tables(groups, tail, 1, str(dev))[:3]


class KLEstimator:
    """k1 / k2 / k3 estimators of KL(new || base) from log-probabilities
    (``data.py:1640-1698``).  Elementwise tensor arithmetic on whatever device holds the
    inputs; the rejection-sampling kernel has its own fused copy of these formulas."""

    def __init__(self, kl_estimator: str = "k1", apply_clamp: bool = True):
        if kl_estimator not in ["k1", "k2", "k3"]:
            raise ValueError(f"Invalid KL estimator: {kl_estimator}. Valid choices: k1, k2, k3")
        self.kl_estimator = kl_estimator
        self.apply_clamp = apply_clamp

    def __call__(self, log_probs: torch.Tensor, log_probs_base: torch.Tensor) -> torch.Tensor:
        return self._compute_approx_kl(log_probs, log_probs_base, self.kl_estimator, self.apply_clamp)

    @staticmethod
    def _compute_approx_kl(log_probs, log_probs_base, kl_estimator: str = "k1", apply_clamp: bool = True):
        diff = log_probs.float() - log_probs_base.float()
        if kl_estimator == "k1":
            est = diff
        elif kl_estimator == "k2":
            est = diff**2 / 2.0
        elif kl_estimator == "k3":
            neg = -diff
            est = neg.exp() - 1 - neg
        else:
            raise ValueError(f"Invalid KL estimator: {kl_estimator}. Valid choices: k1, k2, k3")
        if apply_clamp:
            est = est.clamp(min=-10, max=10)
        return est
