"""``gather_logprobs`` / ``gather_logprobs_entropy`` with the reference's signatures
(``areal/utils/functional/vocab_parallel.py:564-651``), computed by one pass of the row
kernels in ``csrc/logits_rows.hip`` over materialised logits.

``chunk_size`` is accepted and ignored: the reference chunks rows to bound the fp32 copy of
the logits (``:42-62``); the kernel never makes that copy.  ``tp_group`` with more than one
rank is outside the one-GPU scope and raises.
"""

from __future__ import annotations

import math

import torch
import torch.distributed as dist

from areal_amd import _lib

_DTYPE_ID = {torch.float32: 0, torch.bfloat16: 1}


def _rows(logits: torch.Tensor) -> torch.Tensor:
    """View the logits as [T, V] rows with unit stride along V."""
    if logits.dtype not in _DTYPE_ID:
        logits = logits.float()
    v = logits.size(-1)
    rows = logits.reshape(-1, v)
    if rows.stride(-1) != 1 or (rows.size(0) > 1 and rows.stride(0) < v):
        rows = rows.contiguous()
    return rows


class _LogitsLogprobsEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, temperature, with_entropy):
        lib = _lib.load()
        dev = _lib.require_gpu(logits, labels)
        rows = _rows(logits)
        T, V = rows.shape
        lab = labels.reshape(-1).to(torch.int64).contiguous()
        lp = torch.empty(labels.shape, dtype=torch.float32, device=dev)
        ent = torch.empty(labels.shape, dtype=torch.float32, device=dev) if with_entropy else None
        lse2 = torch.empty(T, dtype=torch.float32, device=dev)
        ld = rows.stride(0) if T > 1 else V
        rc = lib.areal_logits_logprobs_entropy_fwd(
            _lib.ptr(rows), _DTYPE_ID[rows.dtype], ld, _lib.ptr(lab), T, V, 1.0 / temperature,
            _lib.ptr(lp), _lib.ptr(ent), _lib.ptr(lse2), _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_logits_logprobs_entropy_fwd")
        ctx.save_for_backward(rows, lab, lse2, ent if with_entropy else lse2)
        ctx.with_entropy = with_entropy
        ctx.temperature = temperature
        ctx.logits_shape = logits.shape
        ctx.logits_dtype = logits.dtype
        ctx.set_materialize_grads(False)
        if with_entropy:
            return lp, ent
        return lp

    @staticmethod
    def backward(ctx, grad_lp, grad_ent=None):
        rows, lab, lse2, ent = ctx.saved_tensors
        if grad_lp is None and grad_ent is None:
            return None, None, None, None
        lib = _lib.load()
        dev = rows.device
        T, V = rows.shape
        glp = grad_lp.reshape(-1).to(torch.float32).contiguous() if grad_lp is not None else None
        gen = grad_ent.reshape(-1).to(torch.float32).contiguous() if grad_ent is not None else None
        dlogits = torch.empty((T, V), dtype=rows.dtype, device=dev)
        ld = rows.stride(0) if T > 1 else V
        rc = lib.areal_logits_logprobs_entropy_bwd(
            _lib.ptr(rows), _DTYPE_ID[rows.dtype], ld, _lib.ptr(lab), T, V, 1.0 / ctx.temperature,
            _lib.ptr(lse2), _lib.ptr(ent if ctx.with_entropy else None), _lib.ptr(glp),
            _lib.ptr(gen), _lib.ptr(dlogits), V, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_logits_logprobs_entropy_bwd")
        dlogits = dlogits.view(ctx.logits_shape)
        if dlogits.dtype != ctx.logits_dtype:
            dlogits = dlogits.to(ctx.logits_dtype)
        return dlogits, None, None, None


def _validate(logits, labels, temperature, tp_group):
    if tp_group is not None and dist.is_initialized() and dist.get_world_size(tp_group) > 1:
        raise NotImplementedError("vocab-parallel logits over several GPUs are not built here")
    if not math.isfinite(temperature) or temperature <= 0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    if tuple(logits.shape[:-1]) != tuple(labels.shape):
        raise ValueError(
            "logits leading dimensions must match labels: "
            f"got {tuple(logits.shape)} and {tuple(labels.shape)}"
        )
    assert logits.numel() > 0, "Input logits must have at least one element"


def gather_logprobs(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    tp_group=None,
    chunk_size: int = 1024,
) -> torch.Tensor:
    """``log_softmax(logits.float() / temperature)[labels]`` with shape ``labels.shape``."""
    del chunk_size
    _validate(logits, labels, temperature, tp_group)
    return _LogitsLogprobsEntropy.apply(logits, labels, float(temperature), False)


def gather_logprobs_entropy(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    tp_group=None,
    chunk_size: int = 1024,
    reuse_logits: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Label log-probabilities and softmax entropy in one pass; both are differentiable,
    as on the reference's single-GPU path (``vocab_parallel.py:75-82``).

    ``reuse_logits`` asks the reference to overwrite fp32 logits in place and lets it fall back
    to the regular path otherwise (``:625-640``); this implementation needs no fp32 copy, so the
    regular path is always taken.
    """
    del chunk_size, reuse_logits
    _validate(logits, labels, temperature, tp_group)
    return _LogitsLogprobsEntropy.apply(logits, labels, float(temperature), True)
