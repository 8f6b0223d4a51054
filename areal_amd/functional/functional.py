"""Actor-loss stage of the hot path: same Python signatures as the reference's
``areal/utils/functional/functional.py`` (``masked_normalization`` :16-53,
``apply_rejection_sampling`` :185-437, ``ppo_actor_loss_fn`` :452-596, ``cispo_loss_fn``
:678-793), computed by the HIP kernels of ``csrc/ppo_loss.hip`` and ``csrc/gae_norm.hip``.

Argument checking (types of exception and their messages) happens here, before any device
work, and follows the reference.  Every call performs exactly one device-to-host copy (the
eight counters of the loss kernel), where the reference performs one to three ``.item()``
synchronisations.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from areal_amd import _lib
from areal_amd.config import RejectionSamplingConfig

_METRIC_ID = {"ratio": 0, "kl_k1": 1, "kl_k2": 2, "kl_k3": 3, "binary_kl": 4}
_AGG_ID = {"sum": 0, "mean": 1, "max": 2}
LOSS_NONE, LOSS_PPO, LOSS_CISPO = -1, 0, 1


@dataclass
class RejectionSamplingResult:
    """Result of rejection sampling (fields as in ``functional.py:152-164``)."""

    loss_mask: torch.Tensor
    behave_imp_weight: torch.Tensor
    filtered_fraction: float


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(torch.float32).contiguous().view(-1)


# Order of the statistics areal_actor_loss_stats reduces (include/areal_hip.h) and the
# denominator each is taken under.
REDUCED_STAT_KEYS = (
    ("importance_weight", "n_valid_tokens"), ("approx_kl", "n_valid_tokens"),
    ("new_logp", "n_valid_tokens"), ("old_logp", "n_valid_tokens"), ("entropy", "n_valid_tokens"),
    ("actor_loss", "n_valid_tokens"), ("clip_ratio", "n_valid_tokens"),
    ("dual_clip_ratio", "n_valid_tokens"), ("logp_diff", "n_valid_tokens"),
    ("logp_abs_diff", "n_valid_tokens"), ("behave_filtered_ratio", "n_valid_tokens"),
    ("behave_imp_weight", "unclipped_behave_tokens"), ("behave_approx_kl", "unclipped_behave_tokens"),
    ("clipped_new_logp", "clipped_tokens"), ("clipped_old_logp", "clipped_tokens"),
    ("extra0", "n_tokens"), ("extra1", "n_tokens"),
)
# The same for areal_sapo_loss's stats output.
SAPO_REDUCED_STAT_KEYS = (
    ("importance_weight", "n_valid_tokens"), ("approx_kl", "n_valid_tokens"),
    ("new_logp", "n_valid_tokens"), ("old_logp", "n_valid_tokens"), ("entropy", "n_valid_tokens"),
    ("actor_loss", "n_valid_tokens"), ("logp_diff", "n_valid_tokens"),
    ("logp_abs_diff", "n_valid_tokens"), ("sapo_soft_gate", "n_valid_tokens"),
    ("sapo_scaled_gate_pos", "n_valid_tokens"), ("sapo_scaled_gate_neg", "n_valid_tokens"),
    ("extra0", "n_tokens"), ("extra1", "n_tokens"),
)


class _HostCopy:
    """A small device tensor on its way to pinned host memory: queued behind the kernels that
    write it, waited for when the host first looks at it."""

    def __init__(self, dev_tensor: torch.Tensor):
        self._host = torch.empty(dev_tensor.shape, dtype=dev_tensor.dtype, pin_memory=True)
        self._host.copy_(dev_tensor, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record(torch.cuda.current_stream(dev_tensor.device))

    def host(self) -> torch.Tensor:
        self._event.synchronize()
        return self._host


class DeferredFloat:
    """A host scalar of a loss call made with ``defer_host_reads=True``: the device-to-host copy
    it comes from is waited for when the value is first used as a number (``float(x)``,
    arithmetic, comparison, formatting), not when the loss function returns."""

    __slots__ = ("_source", "_fn", "_value")

    def __init__(self, source: _HostCopy, fn):
        self._source, self._fn, self._value = source, fn, None

    def __float__(self) -> float:
        if self._value is None:
            self._value = float(self._fn(self._source.host()))
        return self._value

    def __repr__(self) -> str:
        return repr(float(self))

    def __format__(self, spec: str) -> str:
        return format(float(self), spec)

    def __bool__(self) -> bool:
        return bool(float(self))

    def __eq__(self, other) -> bool:
        return float(self) == other

    def __lt__(self, other) -> bool:
        return float(self) < other

    def __le__(self, other) -> bool:
        return float(self) <= other

    def __gt__(self, other) -> bool:
        return float(self) > other

    def __ge__(self, other) -> bool:
        return float(self) >= other

    def __add__(self, other):
        return float(self) + other

    __radd__ = __add__

    def __sub__(self, other):
        return float(self) - other

    def __rsub__(self, other):
        return other - float(self)

    def __mul__(self, other):
        return float(self) * other

    __rmul__ = __mul__

    def __truediv__(self, other):
        return float(self) / other

    def __rtruediv__(self, other):
        return other / float(self)


def _host_value(c, fn):
    """``fn(counters)`` as a float now, or as a ``DeferredFloat`` when the counters are still on
    their way to the host."""
    return DeferredFloat(c, fn) if isinstance(c, _HostCopy) else float(fn(c))


class StatReduction:
    """Ask a loss call to reduce its logged statistics inside the kernel's token pass.

    The reference logs about 25 per-token tensors per micro-batch through ``stats_tracker``
    (each cloned, ``areal/utils/stats_tracker.py:133-171``) and reduces each under its
    denominator mask at export (``:455-560``).  A loss call given a ``StatReduction`` writes none
    of those ``[T]`` tensors: the token kernel accumulates sum, min and max of every statistic
    in registers and ``results`` receives, after the call, ``{key: {"sum", "count", "avg",
    "min", "max"}}`` (``avg`` / ``min`` / ``max`` are ``None`` under an empty denominator, as
    the tracker's ``_avg_of`` / ``_min_of`` / ``_max_of`` return) and ``denominators``
    ``{name: count}``.  The returned ``stat`` dict then holds the host scalars only.

    ``entropy`` and up to two ``extras`` (``{name: tensor}``, reduced over every token, e.g. the
    vocabulary min / max logits) are optional per-token inputs that ride along in the same pass.
    """

    def __init__(self, entropy: torch.Tensor | None = None, extras: dict[str, torch.Tensor] | None = None,
                 keep_behave_mask: bool = False):
        extras = dict(extras or {})
        if len(extras) > 2:
            raise ValueError(f"at most two extra statistics ride along, got {len(extras)}")
        self.entropy = entropy
        self.extras = extras
        # the one per-token output a caller may still need (1 byte per token): the tokens that pass
        # rejection sampling with a positive weight, the denominator of the diagnostics that
        # grpo_loss_fn reduces in a launch of their own
        self.keep_behave_mask = keep_behave_mask
        self.behave_mask: torch.Tensor | None = None
        self._results: dict[str, dict[str, float | None]] = {}
        self._denominators: dict[str, float] = {}
        self._pending = None  # (host copy, arguments of _fill) of a call with deferred host reads

    def _resolve(self) -> None:
        if self._pending is not None:
            copy, n_tokens, has_rs, has_old = self._pending
            self._pending = None
            host = copy.host()
            self._fill(host[8:].view(-1, 4), host[:8], n_tokens, has_rs, has_old)

    def _fill_sapo(self, host: torch.Tensor, counters, n_tokens: int) -> None:
        """Results of ``areal_sapo_loss``'s reduction. SAPO clips nothing: the clip ratios are
        zero on every token of the mask and the clipped-token statistics are empty."""
        self._fill(host, counters, n_tokens, False, True, keys=SAPO_REDUCED_STAT_KEYS)
        nv = float(counters[1])
        zero = dict(sum=0.0, count=nv, avg=None if nv == 0 else 0.0, min=None if nv == 0 else 0.0,
                    max=None if nv == 0 else 0.0, denominator="n_valid_tokens")
        self._results["clip_ratio"] = dict(zero)
        self._results["dual_clip_ratio"] = dict(zero)

    @property
    def results(self) -> dict[str, dict[str, float | None]]:
        self._resolve()
        return self._results

    @property
    def denominators(self) -> dict[str, float]:
        self._resolve()
        return self._denominators

    def _fill(self, host: torch.Tensor, counters, n_tokens: int, has_rs: bool, has_old: bool,
              keys=REDUCED_STAT_KEYS) -> None:
        names = list(self.extras)
        for i, (key, denom) in enumerate(keys):
            if key == "entropy" and self.entropy is None:
                continue
            if key.startswith("behave_") and not has_rs:
                continue
            if key in ("old_logp", "logp_diff", "logp_abs_diff", "clipped_old_logp") and not has_old:
                continue
            if key.startswith("extra"):
                j = int(key[-1])
                if j >= len(names):
                    continue
                key = names[j]
            s, c, mn, mx = host[i].tolist()
            empty = c == 0
            self._results[key] = dict(sum=s, count=c, avg=None if empty else s / c,
                                     min=None if empty else mn, max=None if empty else mx,
                                     denominator=denom)
        self._denominators = dict(n_tokens=float(n_tokens), n_valid_tokens=float(counters[1]),
                                  clipped_tokens=float(counters[4]), dual_clipped_tokens=float(counters[5]))
        if has_rs:
            self._denominators["unclipped_behave_tokens"] = float(counters[6])


def _fill_rs(cfg: _lib.LossConfig, rs: RejectionSamplingConfig | None) -> None:
    if rs is None:
        cfg.rs_enabled = 0
        return
    if rs.metric not in _METRIC_ID:
        raise ValueError(f"Unknown metric: {rs.metric}")
    if rs.agg not in _AGG_ID:
        raise ValueError(f"Unknown agg method: {rs.agg}")
    cfg.rs_enabled = 1
    cfg.rs_seq_level = int(rs.level == "sequence")
    cfg.rs_clamp = int(rs.action != "mask")
    cfg.rs_metric = _METRIC_ID[rs.metric]
    cfg.rs_agg = _AGG_ID[rs.agg]
    cfg.rs_upper = rs.upper
    cfg.rs_has_lower = int(rs.lower is not None)
    cfg.rs_lower = rs.lower if rs.lower is not None else 0.0


def _sequence_layout(shape, cu_seqlens, device):
    """(cu_seqlens int32 tensor or None, n_seqs, uniform_len) for a 1-D or 2-D batch."""
    if len(shape) == 2:
        return None, int(shape[0]), int(shape[1])
    cu = cu_seqlens.to(device=device, dtype=torch.int32).contiguous()
    return cu, int(cu.numel() - 1), 0


def _run_loss_kernel(
    cfg: _lib.LossConfig,
    shape,
    logprobs,
    proximal,
    old,
    advantages,
    mask_bool,
    cu_seqlens,
    want_grad: bool,
    reduction: "StatReduction | None" = None,
):
    """Launch ``areal_actor_loss`` (or, with a ``reduction``, ``areal_actor_loss_stats`` without
    the per-token statistic tensors) and return its outputs and the device counters."""
    lib = _lib.load()
    dev = _lib.require_gpu(proximal, mask_bool, logprobs, old, advantages)
    n = int(mask_bool.numel())
    need_seq = (cfg.rs_enabled and cfg.rs_seq_level) or (cfg.loss_kind == LOSS_PPO and cfg.seq_is)
    cu, n_seqs, uniform_len = (None, 0, 0)
    if need_seq:
        cu, n_seqs, uniform_len = _sequence_layout(shape, cu_seqlens, dev)
    has_loss = cfg.loss_kind != LOSS_NONE
    f32 = dict(dtype=torch.float32, device=dev)
    u8 = dict(dtype=torch.bool, device=dev)
    if reduction is not None:
        return _run_loss_kernel_reduced(lib, dev, cfg, n, n_seqs, uniform_len, cu, logprobs, proximal, old,
                                        advantages, mask_bool, want_grad, reduction)
    out = {
        "loss": torch.empty((), **f32) if has_loss else None,
        "dlp": torch.empty(n, **f32) if (has_loss and want_grad) else None,
        "stat_loss": torch.empty(n, **f32) if has_loss else None,
        "ratio": torch.empty(n, **f32) if has_loss else None,
        "approx_kl": torch.empty(n, **f32) if has_loss else None,
        "clip_mask": torch.empty(n, **u8) if has_loss else None,
        "dual_clip_mask": torch.empty(n, **u8) if (has_loss and cfg.loss_kind == LOSS_PPO) else None,
        "new_mask": torch.empty(n, **u8) if cfg.rs_enabled else None,
        "behave_imp_weight": torch.empty(n, **f32) if cfg.rs_enabled else None,
        "behave_approx_kl": torch.empty(n, **f32) if (cfg.rs_enabled and has_loss) else None,
        "behave_mask": torch.empty(n, **u8) if (cfg.rs_enabled and has_loss) else None,
    }
    counters = torch.empty(8, dtype=torch.float64, device=dev)
    nbytes = lib.areal_actor_loss_workspace_bytes(n, n_seqs)
    ws = _lib.workspace(nbytes, dev)
    rc = lib.areal_actor_loss(
        _lib.ptr(logprobs), _lib.ptr(proximal), _lib.ptr(old), _lib.ptr(advantages),
        _lib.ptr(mask_bool), _lib.ptr(cu), n, n_seqs, uniform_len, ctypes.byref(cfg),
        _lib.ptr(out["loss"]), _lib.ptr(out["dlp"]), _lib.ptr(out["stat_loss"]),
        _lib.ptr(out["ratio"]), _lib.ptr(out["approx_kl"]), _lib.ptr(out["clip_mask"]),
        _lib.ptr(out["dual_clip_mask"]), _lib.ptr(out["new_mask"]),
        _lib.ptr(out["behave_imp_weight"]), _lib.ptr(out["behave_approx_kl"]),
        _lib.ptr(out["behave_mask"]), _lib.ptr(counters), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_actor_loss")
    out["counters_dev"] = counters
    return out


def _run_loss_kernel_reduced(lib, dev, cfg, n, n_seqs, uniform_len, cu, logprobs, proximal, old,
                             advantages, mask_bool, want_grad, reduction):
    """The loss pass with the statistics reduced in the kernel: the only per-token outputs are
    the gradient and, for the sequence-level importance ratio under rejection sampling, the
    narrowed mask and behaviour weight that the per-sequence pass reads back."""
    f32 = dict(dtype=torch.float32, device=dev)
    need_seq_io = bool(cfg.rs_enabled and cfg.loss_kind == LOSS_PPO and cfg.seq_is)
    out = {k: None for k in ("stat_loss", "ratio", "approx_kl", "clip_mask", "dual_clip_mask", "new_mask",
                             "behave_imp_weight", "behave_approx_kl", "behave_mask")}
    out["loss"] = torch.empty((), **f32)
    out["dlp"] = torch.empty(n, **f32) if want_grad else None
    if need_seq_io:
        out["new_mask"] = torch.empty(n, dtype=torch.bool, device=dev)
        out["behave_imp_weight"] = torch.empty(n, **f32)
    if reduction.keep_behave_mask and cfg.rs_enabled:
        out["behave_mask"] = reduction.behave_mask = torch.empty(n, dtype=torch.bool, device=dev)
    # counters [8] and stats [17][4] share one buffer: one device-to-host copy serves both
    n_stats = len(REDUCED_STAT_KEYS)
    both = torch.empty(8 + 4 * n_stats, dtype=torch.float64, device=dev)
    counters, stats = both[:8], both[8:]
    extras = [_f32(t) for t in reduction.extras.values()]
    for t in extras:
        if t.numel() != n:
            raise ValueError(f"extra statistic has {t.numel()} elements, expected {n}")
    ent = _f32(reduction.entropy) if reduction.entropy is not None else None
    if ent is not None and ent.numel() != n:
        raise ValueError(f"entropy has {ent.numel()} elements, expected {n}")
    nbytes = lib.areal_actor_loss_stats_workspace_bytes(n, n_seqs)
    ws = _lib.workspace(nbytes, dev)
    rc = lib.areal_actor_loss_stats(
        _lib.ptr(logprobs), _lib.ptr(proximal), _lib.ptr(old), _lib.ptr(advantages),
        _lib.ptr(mask_bool), _lib.ptr(cu), n, n_seqs, uniform_len, ctypes.byref(cfg),
        _lib.ptr(ent), _lib.ptr(extras[0] if len(extras) > 0 else None),
        _lib.ptr(extras[1] if len(extras) > 1 else None),
        _lib.ptr(out["loss"]), _lib.ptr(out["dlp"]), None, None, None, None, None,
        _lib.ptr(out["new_mask"]), _lib.ptr(out["behave_imp_weight"]), None, _lib.ptr(out["behave_mask"]),
        _lib.ptr(counters), _lib.ptr(stats), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_actor_loss_stats")
    out["counters_dev"] = counters
    out["counters_and_stats_dev"] = both
    return out


class _ActorLoss(torch.autograd.Function):
    """loss = sum(where(mask', pg, 0)) / N0 with the closed-form gradient w.r.t. logprobs."""

    @staticmethod
    def forward(ctx, logprobs, cfg, shape, proximal, old, advantages, mask_bool, cu_seqlens, sink,
                reduction=None):
        want_grad = logprobs.requires_grad
        lp = _f32(logprobs)
        out = _run_loss_kernel(cfg, shape, lp, proximal, old, advantages, mask_bool, cu_seqlens,
                               want_grad, reduction)
        sink.update(out)
        if want_grad:
            ctx.save_for_backward(out["dlp"], out["counters_dev"])
        ctx.shape = logprobs.shape
        ctx.in_dtype = logprobs.dtype
        return out["loss"]

    @staticmethod
    def backward(ctx, grad_loss):
        dlp, counters = ctx.saved_tensors
        lib = _lib.load()
        dev = dlp.device
        g = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        grad = torch.empty_like(dlp)
        rc = lib.areal_actor_loss_grad(
            _lib.ptr(dlp), _lib.ptr(g), _lib.ptr(counters), _lib.ptr(grad), dlp.numel(),
            _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_actor_loss_grad")
        grad = grad.view(ctx.shape)
        if ctx.in_dtype != torch.float32:
            grad = grad.to(ctx.in_dtype)
        return (grad,) + (None,) * 9


def _check_rs_shapes(proximal_logprobs, old_logprobs, loss_mask):
    if proximal_logprobs.shape != old_logprobs.shape:
        raise ValueError(
            f"proximal_logprobs shape {proximal_logprobs.shape} != "
            f"old_logprobs shape {old_logprobs.shape}"
        )
    if proximal_logprobs.shape != loss_mask.shape:
        raise ValueError(
            f"proximal_logprobs shape {proximal_logprobs.shape} != "
            f"loss_mask shape {loss_mask.shape}"
        )
    if proximal_logprobs.ndim not in (1, 2):
        raise ValueError(
            f"Expected 1D (packed) or 2D (padded) tensors, got ndim={proximal_logprobs.ndim}"
        )


def _check_rs_sequences(config, loss_mask, cu_seqlens):
    if config.level == "sequence" and loss_mask.ndim == 1 and cu_seqlens is None:
        raise ValueError(
            "cu_seqlens is required for 1D packed tensors in sequence-level filtering."
        )


def apply_rejection_sampling(
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    loss_mask: torch.Tensor,
    cu_seqlens: torch.Tensor | None,
    config: RejectionSamplingConfig,
) -> RejectionSamplingResult:
    """Filter (``action='mask'``) or truncate (``action='clamp'``) tokens / sequences whose
    divergence between proximal and behaviour policy leaves the configured bounds.

    Same contract as ``functional.py:185-437``: the returned mask has the dtype of the input
    mask; ``filtered_fraction`` is a Python float.
    """
    _check_rs_shapes(proximal_logprobs, old_logprobs, loss_mask)
    cfg = _lib.LossConfig()
    cfg.loss_kind = LOSS_NONE
    _fill_rs(cfg, config)
    _check_rs_sequences(config, loss_mask, cu_seqlens)
    shape = loss_mask.shape
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    out = _run_loss_kernel(
        cfg, shape, None, _f32(proximal_logprobs), _f32(old_logprobs), None, mask_bool,
        cu_seqlens, False,
    )
    c = out["counters_dev"].cpu()
    n_valid, n_filtered = float(c[1]), float(c[3])
    if config.action == "mask":
        new_mask = out["new_mask"].view(shape).to(loss_mask.dtype)
    else:
        new_mask = loss_mask
    return RejectionSamplingResult(
        loss_mask=new_mask,
        behave_imp_weight=out["behave_imp_weight"].view(shape),
        filtered_fraction=n_filtered / max(n_valid, 1.0),
    )


def _loss_common(cfg, logprobs, proximal_logprobs, old_logprobs, advantages, loss_mask,
                 rejection_sampling, cu_seqlens, reduction=None, defer=False):
    shape = logprobs.shape
    if rejection_sampling is not None:
        _check_rs_shapes(proximal_logprobs, old_logprobs, loss_mask)
        _check_rs_sequences(rejection_sampling, loss_mask, cu_seqlens)
    _fill_rs(cfg, rejection_sampling)
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    sink: dict = {}
    # the behaviour log-probs enter the kernel for rejection sampling and, with a reduction,
    # for the old_logp / logp_diff statistics
    want_old = rejection_sampling is not None or (reduction is not None and old_logprobs is not None)
    loss = _ActorLoss.apply(
        logprobs, cfg, shape, _f32(proximal_logprobs),
        _f32(old_logprobs) if want_old else None,
        _f32(advantages), mask_bool, cu_seqlens, sink, reduction,
    )
    if defer:
        # no host synchronisation in this call: the copy is queued and whoever reads a host
        # scalar (or the reduction's results) waits for it then
        if reduction is None:
            c = _HostCopy(sink["counters_dev"])
        else:
            c = _HostCopy(sink["counters_and_stats_dev"])
            reduction._pending = (c, int(mask_bool.numel()), rejection_sampling is not None, want_old)
    elif reduction is None:
        c = sink["counters_dev"].cpu()  # the one host synchronisation of the call
    else:
        host = sink["counters_and_stats_dev"].cpu()  # counters and reduced statistics, one copy
        c = host[:8]
        reduction._fill(host[8:].view(-1, 4), c, int(mask_bool.numel()), rejection_sampling is not None,
                        want_old)
    return loss, sink, c, shape


def _scalar_stats(loss_mask, c):
    n_total = float(loss_mask.numel())
    return dict(
        n_total_tokens=n_total,
        n_valid_tokens=_host_value(c, lambda h: h[1]),
        n_masked_tokens=_host_value(c, lambda h: n_total - float(h[1])),
        masked_token_ratio=_host_value(c, lambda h: 1.0 - float(h[1]) / max(n_total, 1.0)),
    )


def _filtered_fraction(c):
    return _host_value(c, lambda h: float(h[3]) / max(float(h[1]), 1.0))


def _rs_stats(stat, sink, c, shape, rejection_sampling):
    if rejection_sampling is None:
        return
    stat.update(
        behave_approx_kl=sink["behave_approx_kl"].view(shape),
        behave_imp_weight=sink["behave_imp_weight"].view(shape),
        behave_mask=sink["behave_mask"].view(shape),
        filtered_fraction=_filtered_fraction(c),
    )


def ppo_actor_loss_fn(
    logprobs: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: RejectionSamplingConfig | None = None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
    stat_reduction: StatReduction | None = None,
    defer_host_reads: bool = False,
) -> tuple[torch.Tensor, dict]:
    """PPO/GRPO clipped surrogate with optional dual clip, GSPO sequence-level ratio and
    rejection sampling.  Signature, return structure and ``stat`` keys as in
    ``functional.py:452-596``.  ``stat_reduction`` (not in the reference): reduce the logged
    statistics in the kernel instead of returning per-token tensors, see ``StatReduction``.
    ``defer_host_reads`` (not in the reference): the call does not wait for the GPU; the host
    scalars of ``stat`` are ``DeferredFloat`` objects that wait when they are first used."""
    if importance_sampling_level == "sequence":
        if logprobs.ndim == 1 and cu_seqlens is None:
            raise ValueError(
                "cu_seqlens is required for 1D tensors (packed format). "
                "In AReaL, 1D tensors are produced by pack_tensor_dict() and always have "
                "cu_seqlens. For a single sequence, use "
                "cu_seqlens=torch.tensor([0, seq_len], dtype=torch.int32)."
            )
    elif importance_sampling_level != "token":
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. "
            "Must be 'token' or 'sequence'."
        )
    if c_clip is not None:
        assert c_clip > 1.0, c_clip
    cfg = _lib.LossConfig()
    cfg.loss_kind = LOSS_PPO
    cfg.clip_lo = 1.0 - eps_clip
    cfg.clip_hi = 1.0 + (eps_clip if eps_clip_higher is None else eps_clip_higher)
    cfg.has_c_clip = int(c_clip is not None)
    cfg.c_clip = c_clip if c_clip is not None else 0.0
    cfg.seq_is = int(importance_sampling_level == "sequence")
    loss, sink, c, shape = _loss_common(
        cfg, logprobs, proximal_logprobs, old_logprobs, advantages, loss_mask,
        rejection_sampling, cu_seqlens, stat_reduction, defer_host_reads,
    )
    if stat_reduction is not None:
        stat = _scalar_stats(loss_mask, c)
        if rejection_sampling is not None:
            stat["filtered_fraction"] = _filtered_fraction(c)
        return loss, stat
    stat = dict(
        loss=sink["stat_loss"].view(shape),
        importance_weight=sink["ratio"].view(shape),
        approx_kl=sink["approx_kl"].view(shape),
        clip_mask=sink["clip_mask"].view(shape),
        dual_clip_mask=sink["dual_clip_mask"].view(shape),
        **_scalar_stats(loss_mask, c),
    )
    _rs_stats(stat, sink, c, shape, rejection_sampling)
    return loss, stat


def cispo_loss_fn(
    logprobs: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    old_logprobs: torch.Tensor | None = None,
    rejection_sampling: RejectionSamplingConfig | None = None,
    cu_seqlens: torch.Tensor | None = None,
    stat_reduction: StatReduction | None = None,
    defer_host_reads: bool = False,
) -> tuple[torch.Tensor, dict]:
    """CISPO: clipped importance weight under stop-gradient times ``log pi`` (MiniMax-M1).
    Signature, errors and ``stat`` keys as in ``functional.py:678-793``; ``stat_reduction`` and
    ``defer_host_reads`` as in ``ppo_actor_loss_fn``."""
    if eps_clip_higher is None or eps_clip_higher <= 0:
        raise ValueError(
            "CISPO requires a positive eps_clip_higher; the asymmetric upper "
            f"clip is the defining knob (MiniMax-M1 Eq. 4-5). Got {eps_clip_higher!r}."
        )
    cfg = _lib.LossConfig()
    cfg.loss_kind = LOSS_CISPO
    cfg.clip_lo = 1.0 - eps_clip
    cfg.clip_hi = 1.0 + eps_clip_higher
    loss, sink, c, shape = _loss_common(
        cfg, logprobs, proximal_logprobs, old_logprobs, advantages, loss_mask,
        rejection_sampling, cu_seqlens, stat_reduction, defer_host_reads,
    )
    if stat_reduction is not None:
        stat = {}
        if rejection_sampling is not None:
            stat["filtered_fraction"] = _filtered_fraction(c)
        return loss, stat
    stat = dict(
        loss=sink["stat_loss"].view(shape),
        importance_weight=sink["ratio"].view(shape),
        approx_kl=sink["approx_kl"].view(shape),
        clip_mask=sink["clip_mask"].view(shape),
        dual_clip_mask=torch.zeros(shape, dtype=torch.bool, device=logprobs.device),
    )
    _rs_stats(stat, sink, c, shape, rejection_sampling)
    return loss, stat


@torch.no_grad()
def masked_normalization(
    x: torch.Tensor,
    mask: torch.Tensor | None = None,
    dim=None,
    unbiased=False,
    eps=1e-5,
    high_precision=True,
    all_reduce=True,
    reduce_group=None,
):
    """Whiten ``x`` over its masked elements (``functional.py:16-53``): fp64 sums,
    ``var = E[x^2] - E[x]^2``, ``(x * mask - mean) / (sqrt(var) + eps)``, over all dimensions or
    over the dimensions in ``dim`` (every slice along the others gets its own statistics).

    The sums are fp64 whatever ``high_precision`` says; a multi-rank ``all_reduce`` is outside
    the one-GPU scope.
    """
    import torch.distributed as dist

    if all_reduce and dist.is_initialized() and dist.get_world_size(reduce_group) > 1:
        raise NotImplementedError("masked_normalization runs on one GPU; no all_reduce")
    del high_precision
    if mask is not None and mask.shape != x.shape:
        raise ValueError(f"mask must have the shape of x, got {tuple(mask.shape)} and {tuple(x.shape)}")
    lib = _lib.load()
    dev = _lib.require_gpu(x, mask)
    if dim is not None:
        dims = sorted({d % x.ndim for d in ((dim,) if isinstance(dim, int) else tuple(dim))})
    else:
        dims = list(range(x.ndim))
    if len(dims) < x.ndim:
        # reduced dimensions last: [rows, cols], one row per slice along the kept dimensions
        kept = [d for d in range(x.ndim) if d not in dims]
        perm = kept + dims
        xp = x.to(torch.float32).permute(perm).contiguous()
        mp = mask.to(torch.float32).permute(perm).contiguous() if mask is not None else None
        rows = 1
        for d in kept:
            rows *= x.shape[d]
        cols = xp.numel() // max(rows, 1)
        outp = torch.empty_like(xp)
        rc = lib.areal_masked_norm_rows(
            _lib.ptr(xp), _lib.ptr(mp), rows, cols, int(bool(unbiased)), float(eps), _lib.ptr(outp),
            _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_masked_norm_rows")
        inverse = [perm.index(d) for d in range(x.ndim)]
        return outp.permute(inverse).contiguous()
    xf = x.to(torch.float32).contiguous()
    mf = mask.to(torch.float32).contiguous() if mask is not None else None
    out = torch.empty_like(xf)
    n = xf.numel()
    nbytes = lib.areal_masked_norm_workspace_bytes(n)
    ws = _lib.workspace(nbytes, dev)
    rc = lib.areal_masked_norm(
        _lib.ptr(xf), _lib.ptr(mf), n, int(bool(unbiased)), float(eps), _lib.ptr(out),
        _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_masked_norm")
    return out


def reward_overlong_penalty(
    data: dict,
    overlong_tokens: int,
    overlong_penalty_factor: float,
    max_response_length: int,
) -> dict:
    """DAPO's soft penalty for responses that run into the last ``overlong_tokens`` tokens of the
    budget (``functional.py:937-959``): ``rewards[i] += min(-(len_i - (max_response_length -
    overlong_tokens)) / overlong_tokens * overlong_penalty_factor, 0)`` with ``len_i`` the number
    of loss-mask tokens of sample ``i``. ``data["rewards"]`` is updated in place, as in the
    reference; its per-sample Python loop is one vector expression here."""
    rewards = data["rewards"]
    response_lengths = data["loss_mask"].sum(dim=-1).long()
    exceed = response_lengths - (max_response_length - overlong_tokens)
    penalty = torch.clamp(-exceed / overlong_tokens * overlong_penalty_factor, max=0)
    rewards += penalty.to(rewards.dtype)
    data["rewards"] = rewards
    return data

