"""PPO actor-side callers of the kernels: the GRPO loss wrapper and advantage computation.

``grpo_loss_fn`` mirrors ``areal/trainer/ppo/actor.py:527-760`` (which keys it reads from
``input_data``, ``entropy.detach()``, pass-through of the vocabulary statistics, every loss
branch and the logging helpers of ``:1020-1272``) and ``compute_advantages`` mirrors
``PPOActor._compute_advantages`` (``actor.py:178-323``), including turn-level GAE, per-sample
lambda functions and the overlong-response penalty.  Statistics go to an optional ``stats``
dict instead of the reference's process-wide ``stats_tracker``.
"""

from __future__ import annotations

import math
from typing import Any

import torch

from areal_amd.config import RejectionSamplingConfig
from areal_amd.data import KLEstimator, Normalization
from areal_amd import _lib
from areal_amd.functional.aux_losses import _Launch, _ScaledLoss, sapo_loss_fn
from areal_amd.functional.functional import (
    cispo_loss_fn,
    ppo_actor_loss_fn,
    reward_overlong_penalty,
)
from areal_amd.ppo.gae import (
    _compute_token_level_gae,
    _compute_turn_level_gae,
    _token_level_gae_with_row_stats,
    compute_gae_lambda,
)
from areal_amd.ppo.lambda_fn import resolve_gae_lambda_fn

# areal/utils/constants.py:36-92
PROX_LOGP_METHOD_RECOMPUTE = "recompute"
PROX_LOGP_METHOD_LOGLINEAR = "loglinear"
PROX_LOGP_METHOD_METRICS = "metrics"
PROX_LOGP_METHOD_REUSE_TRAIN_LOGP = "reuse_train_logp"
PROX_LOGP_METHODS_ALL = [
    PROX_LOGP_METHOD_RECOMPUTE, PROX_LOGP_METHOD_LOGLINEAR, PROX_LOGP_METHOD_METRICS,
    PROX_LOGP_METHOD_REUSE_TRAIN_LOGP,
]
PROX_APPROX_METHOD_LOGLINEAR = "loglinear"
PROX_APPROX_METHOD_LINEAR = "linear"
PROX_APPROX_METHOD_ROLLOUT = "rollout"
PROX_APPROX_METHODS_ALL = [PROX_APPROX_METHOD_LOGLINEAR, PROX_APPROX_METHOD_LINEAR, PROX_APPROX_METHOD_ROLLOUT]
_APPROX_ID = {PROX_APPROX_METHOD_LOGLINEAR: 0, PROX_APPROX_METHOD_LINEAR: 1, PROX_APPROX_METHOD_ROLLOUT: 2}


def grpo_loss_fn(
    logprobs: torch.Tensor,
    entropy: torch.Tensor,
    input_data: dict,
    eps_clip: float,
    eps_clip_higher: float | None,
    c_clip: float | None,
    rejection_sampling: RejectionSamplingConfig | None = None,
    m2_threshold: float | None = None,
    importance_sampling_level: str = "token",
    current_version: int | None = None,
    prox_logp_method: str = PROX_LOGP_METHOD_RECOMPUTE,
    use_sapo_loss: bool = False,
    sapo_tau_pos: float = 1.0,
    sapo_tau_neg: float = 1.05,
    use_cispo_loss: bool = False,
    use_decoupled_loss: bool = False,
    vocab_min_logits: torch.Tensor | None = None,
    vocab_max_logits: torch.Tensor | None = None,
    vocab_mean_logits: torch.Tensor | None = None,
    vocab_norm_logits: torch.Tensor | None = None,
    stats: dict | None = None,
    stats_mode: str = "tensors",
    defer_host_reads: bool = False,
):
    """Actor loss of one packed micro-batch; returns the scalar loss.

    ``defer_host_reads=True`` (PPO and CISPO losses; not in the reference): the call queues its
    kernels and returns without waiting for the GPU, so that the backward can be queued while the
    forward still runs.  Host scalars in ``stats`` are then ``DeferredFloat`` objects that wait
    when first used, reduced statistics stay in ``stats["reduction"]`` (a ``StatReduction`` whose
    ``results`` wait likewise), and a NaN or Inf in the proximal log-probs, which the reference
    reports by raising here, makes the returned loss NaN instead.

    ``stats`` (optional dict) receives what the reference hands to its ``stats_tracker``.  With
    ``stats_mode="tensors"`` these are the bool denominators and fp32 statistics of the
    micro-batch's token shape, as in the reference.  With ``stats_mode="reduced"`` (every loss
    kind) no per-token statistic tensor comes back: the loss kernel reduces every logged
    statistic under its denominator in its own pass and ``stats[key]`` is
    ``{"sum", "count", "avg", "min", "max", "denominator"}``, ``stats["denominator/<name>"]``
    the token counts (what the tracker's export computes from the clones, ``actor.py:662-733``,
    ``stats_tracker.py:455-560``).  The ``compute_logp/...`` diagnostics of the proximal
    approximations (``actor.py:1138-1226``) are functions of tensors the loss kernel does not
    see; they are evaluated as in the other mode and reduced at once by one launch of the masked
    statistics kernel, under the same denominator (``stats["denominator/compute_logp/
    n_valid_tokens"]``); the staleness statistics are host scalars in both modes.
    """
    if stats_mode not in ("tensors", "reduced"):
        raise ValueError(f"stats_mode must be 'tensors' or 'reduced', got {stats_mode!r}")
    reduction = None
    if stats is not None and stats_mode == "reduced":
        from areal_amd.functional.functional import StatReduction

        extras = {}
        if vocab_min_logits is not None and vocab_max_logits is not None:
            extras = dict(vocab_min_logits=vocab_min_logits, vocab_max_logits=vocab_max_logits)
        reduction = StatReduction(entropy=entropy, extras=extras, keep_behave_mask=True)
    if prox_logp_method not in PROX_LOGP_METHODS_ALL:
        raise ValueError(f"'{prox_logp_method}' is not a valid ProxLogpMethod")
    old_logp = input_data["logprobs"]
    advantages = input_data["advantages"]
    loss_mask = input_data["loss_mask"].bool()
    prox_logp_gt = input_data.get("prox_logp")
    entropy = entropy.detach()

    if prox_logp_method == PROX_LOGP_METHOD_REUSE_TRAIN_LOGP:
        prox_logp_gt = logprobs.detach()
    prox_logp = _resolve_proximal_logp(
        prox_logp_gt=prox_logp_gt,
        prox_logp_method=prox_logp_method,
        old_logp=old_logp,
        logprobs=logprobs.detach(),
        versions=input_data.get("versions"),
        current_version=current_version,
    )

    # The reference stops here when the proximal log-probs hold a NaN or Inf (actor.py:924-928),
    # which costs a host synchronisation before any loss kernel is queued. The same check runs
    # on the device now and is read after the loss call's own synchronisation: same error, one
    # idle gap of the GPU less per micro-batch.
    prox_nonfinite = torch.isfinite(prox_logp).logical_not().any()
    if not prox_logp.is_cuda:  # nothing to overlap with: report at once
        _raise_if_nonfinite(prox_nonfinite, prox_logp_method)

    if m2_threshold is not None:
        loss_mask = _apply_m2po_masking(old_logp, prox_logp, loss_mask, m2_threshold)

    if use_cispo_loss:
        if use_sapo_loss:
            raise ValueError(
                "CISPO and SAPO are mutually exclusive surrogates. "
                "Set at most one of use_cispo_loss / use_sapo_loss."
            )
        if importance_sampling_level != "token":
            raise ValueError(
                "CISPO only supports importance_sampling_level='token'. "
                "Sequence-level (GSPO-style) CISPO has no published surrogate."
            )
        loss, stat = cispo_loss_fn(
            logprobs=logprobs,
            proximal_logprobs=prox_logp,
            advantages=advantages,
            eps_clip=eps_clip,
            eps_clip_higher=eps_clip_higher,
            loss_mask=loss_mask,
            old_logprobs=old_logp,
            rejection_sampling=rejection_sampling,
            cu_seqlens=input_data.get("cu_seqlens"),
            stat_reduction=reduction,
            defer_host_reads=defer_host_reads,
        )
    elif use_sapo_loss:
        if use_decoupled_loss:
            raise ValueError(
                "SAPO is not compatible with `use_decoupled_loss=True`. "
                "Please set `actor.use_decoupled_loss=false` in your configuration."
            )
        loss, stat = sapo_loss_fn(
            logprobs=logprobs,
            old_logprobs=old_logp,
            advantages=advantages,
            tau_pos=sapo_tau_pos,
            tau_neg=sapo_tau_neg,
            loss_mask=loss_mask,
            importance_sampling_level=importance_sampling_level,
            cu_seqlens=input_data.get("cu_seqlens"),
            stat_reduction=reduction,
        )
    else:
        loss, stat = ppo_actor_loss_fn(
            logprobs=logprobs,
            old_logprobs=old_logp,
            advantages=advantages,
            eps_clip=eps_clip,
            eps_clip_higher=eps_clip_higher,
            loss_mask=loss_mask,
            c_clip=c_clip,
            proximal_logprobs=prox_logp,
            rejection_sampling=rejection_sampling,
            importance_sampling_level=importance_sampling_level,
            cu_seqlens=input_data.get("cu_seqlens"),
            stat_reduction=reduction,
            defer_host_reads=defer_host_reads,
        )

    if defer_host_reads and not use_sapo_loss:
        loss = loss + torch.where(prox_nonfinite, float("nan"), 0.0).to(loss.dtype)
    else:
        _raise_if_nonfinite(prox_nonfinite, prox_logp_method)

    # joint distillation (actor.py:629-658)
    teacher_logp = input_data.get("teacher_logp")
    rkl_stat = None
    if teacher_logp is not None:
        rl_loss_weight = input_data.get("rl_loss_weight", 1.0)
        distill_loss_weight = input_data.get("distill_loss_weight", 0.005)
        pure_kd = rl_loss_weight == 0
        value, term = _distill_term(logprobs, old_logp, teacher_logp.detach(), loss_mask, pure_kd)
        if pure_kd:
            loss = (-1 * distill_loss_weight) * value
            rkl_stat = -1 * term
        else:
            loss = rl_loss_weight * loss + distill_loss_weight * value
            rkl_stat = term

    if reduction is not None:
        defer = defer_host_reads and not use_sapo_loss
        if defer:
            stats["reduction"] = reduction
        else:
            stats.update(reduction.results)
            for name, count in reduction.denominators.items():
                stats["denominator/" + name] = count
        # the compute_logp diagnostics: per-token tensors as in the other mode, reduced right away
        from areal_amd.stats import masked_stats

        lp = logprobs.detach()
        diag_mask = reduction.behave_mask if reduction.behave_mask is not None else loss_mask
        diag: dict = {}
        _collect_proximal_approximation_stats(
            diag, prox_logp_method, prox_logp_gt, old_logp, lp, input_data.get("versions"),
            current_version, diag_mask.view(loss_mask.shape),
        )
        den = diag.pop("compute_logp/n_valid_tokens")
        if diag:
            reduced = masked_stats(diag, {k: den for k in diag}, defer=defer)
            if defer:
                stats["compute_logp_reduction"] = reduced
            else:
                for k, v in reduced.items():
                    stats[k] = dict(v, denominator="compute_logp/n_valid_tokens")
                stats["denominator/compute_logp/n_valid_tokens"] = next(iter(reduced.values()))["count"]
        if "versions" in input_data and current_version is not None and not defer:
            _collect_version_staleness_stats(stats, input_data["versions"], current_version, diag_mask.view(loss_mask.shape))
        if vocab_mean_logits is not None or vocab_norm_logits is not None:
            more = {k: v for k, v in (("vocab_mean_logits", vocab_mean_logits), ("vocab_norm_logits", vocab_norm_logits))
                    if v is not None}
            extra = masked_stats(more, {k: None for k in more}, defer=defer)
            if defer:
                stats["vocab_moments_reduction"] = extra
            else:
                for k, v in extra.items():
                    stats[k] = dict(v, denominator="n_tokens")
        for key in ("n_total_tokens", "n_valid_tokens", "n_masked_tokens", "masked_token_ratio"):
            if key in stat:
                stats["scalar/" + key] = stat[key]
        if "filtered_fraction" in stat:
            stats["scalar/rs_filtered_fraction"] = stat["filtered_fraction"]
        if rkl_stat is not None:
            stats["rkl_loss"] = rkl_stat
    elif stats is not None:
        lp = logprobs.detach()
        logp_diff = (old_logp - lp) * loss_mask
        stats.update(
            n_valid_tokens=loss_mask,
            clipped_tokens=stat["clip_mask"],
            dual_clipped_tokens=stat["dual_clip_mask"],
            importance_weight=stat["importance_weight"],
            approx_kl=stat["approx_kl"],
            new_logp=lp,
            old_logp=old_logp,
            entropy=entropy.float(),
            actor_loss=stat["loss"],
            clip_ratio=stat["clip_mask"].float(),
            dual_clip_ratio=stat["dual_clip_mask"].float(),
            logp_diff=logp_diff,
            logp_abs_diff=logp_diff.abs(),
        )
        if "behave_imp_weight" in stat:
            stats.update(
                unclipped_behave_tokens=stat["behave_mask"],
                behave_imp_weight=stat["behave_imp_weight"],
                behave_approx_kl=stat["behave_approx_kl"],
                behave_filtered_ratio=(loss_mask & ~stat["behave_mask"]).float(),
            )
        for key in ("n_total_tokens", "n_valid_tokens", "n_masked_tokens", "masked_token_ratio"):
            if key in stat:
                stats["scalar/" + key] = stat[key]
        if "filtered_fraction" in stat:
            stats["scalar/rs_filtered_fraction"] = stat["filtered_fraction"]
        if vocab_min_logits is not None and vocab_max_logits is not None:
            stats.update(vocab_min_logits=vocab_min_logits, vocab_max_logits=vocab_max_logits)
        if rkl_stat is not None:
            stats["rkl_loss"] = rkl_stat
        if use_sapo_loss:
            stats.update(
                sapo_soft_gate=stat["sapo_soft_gate"],
                sapo_scaled_gate_pos=stat["sapo_scaled_gate_pos"],
                sapo_scaled_gate_neg=stat["sapo_scaled_gate_neg"],
            )
        compute_logp_mask = stat.get("behave_mask", loss_mask)
        _collect_proximal_approximation_stats(
            stats, prox_logp_method, prox_logp_gt, old_logp, lp, input_data.get("versions"),
            current_version, compute_logp_mask,
        )
        if "versions" in input_data and current_version is not None:
            _collect_version_staleness_stats(stats, input_data["versions"], current_version, compute_logp_mask)
        if vocab_mean_logits is not None:
            stats["vocab_mean_logits"] = vocab_mean_logits
        if vocab_norm_logits is not None:
            stats["vocab_norm_logits"] = vocab_norm_logits
    return loss


def compute_prox_logp_approximations(
    old_logp: torch.Tensor,
    logprobs: torch.Tensor,
    versions: torch.Tensor,
    current_version: int,
    method: str | None = None,
) -> dict[str, torch.Tensor]:
    """Version-aware approximations of the proximal policy's log-probs (``actor.py:768-848``):
    one key if ``method`` is given, all three methods otherwise."""
    lib = _lib.load()
    shape = old_logp.shape
    old = old_logp.detach().to(torch.float32).contiguous().view(-1)
    lp = logprobs.detach().to(torch.float32).contiguous().view(-1)
    ver = versions.detach().to(torch.int64).contiguous().view(-1)
    dev = _lib.require_gpu(old, lp, ver)
    out = {}
    for m in ([method] if method else PROX_APPROX_METHODS_ALL):
        if m not in _APPROX_ID:
            continue
        res = torch.empty(old.numel(), dtype=torch.float32, device=dev)
        rc = lib.areal_prox_logp_approx(
            _lib.ptr(old), _lib.ptr(lp), _lib.ptr(ver), old.numel(), int(current_version),
            _APPROX_ID[m], _lib.ptr(res), _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_prox_logp_approx")
        out[m] = res.view(shape)
    return out


def _raise_if_nonfinite(flag: torch.Tensor, prox_logp_method: str) -> None:
    if bool(flag):
        raise RuntimeError(
            f"prox_logp contains NaN or Inf with prox_logp_method='{prox_logp_method}'. "
            "This indicates computation failed."
        )


def _resolve_proximal_logp(prox_logp_gt, prox_logp_method, old_logp, logprobs, versions, current_version):
    """Proximal log-probs to train with: the recomputed ones, or the log-linear approximation
    when the forward pass was skipped (``actor.py:851-930``; same errors)."""
    prox_logp_is_none = prox_logp_gt is None
    if prox_logp_is_none:
        if prox_logp_method not in (PROX_LOGP_METHOD_LOGLINEAR, PROX_LOGP_METHOD_REUSE_TRAIN_LOGP):
            raise ValueError(
                f"prox_logp is None but prox_logp_method='{prox_logp_method}'. "
                "This indicates compute_logp() was skipped incorrectly."
            )
        if versions is None:
            raise ValueError(
                f"prox_logp is None with prox_logp_method='{prox_logp_method}' "
                "but versions not available. "
                "Cannot proceed without either ground truth or approximation."
            )
    prox_logp = prox_logp_gt
    if prox_logp_method == PROX_LOGP_METHOD_LOGLINEAR:
        if prox_logp_is_none and versions is not None and current_version is not None:
            prox_logp = compute_prox_logp_approximations(
                old_logp, logprobs, versions, current_version, PROX_APPROX_METHOD_LOGLINEAR
            )[PROX_APPROX_METHOD_LOGLINEAR]
    if prox_logp is None:
        raise RuntimeError(
            f"prox_logp is None after handling prox_logp_method='{prox_logp_method}'. "
            "This indicates configuration or computation error."
        )
    return prox_logp


def _distill_term(logprobs, old_logp, teacher_logp, loss_mask, pure_kd: bool):
    """``sum(term) / max(count, 1)`` (differentiable w.r.t. ``logprobs``) and the per-token term:
    ``(logprobs - teacher) * mask`` for the joint loss, ``exp(logprobs - old) * (teacher -
    logprobs.detach()) * mask`` for pure distillation (``actor.py:640-656``)."""
    lib = _lib.load()
    shape = logprobs.shape
    f32 = lambda t: t.detach().to(torch.float32).contiguous().view(-1)  # noqa: E731
    old, teacher = f32(old_logp), f32(teacher_logp)
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    dev = _lib.require_gpu(logprobs, old, teacher, mask_bool)
    n = int(mask_bool.numel())

    def launch(want_grad: bool):
        out = {
            "loss": torch.empty((), dtype=torch.float32, device=dev),
            "dsum": torch.empty(n, dtype=torch.float32, device=dev) if want_grad else None,
            "term": torch.empty(n, dtype=torch.float32, device=dev),
            "counters": torch.empty(8, dtype=torch.float64, device=dev),
        }
        nbytes = lib.areal_aux_loss_workspace_bytes(n, 0)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_distill_terms(
            _lib.ptr(f32(logprobs)), _lib.ptr(old), _lib.ptr(teacher), _lib.ptr(mask_bool), n,
            int(pure_kd), _lib.ptr(out["loss"]), _lib.ptr(out["dsum"]), _lib.ptr(out["term"]),
            _lib.ptr(out["counters"]), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_distill_terms")
        return out

    runner = _Launch(launch)
    value = _ScaledLoss.apply(logprobs, runner)
    return value, runner.out["term"].view(shape)


_EPSILON = 1e-8


def _approximation_errors(ground_truth, approximation):
    diff = ground_truth - approximation
    return {
        "abs_error": torch.abs(diff).float(),
        "rel_error": torch.abs(diff / (torch.abs(ground_truth) + _EPSILON)).float(),
        "squared_error": (diff * diff).float(),
    }


def _collect_proximal_approximation_stats(
    stats, prox_logp_method, prox_logp_gt, old_logp, logprobs, versions, current_version, mask
):
    """What ``_log_proximal_approximation_stats`` (``actor.py:1138-1226``) hands to the tracker's
    ``compute_logp`` scope, as ``compute_logp/<key>`` entries of ``stats`` (logging only)."""
    pre = "compute_logp/"
    stats[pre + "n_valid_tokens"] = mask.bool()
    if prox_logp_gt is not None:
        stats[pre + "prox_logp_gt"] = prox_logp_gt.float()
    if versions is None or current_version is None:
        return
    gt = None
    if prox_logp_method == PROX_LOGP_METHOD_LOGLINEAR:
        approximations = compute_prox_logp_approximations(
            old_logp, logprobs, versions, current_version, PROX_APPROX_METHOD_LOGLINEAR
        )
    elif prox_logp_method == PROX_LOGP_METHOD_METRICS and prox_logp_gt is not None:
        approximations = compute_prox_logp_approximations(old_logp, logprobs, versions, current_version, None)
        gt = prox_logp_gt
    else:
        approximations = {}
    for name, approx in approximations.items():
        behave_w = torch.exp(approx - old_logp).float()
        imp_w = torch.exp(logprobs - approx).float()
        stats[f"{pre}{name}/approx_logp"] = approx.float()
        stats[f"{pre}{name}/behave_imp_weight"] = behave_w
        stats[f"{pre}{name}/importance_weight"] = imp_w
        if gt is not None:
            for k, v in _approximation_errors(gt, approx).items():
                stats[f"{pre}{name}/{k}"] = v
            be = _approximation_errors(torch.exp(gt - old_logp).float(), behave_w)
            ie = _approximation_errors(torch.exp(logprobs - gt).float(), imp_w)
            stats[f"{pre}{name}/behave_imp_weight_abs_error"] = be["abs_error"]
            stats[f"{pre}{name}/behave_imp_weight_rel_error"] = be["rel_error"]
            stats[f"{pre}{name}/importance_weight_abs_error"] = ie["abs_error"]
            stats[f"{pre}{name}/importance_weight_rel_error"] = ie["rel_error"]
    log_ratio = (logprobs.float() - old_logp.float()).detach()
    stats[pre + "kl_div_direct"] = -log_ratio
    stats[pre + "kl_div_taylor"] = log_ratio**2 / 2.0
    stats[pre + "kl_div_dual"] = log_ratio.exp() - 1 - log_ratio


def _collect_version_staleness_stats(stats, versions, current_version, mask):
    """The scalars of ``_log_version_staleness_stats`` (``actor.py:1229-1272``) as
    ``scalar/version_stats/<key>`` entries of ``stats``: one reduction launch, one host copy."""
    from areal_amd.stats import masked_stats

    v_behave = versions.float()
    generated = mask.bool() & (versions >= 0)
    res = masked_stats(
        {"proximal": (current_version - 1) - v_behave, "theta": current_version - v_behave},
        {"proximal": generated, "theta": generated},
    )
    if res["proximal"]["count"] == 0:
        return
    pre = "scalar/version_stats/"
    for name in ("proximal", "theta"):
        for k in ("avg", "max", "min"):
            stats[f"{pre}sample_staleness_{name}_{k}"] = res[name][k]
    stats[pre + "v_theta"] = current_version
    stats[pre + "v_proximal"] = current_version - 1
    stats[pre + "n_valid_generated_tokens"] = int(res["proximal"]["count"])


def _apply_m2po_masking(
    old_logp: torch.Tensor,
    prox_logp: torch.Tensor,
    loss_mask: torch.Tensor,
    m2_threshold: float,
) -> torch.Tensor:
    """M2PO (second-moment PPO) masking: drop the tokens with the largest
    ``(old_logp - prox_logp)**2`` until the mean over the remaining masked tokens is below
    ``m2_threshold``; at least one token of a non-empty mask stays
    (``areal/trainer/ppo/actor.py:933-1014``).  The reference sorts; the kernel finds the cut
    with a radix select, and keeps tokens that tie at the cut value in index order."""
    lib = _lib.load()
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    old = old_logp.detach().to(torch.float32).contiguous().view(-1)
    prox = prox_logp.detach().to(torch.float32).contiguous().view(-1)
    dev = _lib.require_gpu(old, prox, mask_bool)
    n = int(mask_bool.numel())
    out = torch.empty(n, dtype=torch.bool, device=dev)
    if n > 0:
        nbytes = lib.areal_m2po_mask_workspace_bytes(n)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_m2po_mask(
            _lib.ptr(old), _lib.ptr(prox), _lib.ptr(mask_bool), n, float(m2_threshold),
            _lib.ptr(out), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_m2po_mask")
    return out.view_as(loss_mask)


def compute_advantages(
    data: dict[str, Any],
    *,
    kl_ctl: float = 0.0,
    kl_estimator: KLEstimator | None = None,
    reward_bias: float = 0.0,
    reward_scaling: float = 1.0,
    reward_clip: float = 20.0,
    reward_norm: Normalization | None = None,
    adv_norm: Normalization | None = None,
    discount: float = 1.0,
    gae_lambda: float | str | torch.Tensor = 1.0,
    mask_no_eos_with_zero: bool = False,
    use_decoupled_loss: bool = False,
    recompute_logprob: bool = False,
    group_sizes: list[int] | None = None,
    gae_timestep_unit: str = "token",
    gae_lambda_fn=None,
    gae_lambda_kwargs: dict | None = None,
    overlong_reward_penalty: bool = False,
    overlong_tokens: int | None = None,
    overlong_penalty_factor: float | None = None,
    max_new_tokens: int | None = None,
) -> dict[str, Any]:
    """Reward shaping, KL-regularised rewards, token- or turn-level GAE and advantage
    normalisation on a padded ``[bs, L]`` batch; writes ``returns, advantages, kl_rewards,
    tot_rewards, loss_mask, logprobs`` back into ``data`` exactly as ``actor.py:178-323`` does.
    ``gae_lambda`` is a number, a ``[bs]`` tensor, or (as in the reference's configuration,
    ``actor.py:84-91``) the dotted path of a per-sample lambda function, which
    ``areal_amd.ppo.lambda_fn.resolve_gae_lambda_fn`` imports; ``gae_lambda_fn`` passes such a
    function ``fn(context, **kwargs) -> [bs] tensor`` directly.  Either way it is called with
    ``gae_lambda_kwargs`` on the batch's length context."""
    if gae_timestep_unit not in ("token", "turn"):
        raise ValueError(f"gae_timestep_unit must be 'token' or 'turn', got {gae_timestep_unit!r}")
    if kl_estimator is None:
        kl_estimator = KLEstimator("k1")
    bs = data["input_ids"].shape[0]
    dev = data["input_ids"].device

    if overlong_reward_penalty:
        assert overlong_tokens is not None
        assert overlong_penalty_factor is not None
        data = reward_overlong_penalty(
            data,
            overlong_tokens=overlong_tokens,
            overlong_penalty_factor=overlong_penalty_factor,
            max_response_length=max_new_tokens,
        )

    reward_score = (data["rewards"] + reward_bias) * reward_scaling
    reward_score = torch.clip(reward_score, max=reward_clip, min=-reward_clip)
    if reward_norm is not None:
        reward_score = reward_norm(reward_score, group_sizes=group_sizes)

    # structural turn ids follow the same next-token convention as the mask and the log-probs
    turn_ids = data.get("turn_ids")
    if turn_ids is not None:
        turn_ids = torch.roll(turn_ids, shifts=-1, dims=-1)
        turn_ids[:, -1] = -1
    elif gae_timestep_unit == "turn":
        raise ValueError(
            "actor.gae_timestep_unit='turn' requires rollout data to "
            "include 'turn_ids'."
        )

    recompute = not use_decoupled_loss and recompute_logprob
    if recompute:
        logp_src = data["prox_logp"]
        if logp_src is None:
            raise ValueError(
                "prox_logp is None but recompute_logprob=True. "
                "This indicates compute_logp() was skipped incorrectly."
            )
    else:
        logp_src = data["logprobs"]
    # One pass (areal_advantage_prep) instead of the reference's chain of tensor ops
    # (actor.py:215-283): rolled float mask, masked old / reference log-probs, KL rewards, their
    # copy zeroed after EOS, the outcome reward at the second-to-last token, and their sum. The
    # reference's in-place updates are kept: `old_logp *= loss_mask` also masks the tensor that
    # prox_logp names (and, in the recompute branch, the caller's prox_logp itself), and
    # `ref_logp *= loss_mask` masks the caller's ref_logp.
    lib = _lib.load()
    _lib.require_gpu(logp_src, data["loss_mask"], data["attention_mask"])
    L = logp_src.shape[-1]

    def as_bytes(t):
        t = t.reshape(bs, L)
        t = t if t.dtype == torch.bool else t != 0
        return t.contiguous().view(torch.uint8)

    def in_place_ok(t):
        return t.dtype == torch.float32 and t.is_contiguous() and not t.requires_grad

    f32 = dict(dtype=torch.float32, device=dev)
    logp_in = logp_src.detach().reshape(bs, L)
    if not in_place_ok(logp_in):
        logp_in = logp_in.float().contiguous()
    old_logp = logp_in if (recompute and in_place_ok(logp_src)) else torch.empty((bs, L), **f32)
    ref_src = data.get("ref_logp")
    ref_in = None
    ref_in_place = False
    if ref_src is not None:
        ref_in_place = in_place_ok(ref_src)
        ref_in = ref_src.reshape(bs, L) if ref_in_place else ref_src.detach().float().contiguous().reshape(bs, L)
    turn_mode = gae_timestep_unit == "turn"
    loss_mask = torch.empty((bs, L), **f32)
    kl_rewards = torch.empty((bs, L), **f32)
    tot_rewards = torch.empty((bs, L), **f32)
    gae_kl_rewards = torch.empty((bs, L), **f32) if turn_mode else None
    gae_outcome_rewards = torch.empty((bs, L), **f32) if turn_mode else None
    seqlens = torch.empty(bs, dtype=torch.int64, device=dev)
    seq_no_eos_mask = torch.empty(bs, dtype=torch.bool, device=dev)
    if getattr(kl_estimator, "kl_estimator", None) not in ("k1", "k2", "k3"):
        raise TypeError("kl_estimator must be a KLEstimator (k1, k2 or k3)")
    est = {"k1": 1, "k2": 2, "k3": 3}[kl_estimator.kl_estimator]
    # temporaries are named so that they outlive the launch (a freed block is handed to the next
    # allocation at once)
    lm_bytes, am_bytes = as_bytes(data["loss_mask"]), as_bytes(data["attention_mask"])
    score_f = reward_score.float().contiguous()
    rc = lib.areal_advantage_prep(
        _lib.ptr(lm_bytes), _lib.ptr(am_bytes),
        _lib.ptr(logp_in), _lib.ptr(ref_in), _lib.ptr(score_f), bs, L,
        0 if recompute else 1, est, int(bool(kl_estimator.apply_clamp)), int(bool(mask_no_eos_with_zero)),
        int(ref_in_place), float(kl_ctl), _lib.ptr(loss_mask), _lib.ptr(old_logp), _lib.ptr(kl_rewards),
        _lib.ptr(gae_kl_rewards), _lib.ptr(gae_outcome_rewards), _lib.ptr(tot_rewards),
        _lib.ptr(seqlens), _lib.ptr(seq_no_eos_mask), _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_advantage_prep")
    old_logp = old_logp.view(logp_src.shape)
    if recompute:
        data["logprobs"] = old_logp
        if old_logp.data_ptr() == logp_src.data_ptr():
            data["prox_logp"] = old_logp
    elif not use_decoupled_loss:
        data["prox_logp"] = old_logp
    # turn mode keeps the token KL as a local actor penalty instead of summing it into turns
    rewards = gae_outcome_rewards if turn_mode else tot_rewards

    values = data["values"] if "values" in data else torch.zeros_like(rewards)
    if gae_lambda_fn is None and isinstance(gae_lambda, (str, bool)):
        gae_lambda_fn, _ = resolve_gae_lambda_fn(gae_lambda)
    if gae_lambda_fn is not None:
        gae_lambda = compute_gae_lambda(gae_lambda_fn, gae_lambda_kwargs, loss_mask, turn_ids, gae_timestep_unit)
    elif not isinstance(gae_lambda, torch.Tensor):
        gae_lambda = float(gae_lambda)
        if not math.isfinite(gae_lambda):
            raise ValueError(f"Static gae_lambda must be finite, got {gae_lambda}")
    if gae_timestep_unit == "turn":
        advantages, returns = _compute_turn_level_gae(
            rewards=rewards,
            values=values,
            loss_mask=loss_mask,
            turn_ids=turn_ids,
            seq_no_eos_mask=seq_no_eos_mask,
            discount=discount,
            gae_lambda=gae_lambda,
        )
        advantages = advantages + gae_kl_rewards
    else:
        # With long padded rows and a normalisation that needs one statistics pass, the GAE kernel
        # sums each row's advantages under the mask while it writes them, and the normalisation
        # is its apply pass alone: two launches for the two stages (same results).
        fused = None
        if isinstance(adv_norm, Normalization) and adv_norm.needs_one_statistics_pass() and rewards.ndim == 2:
            fused = _token_level_gae_with_row_stats(rewards, values, loss_mask, seq_no_eos_mask, discount, gae_lambda)
        if fused is not None:
            advantages, returns, row_stats, mask_f32 = fused
            normed = adv_norm.from_row_stats(advantages, mask_f32, row_stats, group_sizes=group_sizes)
            if normed is not None:
                advantages, adv_norm = normed, None
        else:
            advantages, returns = _compute_token_level_gae(
                rewards=rewards,
                values=values,
                loss_mask=loss_mask,
                seq_no_eos_mask=seq_no_eos_mask,
                discount=discount,
                gae_lambda=gae_lambda,
            )
    data["returns"] = returns
    if adv_norm is not None:
        advantages = adv_norm(advantages, loss_mask, group_sizes=group_sizes)

    data["advantages"] = advantages
    data["kl_rewards"] = kl_rewards
    data["tot_rewards"] = tot_rewards
    data["loss_mask"] = loss_mask
    data["logprobs"] = old_logp
    return data
