"""Oracle: rejection sampling, PPO/GRPO and CISPO actor losses (CPU, test-only).

Restates, with plain differentiable torch ops (so autograd gives the reference's gradient):
  * ``areal/utils/functional/functional.py:185-437`` apply_rejection_sampling, with
    ``_check_bounds`` (:167-182) and ``compute_binary_kl_divergence`` (:440-449);
  * ``areal/utils/data.py:1662-1698`` KLEstimator._compute_approx_kl (k1/k2/k3, no clamp here);
  * ``functional.py:56-149`` sequence-level (GSPO) ratio and mean advantage;
  * ``functional.py:452-596`` ppo_actor_loss_fn and ``:678-793`` cispo_loss_fn.

Every elementwise expression keeps the reference's operation order and dtypes so that the
boolean outputs are the reference's bit for bit.

Pinned by (tests/test_oracle_loss.py): the reference tests' literals for ratio bounds,
geometric-mean sequence filtering, k1/k2/k3 values, clamp mode, sum/max aggregation, boundary
and non-finite cases; the CISPO 6-token fixture with its exact gradient; the GSPO literals
exp(0.5), exp(1.0), exp(1.5) and loss -1.5; the five-case closed-form PPO gradient.
``binary_kl`` has no reference test: pinned by the Bernoulli KL closed form in float64 and the
fp32 case log p = 0 -> NaN -> rejected.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class RSResult:
    loss_mask: torch.Tensor
    behave_imp_weight: torch.Tensor
    filtered_fraction: float


def binary_kl(log_p: torch.Tensor, log_q: torch.Tensor, eps: float = 1e-8) -> torch.Tensor:
    """Bernoulli KL(P||Q) from log-probabilities (functional.py:440-449)."""
    p = torch.clamp(torch.exp(log_p), eps, 1.0 - eps)
    q = torch.clamp(torch.exp(log_q), eps, 1.0 - eps)
    return p * torch.log(p / q) + (1 - p) * torch.log((1 - p) / (1 - q))


def approx_kl(log_probs, log_probs_base, kind: str) -> torch.Tensor:
    """k1/k2/k3 estimators without clamping (data.py:1677-1694)."""
    d = log_probs.float() - log_probs_base.float()
    if kind == "k1":
        return d
    if kind == "k2":
        return d**2 / 2.0
    if kind == "k3":
        n = -d
        return n.exp() - 1 - n
    raise ValueError(kind)


def _within(metric, lower, upper):
    if lower is not None:
        return (metric >= lower) & (metric <= upper)
    return metric <= upper


def _sequence_index(cu_seqlens: torch.Tensor) -> torch.Tensor:
    lens = cu_seqlens[1:] - cu_seqlens[:-1]
    return torch.arange(lens.numel()).repeat_interleave(lens.long())


def _per_sequence(values, mask_bool, seq_idx, n_seqs, how: str):
    """Masked per-sequence sum / mean / max of a packed 1-D tensor; count clamped to >= 1 for
    the mean; all-masked sequences give 0 for max (functional.py:285-334)."""
    zeros = torch.zeros(n_seqs, dtype=values.dtype)
    cnt_raw = torch.zeros(n_seqs, dtype=torch.int32).scatter_add_(0, seq_idx, mask_bool.int())
    cnt = cnt_raw.clamp(min=1)
    masked = torch.where(mask_bool, values, 0.0)
    if how == "sum":
        return zeros.scatter_add_(0, seq_idx, masked)
    if how == "mean":
        return zeros.scatter_add_(0, seq_idx, masked) / cnt.to(values.dtype)
    if how == "max":
        neg = values.masked_fill(~mask_bool, float("-inf"))
        out = torch.full((n_seqs,), float("-inf"), dtype=values.dtype).scatter_reduce_(
            0, seq_idx, neg, reduce="amax"
        )
        return torch.where(cnt_raw == 0, torch.zeros_like(out), out)
    raise ValueError(f"Unknown agg method: {how}")


def rejection_sampling(
    prox, old, loss_mask, cu_seqlens, *, level="token", action="mask", metric="ratio",
    agg="mean", upper=5.0, lower=None,
) -> RSResult:
    """apply_rejection_sampling (functional.py:185-437)."""
    if action == "clamp" and lower is None:
        lower = 0.0  # RejectionSamplingConfig.__post_init__, cli_args.py:1657-1658
    log_ratio = prox.detach().float() - old.detach().float()
    log_ratio = torch.where(torch.isfinite(log_ratio), log_ratio, 0.0)
    if metric == "ratio":
        m = torch.exp(log_ratio)
    elif metric in ("kl_k1", "kl_k2", "kl_k3"):
        m = approx_kl(prox.detach(), old.detach(), metric[3:])
    elif metric == "binary_kl":
        m = torch.maximum(binary_kl(prox.detach(), old.detach()), binary_kl(old.detach(), prox.detach()))
    else:
        raise ValueError(f"Unknown metric: {metric}")
    w = torch.exp(log_ratio)
    w_before = w
    geometric = metric == "ratio"
    mask_bool = loss_mask.bool()
    in_bounds = None
    if level == "sequence":
        agg_src = log_ratio if geometric else m
        if loss_mask.ndim == 1:
            if cu_seqlens is None:
                raise ValueError("cu_seqlens is required for 1D packed tensors in sequence-level filtering.")
            n_seqs = cu_seqlens.numel() - 1
            idx = _sequence_index(cu_seqlens)
            if geometric:
                w = torch.exp(_per_sequence(log_ratio, mask_bool, idx, n_seqs, "mean"))[idx]
                w_before = w
            seq_agg = _per_sequence(agg_src, mask_bool, idx, n_seqs, agg)
            seq_metric = torch.exp(seq_agg) if geometric else seq_agg
            ok_seq = _within(seq_metric, lower, upper)
            ok_tok = ok_seq[idx]
        else:
            masked = torch.where(mask_bool, agg_src, 0.0)
            cnt = loss_mask.sum(dim=-1, keepdim=True).clamp(min=1)
            if geometric:
                w = torch.exp(masked.sum(-1, keepdim=True) / cnt).expand_as(log_ratio)
                w_before = w
            if agg == "sum":
                seq_agg = masked.sum(-1, keepdim=True)
            elif agg == "mean":
                seq_agg = masked.sum(-1, keepdim=True) / cnt
            elif agg == "max":
                seq_agg = agg_src.masked_fill(~mask_bool, float("-inf")).max(-1, keepdim=True)[0]
                empty = loss_mask.sum(-1, keepdim=True) == 0
                seq_agg = torch.where(empty, torch.zeros_like(seq_agg), seq_agg)
            else:
                raise ValueError(f"Unknown agg method: {agg}")
            seq_metric = torch.exp(seq_agg) if geometric else seq_agg
            ok_tok = _within(seq_metric, lower, upper).expand_as(loss_mask)
        if action == "mask":
            in_bounds = ok_tok
        else:
            w = torch.where(~ok_tok, w.clamp(min=lower, max=upper), w)
    else:
        if action == "mask":
            in_bounds = _within(m, lower, upper)
        else:
            w = w.clamp(min=lower, max=upper)

    if action == "mask":
        new_mask = (mask_bool & in_bounds).to(loss_mask.dtype)
        filtered = (mask_bool & ~in_bounds).sum().item()
    else:
        new_mask = loss_mask
        filtered = (mask_bool & (w_before != w)).sum().item()
    frac = filtered / max(mask_bool.sum().item(), 1)
    w = torch.where(new_mask.bool(), w, 0.0)
    return RSResult(new_mask, w, frac)


def sequence_ratio_and_advantages(log_ratio, advantages, loss_mask, cu_seqlens):
    """Geometric-mean ratio and mean advantage per sequence, broadcast to tokens, zero outside
    the mask (functional.py:56-149)."""
    if log_ratio.ndim == 1:
        if cu_seqlens is None:
            raise ValueError("cu_seqlens is required for 1D tensors (packed format).")
        n_seqs = cu_seqlens.numel() - 1
        idx = _sequence_index(cu_seqlens)
        cnt = torch.zeros(n_seqs, dtype=torch.int32).scatter_add_(0, idx, loss_mask.int()).clamp(min=1)
        lr_sum = torch.zeros(n_seqs, dtype=log_ratio.dtype).scatter_add(
            0, idx, torch.where(loss_mask, log_ratio, 0.0)
        )
        adv_sum = torch.zeros(n_seqs, dtype=advantages.dtype).scatter_add(
            0, idx, torch.where(loss_mask, advantages, 0.0)
        )
        ratio = torch.exp(lr_sum / cnt.to(log_ratio.dtype))[idx]
        adv = (adv_sum / cnt.to(advantages.dtype))[idx]
    else:
        cnt = loss_mask.sum(dim=1, keepdim=True).clamp(min=1)
        ratio = torch.exp(torch.where(loss_mask, log_ratio, 0.0).sum(1, keepdim=True) / cnt).expand_as(log_ratio)
        adv = (torch.where(loss_mask, advantages, 0.0).sum(-1, keepdim=True) / cnt).expand_as(log_ratio)
    return torch.where(loss_mask, ratio, 0.0), torch.where(loss_mask, adv, 0.0)


def ppo_actor_loss(
    logprobs, proximal_logprobs, old_logprobs, advantages, eps_clip, loss_mask,
    eps_clip_higher=None, c_clip=None, rejection_sampling_cfg: dict | None = None,
    importance_sampling_level="token", cu_seqlens=None,
):
    """ppo_actor_loss_fn (functional.py:452-596). ``rejection_sampling_cfg`` holds the keyword
    arguments of :func:`rejection_sampling` (level, action, metric, agg, upper, lower)."""
    n0 = loss_mask.count_nonzero() or 1
    stat_mask = loss_mask
    rs = None
    if rejection_sampling_cfg is not None:
        rs = rejection_sampling(proximal_logprobs, old_logprobs, loss_mask, cu_seqlens, **rejection_sampling_cfg)
        loss_mask = rs.loss_mask
    if importance_sampling_level == "sequence":
        ratio, advantages = sequence_ratio_and_advantages(
            logprobs - proximal_logprobs, advantages, loss_mask, cu_seqlens
        )
    elif importance_sampling_level == "token":
        ratio = torch.where(stat_mask, torch.exp(logprobs - proximal_logprobs), 0)
    else:
        raise ValueError(f"Invalid importance_sampling_level: {importance_sampling_level}.")
    hi = eps_clip if eps_clip_higher is None else eps_clip_higher
    clipped = torch.clamp(ratio, 1.0 - eps_clip, 1.0 + hi)
    pg1 = -advantages * ratio
    pg2 = -advantages * clipped
    clip_mask = pg1.detach() < pg2.detach()
    pg = torch.max(pg1, pg2)
    if c_clip is not None:
        assert c_clip > 1.0, c_clip
        pg3 = torch.sign(advantages) * c_clip * advantages
        dual = pg3.detach() < pg.detach()
        pg = torch.min(pg, pg3)
    else:
        dual = torch.zeros_like(clip_mask)
    stat = {}
    if rs is not None:
        bkl = proximal_logprobs.detach() - old_logprobs.detach()
        bmask = (rs.behave_imp_weight > 0).logical_and(loss_mask.bool())
        pg = pg * rs.behave_imp_weight
        stat.update(
            behave_approx_kl=torch.where(bmask, bkl, 0.0), behave_imp_weight=rs.behave_imp_weight,
            behave_mask=bmask, filtered_fraction=rs.filtered_fraction,
        )
    token_loss = pg.detach()
    loss = torch.where(loss_mask, pg, 0).sum() / n0
    n_total = stat_mask.numel()
    n_valid = stat_mask.count_nonzero().item()
    stat.update(
        loss=token_loss, importance_weight=ratio.detach(),
        approx_kl=(logprobs - proximal_logprobs).detach(),
        clip_mask=clip_mask & stat_mask, dual_clip_mask=dual & stat_mask,
        n_total_tokens=float(n_total), n_valid_tokens=float(n_valid),
        n_masked_tokens=float(n_total - n_valid),
        masked_token_ratio=1.0 - n_valid / max(n_total, 1),
        new_mask=loss_mask,
    )
    return loss, stat


def cispo_loss(
    logprobs, proximal_logprobs, advantages, eps_clip, loss_mask, eps_clip_higher=None,
    old_logprobs=None, rejection_sampling_cfg: dict | None = None, cu_seqlens=None,
):
    """cispo_loss_fn (functional.py:678-793)."""
    if eps_clip_higher is None or eps_clip_higher <= 0:
        raise ValueError(f"CISPO requires a positive eps_clip_higher; Got {eps_clip_higher!r}.")
    n0 = loss_mask.count_nonzero() or 1
    rs = None
    if rejection_sampling_cfg is not None:
        rs = rejection_sampling(proximal_logprobs, old_logprobs, loss_mask, cu_seqlens, **rejection_sampling_cfg)
        loss_mask = rs.loss_mask
    advantages = advantages.detach()
    log_ratio = (logprobs - proximal_logprobs).detach()
    ratio = torch.exp(log_ratio)
    rc = torch.clamp(ratio, 1.0 - eps_clip, 1.0 + eps_clip_higher).detach()
    pg = -rc * advantages * logprobs
    stat = {}
    if rs is not None:
        bkl = proximal_logprobs.detach() - old_logprobs.detach()
        bmask = (rs.behave_imp_weight > 0).logical_and(loss_mask.bool())
        pg = pg * rs.behave_imp_weight
        stat.update(
            behave_approx_kl=torch.where(bmask, bkl, 0.0), behave_imp_weight=rs.behave_imp_weight,
            behave_mask=bmask, filtered_fraction=rs.filtered_fraction,
        )
    token_loss = pg.detach()
    loss = torch.where(loss_mask, pg, 0).sum() / n0
    stat.update(
        loss=token_loss, importance_weight=ratio, approx_kl=log_ratio,
        clip_mask=(rc != ratio).logical_and(loss_mask),
        dual_clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool), new_mask=loss_mask,
    )
    return loss, stat


def ppo_closed_form_grad(logprobs, prox, adv, mask_kept, n0, lo, hi, c_clip=None, weight=None):
    """d loss / d logprobs of the token-level clipped surrogate without autograd:
    -A * ratio where the unclipped branch is active (or tied), times the dual-clip keep factor,
    times the behaviour weight, masked, divided by the pre-rejection token count."""
    ratio = torch.exp(logprobs - prox)
    clipped = ratio.clamp(lo, hi)
    pg1, pg2 = -adv * ratio, -adv * clipped
    in_band = ((ratio >= lo) & (ratio <= hi)).float()
    g1 = (pg1 > pg2).float() + 0.5 * (pg1 == pg2).float()
    g2 = (pg2 > pg1).float() + 0.5 * (pg1 == pg2).float()
    d = -adv * (g1 + g2 * in_band) * ratio
    if c_clip is not None:
        pg = torch.maximum(pg1, pg2)
        pg3 = torch.sign(adv) * c_clip * adv
        d = d * ((pg < pg3).float() + 0.5 * (pg == pg3).float())
    if weight is not None:
        d = d * weight
    return torch.where(mask_kept, d, 0.0) / n0
