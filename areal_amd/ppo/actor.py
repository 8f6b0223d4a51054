"""PPO actor-side callers of the kernels: the GRPO loss wrapper and advantage computation.

``grpo_loss_fn`` mirrors the call shape of ``areal/trainer/ppo/actor.py:527-760`` (which keys
it reads from ``input_data``, ``entropy.detach()``, pass-through of the vocabulary statistics)
and ``compute_advantages`` mirrors ``PPOActor._compute_advantages`` (``actor.py:178-323``).
Features of the reference that are not on this path (M2PO masking, SAPO, distillation terms,
proximal-logp approximation, turn-level GAE) raise ``NotImplementedError``.
"""

from __future__ import annotations

import math
from typing import Any

import torch

from areal_amd.config import RejectionSamplingConfig
from areal_amd.data import KLEstimator, Normalization
from areal_amd import _lib
from areal_amd.functional.aux_losses import sapo_loss_fn
from areal_amd.functional.functional import cispo_loss_fn, ppo_actor_loss_fn
from areal_amd.ppo.gae import _compute_token_level_gae

PROX_LOGP_METHOD_RECOMPUTE = "recompute"
PROX_LOGP_METHOD_REUSE_TRAIN_LOGP = "reuse_train_logp"


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
):
    """Actor loss of one packed micro-batch; returns the scalar loss.

    ``stats`` (optional dict) receives what the reference hands to its ``stats_tracker``:
    bool denominators and fp32 statistics, all of the micro-batch's token shape.
    """
    del current_version
    if input_data.get("teacher_logp") is not None:
        raise NotImplementedError("distillation terms are not part of this path")

    old_logp = input_data["logprobs"]
    advantages = input_data["advantages"]
    loss_mask = input_data["loss_mask"].bool()
    prox_logp = input_data.get("prox_logp")
    entropy = entropy.detach()

    if prox_logp_method == PROX_LOGP_METHOD_REUSE_TRAIN_LOGP:
        prox_logp = logprobs.detach()
    elif prox_logp_method != PROX_LOGP_METHOD_RECOMPUTE:
        raise NotImplementedError(f"prox_logp_method='{prox_logp_method}' is not part of this path")
    if prox_logp is None:
        raise ValueError(
            f"prox_logp is None but prox_logp_method='{prox_logp_method}'. "
            "This indicates compute_logp() was skipped incorrectly."
        )
    if torch.isnan(prox_logp).any() or torch.isinf(prox_logp).any():
        raise RuntimeError(
            f"prox_logp contains NaN or Inf with prox_logp_method='{prox_logp_method}'. "
            "This indicates computation failed."
        )

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
        )

    if stats is not None:
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
        if use_sapo_loss:
            stats.update(
                sapo_soft_gate=stat["sapo_soft_gate"],
                sapo_scaled_gate_pos=stat["sapo_scaled_gate_pos"],
                sapo_scaled_gate_neg=stat["sapo_scaled_gate_neg"],
            )
        if vocab_mean_logits is not None:
            stats["vocab_mean_logits"] = vocab_mean_logits
        if vocab_norm_logits is not None:
            stats["vocab_norm_logits"] = vocab_norm_logits
    return loss


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
    gae_lambda: float | torch.Tensor = 1.0,
    mask_no_eos_with_zero: bool = False,
    use_decoupled_loss: bool = False,
    recompute_logprob: bool = False,
    group_sizes: list[int] | None = None,
) -> dict[str, Any]:
    """Reward shaping, KL-regularised rewards, token-level GAE and advantage normalisation on a
    padded ``[bs, L]`` batch; writes ``returns, advantages, kl_rewards, tot_rewards, loss_mask,
    logprobs`` back into ``data`` exactly as ``actor.py:178-323`` does."""
    if kl_estimator is None:
        kl_estimator = KLEstimator("k1")
    bs = data["input_ids"].shape[0]
    dev = data["input_ids"].device
    batch_indices = torch.arange(bs, device=dev, dtype=torch.long)

    reward_score = (data["rewards"] + reward_bias) * reward_scaling
    reward_score = torch.clip(reward_score, max=reward_clip, min=-reward_clip)
    if reward_norm is not None:
        reward_score = reward_norm(reward_score, group_sizes=group_sizes)

    loss_mask = torch.roll(data["loss_mask"].float(), shifts=-1, dims=-1)

    if not use_decoupled_loss and recompute_logprob:
        prox = data["prox_logp"]
        if prox is None:
            raise ValueError(
                "prox_logp is None but recompute_logprob=True. "
                "This indicates compute_logp() was skipped incorrectly."
            )
        old_logp = data["logprobs"] = prox
    else:
        old_logp = torch.roll(data["logprobs"], shifts=-1, dims=-1)
        if not use_decoupled_loss:
            data["prox_logp"] = old_logp
    ref_logp = data.get("ref_logp")
    if ref_logp is None:
        ref_logp = torch.zeros_like(old_logp)
    ref_logp = ref_logp * loss_mask
    old_logp = old_logp * loss_mask

    attn_mask = data["attention_mask"]
    seqlens = attn_mask.sum(-1).long()
    seq_no_eos_mask = seqlens == attn_mask.shape[1]
    rewards = -kl_ctl * kl_estimator(old_logp, ref_logp)
    kl_rewards = rewards.clone()
    rewards[batch_indices, seqlens - 1] = 0
    gae_kl_rewards = rewards.clone()
    indices = torch.clip(seqlens - 2, min=0)
    gae_outcome_rewards = torch.zeros_like(rewards)
    if mask_no_eos_with_zero:
        gae_outcome_rewards[batch_indices, indices] = torch.where(
            seq_no_eos_mask, torch.zeros_like(reward_score), reward_score
        )
    else:
        gae_outcome_rewards[batch_indices, indices] = reward_score
    rewards = gae_kl_rewards + gae_outcome_rewards

    values = data["values"] if "values" in data else torch.zeros_like(rewards)
    if not isinstance(gae_lambda, torch.Tensor):
        gae_lambda = float(gae_lambda)
        if not math.isfinite(gae_lambda):
            raise ValueError(f"Static gae_lambda must be finite, got {gae_lambda}")
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
    data["tot_rewards"] = gae_kl_rewards + gae_outcome_rewards
    data["loss_mask"] = loss_mask
    data["logprobs"] = old_logp
    return data
