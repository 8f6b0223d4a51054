"""Oracle: reward shaping in front of GAE (CPU, test-only).

Restates ``PPOActor._compute_advantages`` lines ``areal/trainer/ppo/actor.py:215-283`` with the
same tensor ops in the same order, and the KL estimators of ``areal/utils/data.py:1662-1698``.

Pinned by (tests/test_oracle_gae_norm.py): the estimators' closed forms at hand-picked values
(k1 = d, k2 = d^2 / 2, k3 = e^-d - 1 + d, clamp to [-10, 10]); a hand-computed 2 x 5 batch for
the roll, the zero after EOS, the outcome slot max(seqlen - 2, 0), the truncated-row rule and the
index -1 of an empty row. The reference has no test of these lines on their own ("parity
unpinned" against the reference's tests; its end-to-end GAE literals pin what follows them).
"""

from __future__ import annotations

import torch


def approx_kl(log_probs, log_probs_base, kl_estimator="k1", apply_clamp=True):
    """KLEstimator._compute_approx_kl (data.py:1662-1698)."""
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


def shape_rewards(loss_mask, attention_mask, logprobs, ref_logp, reward_score, kl_ctl,
                  kl_estimator="k1", apply_clamp=True, mask_no_eos_with_zero=False, roll_logp=True):
    """actor.py:215-283: returns dict(loss_mask, old_logp, ref_logp, kl_rewards, gae_kl_rewards,
    gae_outcome_rewards, tot_rewards, seqlens, seq_no_eos_mask)."""
    bs = loss_mask.shape[0]
    idx = torch.arange(bs)
    lm = torch.roll(loss_mask.float(), shifts=-1, dims=-1)
    old = torch.roll(logprobs, shifts=-1, dims=-1) if roll_logp else logprobs.clone()
    ref = torch.zeros_like(old) if ref_logp is None else ref_logp.clone()
    ref = ref * lm
    old = old * lm
    seqlens = attention_mask.sum(-1).long()
    no_eos = seqlens == attention_mask.shape[1]
    rewards = -kl_ctl * approx_kl(old, ref, kl_estimator, apply_clamp)
    kl_rewards = rewards.clone()
    rewards[idx, seqlens - 1] = 0
    gae_kl = rewards.clone()
    indices = torch.clip(seqlens - 2, min=0)
    outcome = torch.zeros_like(rewards)
    if mask_no_eos_with_zero:
        outcome[idx, indices] = torch.where(no_eos, torch.zeros_like(reward_score), reward_score)
    else:
        outcome[idx, indices] = reward_score
    return dict(loss_mask=lm, old_logp=old, ref_logp=ref, kl_rewards=kl_rewards, gae_kl_rewards=gae_kl,
                gae_outcome_rewards=outcome, tot_rewards=gae_kl + outcome, seqlens=seqlens,
                seq_no_eos_mask=no_eos)
