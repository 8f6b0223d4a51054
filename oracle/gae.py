"""Oracle: token-level GAE (CPU, test-only).

``gae_padded`` restates ``areal/trainer/ppo/gae.py:10-36`` (fp32 recurrence over the columns of
padded ``[bs, L]`` tensors).  ``gae_packed`` is the same recurrence run per sequence of a packed
batch; it equals ``gae_padded`` on the padded form of the same data when the mask is zero on
padding (checked in tests/test_oracle_gae.py), which is how the packed kernel is tied to the
reference.

Pinned by: the reference's exact literals [[0.25,0.5,1.0,0.0],[0,0,1,0]] for per-sample lambda,
the closed form A_t = sum_k (gamma*lambda)^k delta_{t+k} on an unmasked sequence, the bootstrap
case (no_eos), and masked positions carrying the state through unchanged.
"""

from __future__ import annotations

import torch


def gae_padded(rewards, values, loss_mask, seq_no_eos_mask, discount, gae_lambda):
    bs, width = rewards.shape
    rev = [torch.zeros(bs, dtype=torch.float32)]
    last = torch.zeros(bs, dtype=torch.float32)
    nxt = values[:, width - 1] * seq_no_eos_mask
    c = discount * gae_lambda
    for t in reversed(range(width - 1)):
        delta = rewards[:, t] + discount * nxt - values[:, t]
        cand = delta + c * last
        m = loss_mask[:, t]
        keep = 1 - m
        nxt = nxt * keep + values[:, t] * m
        last = last * keep + cand * m
        rev.append(last)
    adv = torch.stack(rev[::-1], dim=1)
    return adv, adv + values


def gae_packed(rewards, values, loss_mask, cu_seqlens, seq_no_eos_mask, discount, gae_lambda):
    """Run ``gae_padded`` on each sequence ``[cu[i], cu[i+1])`` of 1-D packed tensors."""
    adv = torch.zeros_like(values, dtype=torch.float32)
    n_seqs = cu_seqlens.numel() - 1
    for i in range(n_seqs):
        s, e = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        if e <= s:
            continue
        lam = gae_lambda[i] if isinstance(gae_lambda, torch.Tensor) else gae_lambda
        no_eos = seq_no_eos_mask[i : i + 1] if seq_no_eos_mask is not None else torch.zeros(1, dtype=torch.bool)
        a, _ = gae_padded(
            rewards[s:e][None].float(), values[s:e][None].float(), loss_mask[s:e][None].float(),
            no_eos, discount, lam,
        )
        adv[s:e] = a[0]
    return adv, adv + values
