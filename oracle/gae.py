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


def gae_turn_level(rewards, values, loss_mask, turn_ids, seq_no_eos_mask, discount, gae_lambda):
    """Turn-level GAE (``areal/trainer/ppo/gae.py:82-163``): every generated turn is one
    timestep; its reward is the sum of its active tokens' rewards, its value the value at its
    first active token; the turn's advantage is broadcast to its tokens.

    Pinned by the reference's literals (tests/test_ppo_gae.py:81-151): [[2,2,2,2]] for lambda
    0.5 over two turns; gaps / unused ids with bootstrap giving advantages
    [[3.75,3.75,0,6,6]] and returns [[4.75,4.75,9,8,8]]; per-sample lambda [[2,2,2,2],[1,1,2,2]].
    Validation raises as the reference does on the CPU (RuntimeError from the asserts)."""
    if turn_ids.shape != loss_mask.shape:
        raise ValueError(f"turn_ids must have shape {loss_mask.shape}, got {turn_ids.shape}")
    if turn_ids.dtype not in (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64):
        raise ValueError(f"turn_ids must use an integer dtype, got {turn_ids.dtype}")
    bs, width = rewards.shape
    valid = loss_mask.bool()
    if not torch.all(~valid | (turn_ids >= 0)):
        raise RuntimeError("turn_ids must be non-negative at every active loss token")
    if not torch.all(~valid | (turn_ids < width)):
        raise RuntimeError("turn_ids at active loss tokens must be smaller than the sequence length")
    active = torch.where(valid, turn_ids, torch.full_like(turn_ids, -1))
    if not torch.all(~valid | (turn_ids >= torch.cummax(active, dim=1).values)):
        raise RuntimeError("turn_ids at active loss tokens must be temporally nondecreasing")
    safe = torch.clamp(turn_ids.long(), min=0, max=width - 1)
    turn_rewards = torch.zeros_like(rewards).scatter_add_(1, safe, rewards * valid.to(rewards.dtype))
    pos = torch.arange(width).expand(bs, -1)
    first = torch.full_like(safe, width).scatter_reduce_(
        1, safe, torch.where(valid, pos, torch.full_like(pos, width)), reduce="amin", include_self=True
    )
    valid_turn = first < width
    turn_values = values.gather(1, first.clamp(max=width - 1)) * valid_turn.to(values.dtype)
    turn_adv = torch.zeros(bs, width, dtype=torch.float32)
    last = torch.zeros(bs, dtype=torch.float32)
    nxt = values[:, width - 1] * seq_no_eos_mask
    c = discount * gae_lambda
    for k in reversed(range(width)):
        delta = turn_rewards[:, k] + discount * nxt - turn_values[:, k]
        new = delta + c * last
        m = valid_turn[:, k]
        turn_adv[:, k] = torch.where(m, new, torch.zeros_like(last))
        nxt = torch.where(m, turn_values[:, k], nxt)
        last = torch.where(m, new, last)
    turn_ret = turn_adv + turn_values
    adv = torch.gather(turn_adv, 1, safe) * loss_mask
    ret = torch.gather(turn_ret, 1, safe) * loss_mask + values * (1 - loss_mask)
    return adv, ret
