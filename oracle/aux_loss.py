"""Oracle: SAPO policy loss, PPO critic loss, DPO sequence log-ratios (CPU, test-only).

Restates with plain differentiable torch ops (autograd gives the reference's gradient):
  * ``areal/utils/functional/functional.py:599-675`` sapo_loss_fn (sequence-level branch through
    ``oracle.loss.sequence_ratio_and_advantages``, functional.py:56-149);
  * ``functional.py:859-933`` _huber_loss, _mse_loss, ppo_critic_loss_fn;
  * ``functional.py:796-856`` dpo_pair_logratios, dpo_preference_loss.

Pinned by (tests/test_oracle_aux_loss.py):
  * SAPO: the reference tests' literals (tests/test_functional.py:923-954 loss -2.0 and gate 2.0
    at ratio 1; :956-1036 gate selection by advantage sign; :1160-1195 equal gradients for
    tau = 1 and tau = 2 at ratio 1; :1197-1224 the masked mean formula), plus the closed-form
    gradient -4 g (1 - g) A r / N against autograd.
  * critic loss: the reference has no test for it ("parity unpinned" against the reference):
    pinned by hand-computed cases on both sides of the clip band, the huber branch beyond
    delta = 10, the mask denominator, and torch autograd of the textbook formula.
  * DPO: no reference test either ("parity unpinned"): pinned by brute-force per-sequence
    Python sums with the shifted mask, the pairing layout, and log-sigmoid / IPO closed forms.
"""

from __future__ import annotations

import functools

import torch

from oracle.loss import sequence_ratio_and_advantages


def sapo_loss(logprobs, old_logprobs, advantages, tau_pos, tau_neg, loss_mask,
              importance_sampling_level="token", cu_seqlens=None):
    """sapo_loss_fn (functional.py:599-675)."""
    if tau_pos <= 0 or tau_neg <= 0:
        raise ValueError("SAPO temperatures (tau_pos, tau_neg) must be positive.")
    n0 = loss_mask.count_nonzero() or 1
    advantages = advantages.detach()
    log_ratio = logprobs - old_logprobs
    if importance_sampling_level == "sequence":
        ratio, advantages = sequence_ratio_and_advantages(log_ratio, advantages, loss_mask, cu_seqlens)
    elif importance_sampling_level == "token":
        ratio = torch.exp(log_ratio)
    else:
        raise ValueError(f"Invalid importance_sampling_level: {importance_sampling_level}.")
    gate_pos = torch.sigmoid(tau_pos * (ratio - 1.0)) * (4.0 / tau_pos)
    gate_neg = torch.sigmoid(tau_neg * (ratio - 1.0)) * (4.0 / tau_neg)
    soft_gate = torch.where(advantages > 0, gate_pos, gate_neg)
    pg = -soft_gate * advantages
    loss = torch.where(loss_mask, pg, 0).sum() / n0
    stat = dict(
        loss=pg.detach(), importance_weight=ratio.detach(), approx_kl=log_ratio.detach(),
        clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        dual_clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        sapo_soft_gate=soft_gate.detach(), sapo_scaled_gate_pos=gate_pos.detach(),
        sapo_scaled_gate_neg=gate_neg.detach(),
    )
    return loss, stat


def _huber(x, y, delta):
    diff = torch.abs(x - y)
    return torch.where(diff < delta, 0.5 * diff**2, delta * (diff - 0.5 * delta))


def _mse(x, y):
    return 0.5 * (x - y) ** 2


def critic_loss(value, old_value, target_value, value_eps_clip, loss_mask=None, loss_fn_type="mse"):
    """ppo_critic_loss_fn (functional.py:869-933)."""
    if loss_fn_type == "huber":
        fn = functools.partial(_huber, delta=10.0)
    elif loss_fn_type == "mse":
        fn = _mse
    else:
        raise NotImplementedError(f"Unknown loss fn type: {loss_fn_type}")
    original = fn(value, target_value)
    clipped_value = old_value + (value - old_value).clamp(-value_eps_clip, value_eps_clip)
    clipped = fn(clipped_value, target_value)
    value_loss = torch.max(original, clipped)
    clip_mask = clipped.detach() > original.detach()
    if loss_mask is not None:
        clip_mask = clip_mask.logical_and(loss_mask)
    stat = dict(clip_mask=clip_mask, loss=value_loss.detach())
    if loss_mask is not None:
        value_loss = torch.where(loss_mask, value_loss, 0).sum() / loss_mask.count_nonzero()
    else:
        value_loss = value_loss.mean()
    return value_loss, stat


def dpo_pair_logratios(logprobs, ref_logprobs, cu_seqlens, loss_mask, valid_pairs):
    """dpo_pair_logratios (functional.py:796-841): (policy, reference, lengths), each [K, 2]."""
    shifted = torch.zeros_like(loss_mask)
    if loss_mask.shape[0] > 1:
        shifted[:-1] = loss_mask[1:]
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    shifted.index_fill_(0, (cu_seqlens[1:] - 1)[seqlens > 0].long(), False)
    n_seqs = seqlens.shape[0]
    seq_ids = torch.repeat_interleave(torch.arange(n_seqs), seqlens.long())
    masked = shifted.to(dtype=logprobs.dtype)
    policy = torch.zeros(n_seqs, dtype=torch.float64).index_add(0, seq_ids, (logprobs * masked).double())
    ref = torch.zeros(n_seqs, dtype=torch.float64).index_add(0, seq_ids, (ref_logprobs * masked).double())
    lens = torch.zeros(n_seqs, dtype=torch.float64).index_add(0, seq_ids, shifted.double())
    return policy.view(-1, 2)[valid_pairs], ref.view(-1, 2)[valid_pairs], lens.view(-1, 2)[valid_pairs]


def dpo_preference_loss(logits, *, beta, loss_type="sigmoid"):
    """dpo_preference_loss (functional.py:844-856)."""
    if loss_type == "sigmoid":
        return -torch.nn.functional.logsigmoid(beta * logits.float())
    if loss_type == "ipo":
        return (logits.float() - 1.0 / (2.0 * beta)) ** 2
    raise ValueError(f"Unsupported DPO loss_type: {loss_type!r}")


def m2po_mask(old_logp, prox_logp, loss_mask, m2_threshold):
    """_apply_m2po_masking + _get_m2po_loss_mask (areal/trainer/ppo/actor.py:933-1014): sort the
    masked tokens by m2 = (old - prox)^2 descending and drop the largest until the mean of the
    rest is below the threshold (at least one token stays).

    The reference has no test for it ("parity unpinned" against the reference). Pinned by
    hand-computed cases (tests/test_oracle_aux_loss.py) and by the defining property checked
    with brute force: the kept set is the largest set of smallest-m2 tokens whose mean is below
    the threshold, or the single smallest token when no such set exists."""
    delta = old_logp - prox_logp
    m2 = delta * delta
    flat = loss_mask.reshape(-1).bool()
    sel = m2.reshape(-1)[flat]
    if sel.numel() == 0:
        return loss_mask
    sorted_m2, indices = torch.sort(sel, descending=True)
    restored = torch.argsort(indices)
    n = sorted_m2.numel()
    suffix = sorted_m2.flip(0).cumsum(0).flip(0)
    counts = torch.arange(n, 0, -1, dtype=sorted_m2.dtype)
    below = torch.where(suffix / counts < m2_threshold)[0]
    num_to_mask = int(below[0]) if len(below) > 0 else n - 1
    keep_sorted = torch.ones(n, dtype=torch.bool)
    keep_sorted[:num_to_mask] = False
    full = torch.zeros_like(flat)
    full[flat] = keep_sorted[restored]
    return full.view_as(loss_mask)


def prox_logp_approximations(old_logp, logprobs, versions, current_version, method=None):
    """compute_prox_logp_approximations (areal/trainer/ppo/actor.py:768-848).

    Pinned by the reference's literals (tests/test_prox_approx.py:24-211): log-linear
    [-1.25, -2.25, -3.25] at alpha 0.5, mixed versions [-1.375, -2.1], alpha 0 when the behaviour
    version is the proximal one or equals the current one, prompt tokens (version < 0) unchanged,
    linear log(0.375), rollout = old."""
    v_prox = current_version - 1
    v_behave = versions.float()
    v_theta = float(current_version)
    generated = versions >= 0
    diff = v_theta - v_behave
    gap = v_prox - v_behave
    alpha = torch.where((diff > 0) & generated, gap / diff, torch.zeros_like(v_behave)).clamp(0.0, 1.0)
    out = {}
    for m in ([method] if method else ["loglinear", "linear", "rollout"]):
        if m == "loglinear":
            out[m] = old_logp + alpha * (logprobs - old_logp)
        elif m == "linear":
            out[m] = torch.log((1 - alpha) * torch.exp(old_logp) + alpha * torch.exp(logprobs) + 1e-10)
        elif m == "rollout":
            out[m] = old_logp.clone()
    return out


def distill_loss(loss, logprobs, old_logp, teacher_logp, loss_mask, rl_loss_weight=1.0, distill_loss_weight=0.005):
    """The joint-distillation tail of grpo_loss_fn (actor.py:629-658): returns (loss, rkl_stat).

    No reference test covers it ("parity unpinned"): pinned by hand-computed two-token cases of
    both branches and by autograd of these same expressions."""
    teacher_logp = teacher_logp.detach()
    if rl_loss_weight == 0:
        reward = teacher_logp - logprobs.detach()
        iw = torch.exp(logprobs - old_logp)
        term = iw * reward * loss_mask
        return -1 * distill_loss_weight * term.sum() / loss_mask.sum().clamp(min=1), -1 * term
    per_token = (logprobs - teacher_logp) * loss_mask
    penalty = per_token.sum() / loss_mask.sum().clamp(min=1)
    return rl_loss_weight * loss + distill_loss_weight * penalty, per_token
