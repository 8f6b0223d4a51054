"""SAPO policy loss, PPO critic loss and DPO sequence log-ratios on MI355X.

Same Python signatures, return structures and error behaviour as the reference's
``areal/utils/functional/functional.py``: ``sapo_loss_fn`` (:599-675), ``ppo_critic_loss_fn``
(:869-933), ``dpo_pair_logratios`` (:796-841) and ``dpo_preference_loss`` (:844-856).  The
per-token work runs in the HIP kernels of ``csrc/aux_loss.hip``; the gradient is the kernels'
closed form, not autograd through torch ops.
"""

from __future__ import annotations

import torch

from areal_amd import _lib
from areal_amd.functional.functional import _f32, _sequence_layout


class _ScaledLoss(torch.autograd.Function):
    """Scalar loss whose gradient w.r.t. its first input is ``dsum * upstream / count`` (the
    kernels write ``dsum = d(loss sum)/d input`` and the count into ``counters[1]``)."""

    @staticmethod
    def forward(ctx, x, launch):
        out = launch(x.requires_grad)
        if x.requires_grad:
            ctx.save_for_backward(out["dsum"], out["counters"])
        ctx.shape = x.shape
        ctx.in_dtype = x.dtype
        launch.out = out
        return out["loss"]

    @staticmethod
    def backward(ctx, grad_loss):
        dsum, counters = ctx.saved_tensors
        lib = _lib.load()
        dev = dsum.device
        g = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        grad = torch.empty_like(dsum)
        rc = lib.areal_actor_loss_grad(
            _lib.ptr(dsum), _lib.ptr(g), _lib.ptr(counters), _lib.ptr(grad), dsum.numel(),
            _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_actor_loss_grad")
        grad = grad.view(ctx.shape)
        if ctx.in_dtype != torch.float32:
            grad = grad.to(ctx.in_dtype)
        return grad, None


class _Launch:
    """Callable handed to ``_ScaledLoss``; keeps the kernel outputs for the caller."""

    def __init__(self, fn):
        self.fn = fn
        self.out = None

    def __call__(self, want_grad: bool):
        return self.fn(want_grad)


def sapo_loss_fn(
    logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    tau_pos: float,
    tau_neg: float,
    loss_mask: torch.Tensor,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
    stat_reduction=None,
) -> tuple[torch.Tensor, dict]:
    """SAPO loss with asymmetric sigmoid gates; ``stat`` keys as in ``functional.py:661-673``.
    ``stat_reduction`` (a ``StatReduction``; not in the reference): the token kernel reduces the
    logged statistics itself and no per-token statistic tensor is written; ``stat`` then holds
    the host scalars ``n_total_tokens`` and ``n_valid_tokens`` only."""
    if tau_pos <= 0 or tau_neg <= 0:
        raise ValueError("SAPO temperatures (tau_pos, tau_neg) must be positive.")
    if importance_sampling_level == "sequence":
        if logprobs.ndim == 1 and cu_seqlens is None:
            raise ValueError(
                "cu_seqlens is required for 1D tensors (packed format). "
                "In AReaL, 1D tensors are produced by pack_tensor_dict() and always have cu_seqlens. "
                "For a single sequence, use cu_seqlens=torch.tensor([0, seq_len], dtype=torch.int32)."
            )
    elif importance_sampling_level != "token":
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. "
            "Must be 'token' or 'sequence'."
        )
    lib = _lib.load()
    shape = logprobs.shape
    seq_level = importance_sampling_level == "sequence"
    old, adv = _f32(old_logprobs), _f32(advantages)
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    dev = _lib.require_gpu(logprobs, old, adv, mask_bool)
    n = int(mask_bool.numel())
    cu, n_seqs, uniform_len = (None, 0, 0)
    if seq_level:
        cu, n_seqs, uniform_len = _sequence_layout(shape, cu_seqlens, dev)

    names = ("stat_loss", "ratio", "approx_kl", "soft_gate", "gate_pos", "gate_neg")
    red = stat_reduction
    ent = extras = None
    if red is not None:
        from areal_amd.functional.functional import SAPO_REDUCED_STAT_KEYS

        extras = [_f32(t) for t in red.extras.values()]
        ent = _f32(red.entropy) if red.entropy is not None else None
        for t in extras + ([ent] if ent is not None else []):
            if t.numel() != n:
                raise ValueError(f"a statistic rides along with {t.numel()} elements, expected {n}")

    def launch(want_grad: bool):
        f32 = dict(dtype=torch.float32, device=dev)
        out = {k: (torch.empty(n, **f32) if red is None else None) for k in names}
        out["loss"] = torch.empty((), **f32)
        out["dsum"] = torch.empty(n, **f32) if want_grad else None
        # counters [8] and, with a reduction, stats [13][4] in one buffer: one copy to the host
        n_stats = len(SAPO_REDUCED_STAT_KEYS) if red is not None else 0
        both = torch.empty(8 + 4 * n_stats, dtype=torch.float64, device=dev)
        out["counters"], out["both"] = both[:8], both
        nbytes = lib.areal_aux_loss_workspace_bytes(n, n_seqs)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_sapo_loss(
            _lib.ptr(_f32(logprobs)), _lib.ptr(old), _lib.ptr(adv), _lib.ptr(mask_bool),
            _lib.ptr(cu), n, n_seqs, uniform_len, float(tau_pos), float(tau_neg), int(seq_level),
            _lib.ptr(out["loss"]), _lib.ptr(out["dsum"]), _lib.ptr(out["stat_loss"]),
            _lib.ptr(out["ratio"]), _lib.ptr(out["approx_kl"]), _lib.ptr(out["soft_gate"]),
            _lib.ptr(out["gate_pos"]), _lib.ptr(out["gate_neg"]), _lib.ptr(out["counters"]),
            _lib.ptr(ent), _lib.ptr(extras[0] if extras else None),
            _lib.ptr(extras[1] if extras and len(extras) > 1 else None),
            _lib.ptr(both[8:]) if red is not None else None,
            _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_sapo_loss")
        return out

    runner = _Launch(launch)
    loss = _ScaledLoss.apply(logprobs, runner)
    out = runner.out
    if red is not None:
        host = out["both"].cpu()  # the one host synchronisation of the call
        red._fill_sapo(host[8:].view(-1, 4), host[:8], n)
        return loss, dict(n_total_tokens=float(n), n_valid_tokens=float(host[1]),
                          n_masked_tokens=float(n) - float(host[1]),
                          masked_token_ratio=1.0 - float(host[1]) / max(float(n), 1.0))
    stat = dict(
        loss=out["stat_loss"].view(shape),
        importance_weight=out["ratio"].view(shape),
        approx_kl=out["approx_kl"].view(shape),
        clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        dual_clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        sapo_soft_gate=out["soft_gate"].view(shape),
        sapo_scaled_gate_pos=out["gate_pos"].view(shape),
        sapo_scaled_gate_neg=out["gate_neg"].view(shape),
    )
    return loss, stat


def ppo_critic_loss_fn(
    value: torch.Tensor,
    old_value: torch.Tensor,
    target_value: torch.Tensor,
    value_eps_clip: float,
    loss_mask: torch.Tensor | None = None,
    loss_fn_type: str = "mse",
) -> tuple[torch.Tensor, dict]:
    """Clipped PPO critic loss; inputs of one common shape, fp32 (``functional.py:869-933``)."""
    assert value.dtype == torch.float32
    assert old_value.dtype == torch.float32
    assert target_value.dtype == torch.float32
    if loss_fn_type not in ("huber", "mse"):
        raise NotImplementedError(f"Unknown loss fn type: {loss_fn_type}")
    lib = _lib.load()
    shape = value.shape
    old, target = _f32(old_value), _f32(target_value)
    mask_bool = loss_mask.detach().bool().contiguous().view(-1) if loss_mask is not None else None
    dev = _lib.require_gpu(value, old, target, mask_bool)
    n = int(value.numel())

    def launch(want_grad: bool):
        out = {
            "loss": torch.empty((), dtype=torch.float32, device=dev),
            "dsum": torch.empty(n, dtype=torch.float32, device=dev) if want_grad else None,
            "stat_loss": torch.empty(n, dtype=torch.float32, device=dev),
            "clip_mask": torch.empty(n, dtype=torch.bool, device=dev),
            "counters": torch.empty(8, dtype=torch.float64, device=dev),
        }
        nbytes = lib.areal_aux_loss_workspace_bytes(n, 0)
        ws = _lib.workspace(nbytes, dev)
        rc = lib.areal_critic_loss(
            _lib.ptr(_f32(value)), _lib.ptr(old), _lib.ptr(target), _lib.ptr(mask_bool), n,
            float(value_eps_clip), int(loss_fn_type == "huber"), _lib.ptr(out["loss"]),
            _lib.ptr(out["dsum"]), _lib.ptr(out["stat_loss"]), _lib.ptr(out["clip_mask"]),
            _lib.ptr(out["counters"]), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_critic_loss")
        return out

    runner = _Launch(launch)
    loss = _ScaledLoss.apply(value, runner)
    out = runner.out
    stat = dict(clip_mask=out["clip_mask"].view(shape), loss=out["stat_loss"].view(shape))
    return loss, stat


class _SeqLogps(torch.autograd.Function):
    """Per-sequence fp64 sums of the shifted-mask log-probs; gradient to ``logprobs`` only."""

    @staticmethod
    def forward(ctx, logprobs, ref_logprobs, cu, mask_bool):
        lib = _lib.load()
        dev = logprobs.device
        n, n_seqs = int(logprobs.numel()), int(cu.numel() - 1)
        sums = torch.zeros((n_seqs, 3), dtype=torch.float64, device=dev)
        shifted = torch.zeros(n, dtype=torch.bool, device=dev)
        rc = lib.areal_dpo_seq_logps(
            _lib.ptr(_f32(logprobs)), _lib.ptr(_f32(ref_logprobs)), _lib.ptr(mask_bool),
            _lib.ptr(cu), n, n_seqs, _lib.ptr(sums), _lib.ptr(shifted), _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_dpo_seq_logps")
        ctx.save_for_backward(shifted, cu)
        ctx.shape = logprobs.shape
        ctx.in_dtype = logprobs.dtype
        policy, ref, lens = sums[:, 0], sums[:, 1], sums[:, 2]
        ctx.mark_non_differentiable(ref, lens)
        return policy, ref, lens

    @staticmethod
    def backward(ctx, g_policy, *unused):
        shifted, cu = ctx.saved_tensors
        lib = _lib.load()
        dev = shifted.device
        n, n_seqs = int(shifted.numel()), int(cu.numel() - 1)
        grad = torch.empty(n, dtype=torch.float32, device=dev)
        g = g_policy.detach().to(torch.float64).contiguous()
        rc = lib.areal_dpo_seq_logps_grad(
            _lib.ptr(g), _lib.ptr(shifted), _lib.ptr(cu), n, n_seqs, _lib.ptr(grad),
            _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_dpo_seq_logps_grad")
        return grad.view(ctx.shape).to(ctx.in_dtype), None, None, None


def dpo_pair_logratios(
    logprobs: torch.Tensor,
    ref_logprobs: torch.Tensor,
    cu_seqlens: torch.Tensor,
    loss_mask: torch.Tensor,
    valid_pairs: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-sequence masked log-prob sums of a packed ``[chosen_0, rejected_0, ...]`` batch,
    paired up: ``(policy_logps, ref_logps, completion_lens)``, each ``(K, 2)`` fp64."""
    dev = _lib.require_gpu(logprobs, ref_logprobs, cu_seqlens, loss_mask)
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    mask_bool = loss_mask.detach().bool().contiguous().view(-1)
    policy, ref, lens = _SeqLogps.apply(logprobs, ref_logprobs, cu, mask_bool)
    return (
        policy.view(-1, 2)[valid_pairs],
        ref.view(-1, 2)[valid_pairs],
        lens.view(-1, 2)[valid_pairs],
    )


def dpo_preference_loss(
    logits: torch.Tensor, *, beta: float, loss_type: str = "sigmoid"
) -> torch.Tensor:
    """Per-pair preference loss from DPO log-ratio logits (K values: plain tensor ops)."""
    if loss_type == "sigmoid":
        return -torch.nn.functional.logsigmoid(beta * logits.float())
    if loss_type == "ipo":
        return (logits.float() - 1.0 / (2.0 * beta)) ** 2
    raise ValueError(f"Unsupported DPO loss_type: {loss_type!r}")
