"""Generalised advantage estimation on MI355X.

``_compute_token_level_gae`` keeps the reference's padded signature
(``areal/trainer/ppo/gae.py:10-36``); ``compute_gae_packed`` is the same recurrence on the
packed layout (``cu_seqlens``), which the reference does not have.  Both run the segmented
reverse scan of ``csrc/gae_norm.hip``.
"""

from __future__ import annotations

import torch

from areal_amd import _lib


def _launch(rewards, values, mask, cu, no_eos, lam_seq, n_seqs, uniform_len, discount, lam):
    lib = _lib.load()
    dev = _lib.require_gpu(rewards, values, mask, cu, no_eos, lam_seq)
    n = rewards.numel()
    adv = torch.empty(rewards.shape, dtype=torch.float32, device=dev)
    ret = torch.empty(rewards.shape, dtype=torch.float32, device=dev)
    if n == 0:
        return adv, ret
    nbytes = lib.areal_gae_workspace_bytes(n)
    ws = _lib.workspace(nbytes, dev)
    rc = lib.areal_gae_packed(
        _lib.ptr(rewards), _lib.ptr(values), _lib.ptr(mask), _lib.ptr(cu), _lib.ptr(no_eos),
        _lib.ptr(lam_seq), n, n_seqs, uniform_len, float(discount), float(lam),
        _lib.ptr(adv), _lib.ptr(ret), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_gae_packed")
    return adv, ret


def _split_lambda(gae_lambda, n_seqs, device):
    if isinstance(gae_lambda, torch.Tensor):
        lam_seq = gae_lambda.to(device=device, dtype=torch.float32).reshape(-1).contiguous()
        if lam_seq.numel() == 1:
            lam_seq = lam_seq.expand(n_seqs).contiguous()
        if lam_seq.numel() != n_seqs:
            raise ValueError(
                f"gae_lambda must be a float or hold one value per sequence ({n_seqs}), "
                f"got {tuple(gae_lambda.shape)}"
            )
        return lam_seq, 0.0
    return None, float(gae_lambda)


def _compute_token_level_gae(
    rewards: torch.Tensor,
    values: torch.Tensor,
    loss_mask: torch.Tensor,
    seq_no_eos_mask: torch.Tensor,
    discount: float,
    gae_lambda: float | torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    """GAE with each generated token as one timestep, on padded ``[bs, max_seqlen]`` tensors.
    Returns ``(advantages, returns)``; ``returns = advantages + values``."""
    bs, max_seqlen = rewards.shape
    dev = rewards.device
    lam_seq, lam = _split_lambda(gae_lambda, bs, dev)
    return _launch(
        rewards.to(torch.float32).contiguous(),
        values.to(torch.float32).contiguous(),
        loss_mask.to(torch.float32).contiguous(),
        None,
        seq_no_eos_mask.to(torch.bool).contiguous(),
        lam_seq, bs, max_seqlen, discount, lam,
    )


def _token_level_gae_with_row_stats(rewards, values, loss_mask, seq_no_eos_mask, discount, gae_lambda):
    """``_compute_token_level_gae`` that also returns, per row, the masked sums of the advantages
    which ``Normalization.from_row_stats`` needs (``[5, bs]`` fp64), or ``None`` when the layout
    does not allow it (rows shorter than one 2048-token tile)."""
    bs, max_seqlen = rewards.shape
    if max_seqlen < 2048 or bs == 0:
        return None
    lib = _lib.load()
    dev = _lib.require_gpu(rewards, values, loss_mask)
    lam_seq, lam = _split_lambda(gae_lambda, bs, dev)
    r = rewards.to(torch.float32).contiguous()
    v = values.to(torch.float32).contiguous()
    m = loss_mask.to(torch.float32).contiguous()
    no_eos = seq_no_eos_mask.to(torch.bool).contiguous()
    adv, ret = torch.empty_like(r), torch.empty_like(r)
    row_stats = torch.empty((5, bs), dtype=torch.float64, device=dev)
    rc = lib.areal_gae_padded_row_stats(
        _lib.ptr(r), _lib.ptr(v), _lib.ptr(m), _lib.ptr(no_eos), _lib.ptr(lam_seq), bs, max_seqlen,
        float(discount), float(lam), _lib.ptr(adv), _lib.ptr(ret), _lib.ptr(row_stats), _lib.stream_ptr(dev),
    )
    if rc == _lib.ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "areal_gae_padded_row_stats")
    return adv, ret, row_stats, m


def compute_gae_packed(
    rewards: torch.Tensor,
    values: torch.Tensor,
    loss_mask: torch.Tensor,
    cu_seqlens: torch.Tensor,
    seq_no_eos_mask: torch.Tensor | None,
    discount: float,
    gae_lambda: float | torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The same recurrence over 1-D packed tensors: sequence ``i`` is
    ``[cu_seqlens[i], cu_seqlens[i+1])``; its last position gets advantage 0 and, when
    ``seq_no_eos_mask[i]``, bootstraps the next value from ``values`` there."""
    if rewards.ndim != 1:
        raise ValueError(f"packed GAE expects 1D tensors, got ndim={rewards.ndim}")
    dev = rewards.device
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    n_seqs = cu.numel() - 1
    lam_seq, lam = _split_lambda(gae_lambda, n_seqs, dev)
    no_eos = seq_no_eos_mask.to(device=dev, dtype=torch.bool).contiguous() if seq_no_eos_mask is not None else None
    return _launch(
        rewards.to(torch.float32).contiguous(),
        values.to(torch.float32).contiguous(),
        loss_mask.to(torch.float32).contiguous(),
        cu, no_eos, lam_seq, n_seqs, 0, discount, lam,
    )


def compute_gae_packed_normalized(
    rewards: torch.Tensor,
    values: torch.Tensor,
    loss_mask: torch.Tensor,
    cu_seqlens: torch.Tensor,
    seq_no_eos_mask: torch.Tensor | None,
    discount: float,
    gae_lambda: float | torch.Tensor,
    adv_norm,
    group_sizes: list[int] | None = None,
    max_group_tokens: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``compute_gae_packed`` followed by ``adv_norm`` (a ``Normalization``) of the advantages
    under ``loss_mask``, with groups of whole sequences: what ``compute_advantages`` does after
    GAE (``areal/trainer/ppo/actor.py:344-350``), on the packed layout.  Returns ``(normalised
    advantages, returns, raw advantages)``.  Two launches when the normalisation needs one
    statistics pass (the GAE kernel leaves the sums), else GAE and the three normalisation passes."""
    if rewards.ndim != 1:
        raise ValueError(f"packed GAE expects 1D tensors, got ndim={rewards.ndim}")
    lib = _lib.load()
    dev = _lib.require_gpu(rewards, values, loss_mask, cu_seqlens)
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    n, n_seqs = rewards.numel(), cu.numel() - 1
    r = rewards.to(torch.float32).contiguous()
    v = values.to(torch.float32).contiguous()
    m = loss_mask.to(torch.float32).contiguous()
    if n > 0 and n_seqs > 0 and adv_norm.needs_one_statistics_pass():
        lam_seq, lam = _split_lambda(gae_lambda, n_seqs, dev)
        no_eos = seq_no_eos_mask.to(device=dev, dtype=torch.bool).contiguous() if seq_no_eos_mask is not None else None
        index, rows, _ = adv_norm._packed_groups(n_seqs, group_sizes, dev)
        offsets = cu.to(torch.int64)[index]
        nbytes = lib.areal_gae_segment_stats_bytes(n, rows.numel())
        seg = torch.empty(nbytes // 8, dtype=torch.float64, device=dev)
        adv, ret = torch.empty_like(r), torch.empty_like(r)
        rc = lib.areal_gae_packed_group_stats(
            _lib.ptr(r), _lib.ptr(v), _lib.ptr(m), _lib.ptr(cu), _lib.ptr(no_eos), _lib.ptr(lam_seq), n, n_seqs,
            float(discount), float(lam), _lib.ptr(offsets), rows.numel(), _lib.ptr(adv), _lib.ptr(ret),
            _lib.ptr(seg), nbytes, _lib.stream_ptr(dev),
        )
        if rc != _lib.ERR_UNSUPPORTED:
            _lib.check(rc, "areal_gae_packed_group_stats")
            normed = adv_norm.packed(adv, m, cu, group_sizes, max_group_tokens, segment_stats=seg)
            return normed, ret, adv
    adv, ret = compute_gae_packed(r, v, m, cu, seq_no_eos_mask, discount, gae_lambda)
    return adv_norm.packed(adv, m, cu, group_sizes, max_group_tokens), ret, adv


_TURN_ID_ERRORS = (
    (1, "turn_ids must be non-negative at every active loss token"),
    (2, "turn_ids at active loss tokens must be smaller than the sequence length"),
    (4, "turn_ids at active loss tokens must be temporally nondecreasing"),
)


def _compute_turn_level_gae(
    rewards: torch.Tensor,
    values: torch.Tensor,
    loss_mask: torch.Tensor,
    turn_ids: torch.Tensor,
    seq_no_eos_mask: torch.Tensor,
    discount: float,
    gae_lambda: float | torch.Tensor,
    validate: bool = True,
) -> tuple[torch.Tensor, torch.Tensor]:
    """GAE with each generated turn treated as one timestep, on padded ``[bs, max_seqlen]``
    tensors (``areal/trainer/ppo/gae.py:82-163``).

    Shape, device and dtype errors are raised as in the reference.  Malformed turn ids at
    active tokens (negative, too large, going backwards) are found by the kernel; with
    ``validate=True`` the flag is read back (one host synchronisation) and raised as the
    reference's ``RuntimeError``; the reference uses device-side asserts there, which on a GPU
    would abort the process.  ``validate=False`` skips the read-back.
    """
    if turn_ids.shape != loss_mask.shape:
        raise ValueError(f"turn_ids must have shape {loss_mask.shape}, got {turn_ids.shape}")
    if turn_ids.device != loss_mask.device:
        raise ValueError(
            "turn_ids and loss_mask must be on the same device, got "
            f"{turn_ids.device} and {loss_mask.device}"
        )
    if turn_ids.dtype not in (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64):
        raise ValueError(f"turn_ids must use an integer dtype, got {turn_ids.dtype}")
    lib = _lib.load()
    bs, max_seqlen = rewards.shape
    r = rewards.to(torch.float32).contiguous()
    v = values.to(torch.float32).contiguous()
    m = loss_mask.to(torch.float32).contiguous()
    # ids beyond int32 cannot be valid (they must be smaller than the sequence length)
    ids = turn_ids.clamp(min=-1, max=2**31 - 1).to(torch.int32).contiguous()
    dev = _lib.require_gpu(r, v, m, ids)
    lam_seq, lam = _split_lambda(gae_lambda, bs, dev)
    no_eos = seq_no_eos_mask.to(device=dev, dtype=torch.bool).contiguous()
    adv = torch.empty((bs, max_seqlen), dtype=torch.float32, device=dev)
    ret = torch.empty((bs, max_seqlen), dtype=torch.float32, device=dev)
    if bs == 0 or max_seqlen == 0:
        return adv, ret
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    nbytes = lib.areal_turn_gae_workspace_bytes(bs, max_seqlen)
    ws = _lib.workspace(nbytes, dev)
    rc = lib.areal_turn_gae(
        _lib.ptr(r), _lib.ptr(v), _lib.ptr(m), _lib.ptr(ids), _lib.ptr(no_eos), _lib.ptr(lam_seq),
        bs, max_seqlen, float(discount), float(lam), _lib.ptr(adv), _lib.ptr(ret),
        _lib.ptr(status), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_turn_gae")
    if validate:
        _raise_turn_id_errors(status)
    return adv, ret


def _raise_turn_id_errors(status: torch.Tensor) -> None:
    flags = int(status.item())
    for bit, message in _TURN_ID_ERRORS:
        if flags & bit:
            raise RuntimeError(message)


def _build_gae_lambda_context(
    loss_mask: torch.Tensor,
    turn_ids: torch.Tensor | None,
    *,
    gae_timestep_unit: str,
    validate: bool = True,
) -> dict[str, torch.Tensor]:
    """Per-sample lengths from the GAE eligibility mask (``areal/trainer/ppo/gae.py:166-205``):
    ``effective_token_lengths`` (active tokens), ``turn_counts`` (distinct active turn ids, zero
    without ``turn_ids``) and ``timestep_lengths`` (the one ``gae_timestep_unit`` selects)."""
    if turn_ids is None and gae_timestep_unit == "turn":
        raise ValueError("Turn-level GAE requires rollout data to include 'turn_ids'.")
    if turn_ids is not None:
        if turn_ids.shape != loss_mask.shape:
            raise ValueError(f"turn_ids must have shape {loss_mask.shape}, got {turn_ids.shape}")
        if turn_ids.device != loss_mask.device:
            raise ValueError(
                "turn_ids and loss_mask must be on the same device, got "
                f"{turn_ids.device} and {loss_mask.device}"
            )
        if turn_ids.dtype not in (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64):
            raise ValueError(f"turn_ids must use an integer dtype, got {turn_ids.dtype}")
    lib = _lib.load()
    bs, max_seqlen = loss_mask.shape
    m = loss_mask.to(torch.float32).contiguous()
    ids = turn_ids.clamp(min=-1, max=2**31 - 1).to(torch.int32).contiguous() if turn_ids is not None else None
    dev = _lib.require_gpu(m, ids)
    token_lengths = torch.zeros(bs, dtype=torch.int64, device=dev)
    turn_counts = torch.zeros(bs, dtype=torch.int64, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    rc = lib.areal_gae_lambda_context(
        _lib.ptr(m), _lib.ptr(ids), bs, max_seqlen, _lib.ptr(token_lengths), _lib.ptr(turn_counts),
        _lib.ptr(status), _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_gae_lambda_context")
    if validate and turn_ids is not None:
        _raise_turn_id_errors(status)
    return {
        "effective_token_lengths": token_lengths,
        "turn_counts": turn_counts,
        "timestep_lengths": token_lengths if gae_timestep_unit == "token" else turn_counts,
    }


def compute_gae_lambda(gae_lambda_fn, gae_lambda_kwargs, loss_mask, turn_ids, gae_timestep_unit):
    """One lambda per local trajectory from a custom function, with the reference's checks of
    its output (``areal/trainer/ppo/actor.py:325-362``)."""
    context = _build_gae_lambda_context(loss_mask, turn_ids, gae_timestep_unit=gae_timestep_unit)
    gae_lambda = gae_lambda_fn(context, **(gae_lambda_kwargs or {}))
    if not isinstance(gae_lambda, torch.Tensor):
        raise TypeError(
            "gae_lambda function must return a torch.Tensor with shape "
            f"[{loss_mask.shape[0]}], got {type(gae_lambda).__name__}"
        )
    expected_shape = torch.Size([loss_mask.shape[0]])
    if gae_lambda.shape != expected_shape:
        raise ValueError(
            "gae_lambda function must return one value per local trajectory: "
            f"expected shape {expected_shape}, got {gae_lambda.shape}"
        )
    if gae_lambda.device != loss_mask.device:
        raise ValueError(
            "gae_lambda output and loss_mask must be on the same device, got "
            f"{gae_lambda.device} and {loss_mask.device}"
        )
    if not torch.is_floating_point(gae_lambda):
        raise TypeError(f"gae_lambda function must return a floating-point tensor, got {gae_lambda.dtype}")
    if not bool(torch.all(torch.isfinite(gae_lambda))):
        raise RuntimeError("gae_lambda function returned a non-finite value")
    return gae_lambda.detach().float()
