"""Per-sample GAE lambda functions and their resolution.

Host-side mirror of ``areal/trainer/ppo/lambda_fn.py`` (same names, arguments, errors): the
functions map per-trajectory lengths (``[bs]`` tensors) to one lambda per trajectory, which the
GAE kernels take as their per-sequence lambda.  The lengths themselves come from
``areal_amd.ppo.gae._build_gae_lambda_context`` (one kernel over the loss mask and turn ids).
"""

from __future__ import annotations

import functools
import importlib
import math
from collections.abc import Callable
from typing import TypedDict

import torch

__all__ = [
    "GAELambdaContext",
    "GAELambdaFn",
    "constant_gae_lambda",
    "relative_position_gae_lambda",
    "resolve_gae_lambda_fn",
    "vapo_length_adaptive_gae",
]


class GAELambdaContext(TypedDict):
    """Batch-local trajectory lengths available to a GAE lambda function."""

    effective_token_lengths: torch.Tensor
    turn_counts: torch.Tensor
    timestep_lengths: torch.Tensor


GAELambdaFn = Callable[..., torch.Tensor]


def constant_gae_lambda(context: GAELambdaContext, *, value: float) -> torch.Tensor:
    """One constant lambda for every local trajectory (``lambda_fn.py:37-47``)."""
    return torch.full_like(context["timestep_lengths"], fill_value=value, dtype=torch.float32)


def vapo_length_adaptive_gae(context: GAELambdaContext, *, alpha: float) -> torch.Tensor:
    """VAPO's ``lambda = 1 - 1 / (alpha * length)``, zero for empty trajectories
    (``lambda_fn.py:50-69``)."""
    if isinstance(alpha, bool) or not isinstance(alpha, int | float) or alpha <= 0:
        raise ValueError(f"alpha must be a positive number, got {alpha!r}")
    lengths = context["timestep_lengths"]
    safe = lengths.to(dtype=torch.float32).clamp_min(1.0)
    lam = (1.0 - 1.0 / (float(alpha) * safe)).clamp_min(0.0)
    return torch.where(lengths > 0, lam, torch.zeros_like(lam))


def relative_position_gae_lambda(context: GAELambdaContext, *, q: float) -> torch.Tensor:
    """``lambda = q ** (1 / (L - 1))``: a terminal reward keeps the fraction ``q`` at the first
    timestep whatever the length; one timestep -> 1, none -> 0 (``lambda_fn.py:72-112``)."""
    if isinstance(q, bool) or not isinstance(q, int | float) or not math.isfinite(q) or not 0 < q <= 1:
        raise ValueError(f"q must be a finite number in (0, 1], got {q!r}")
    lengths = context["timestep_lengths"]
    decay_steps = (lengths - 1).clamp_min(1).to(dtype=torch.float32)
    step = torch.exp(math.log(float(q)) / decay_steps)
    return torch.where(
        lengths > 1, step, torch.where(lengths == 1, torch.ones_like(step), torch.zeros_like(step))
    )


def _import_from_string(path: str):
    module_name, _, attr = path.rpartition(".")
    if not module_name:
        raise ImportError(f"'{path}' is not a dotted path to a function")
    return getattr(importlib.import_module(module_name), attr)


def resolve_gae_lambda_fn(gae_lambda: float | str) -> tuple[GAELambdaFn, bool]:
    """A static value or a dotted function path -> (callable, came from a custom path)
    (``lambda_fn.py:115-137``)."""
    if isinstance(gae_lambda, bool):
        raise TypeError("gae_lambda must be a float or dotted function path, not bool")
    if isinstance(gae_lambda, int | float):
        return functools.partial(constant_gae_lambda, value=float(gae_lambda)), False
    if not isinstance(gae_lambda, str) or not gae_lambda:
        raise TypeError(
            "gae_lambda must be a float or a non-empty dotted function path, "
            f"got {gae_lambda!r}"
        )
    fn = _import_from_string(gae_lambda)
    if not callable(fn):
        raise TypeError(f"Imported gae_lambda object is not callable: {gae_lambda}")
    return fn, True
