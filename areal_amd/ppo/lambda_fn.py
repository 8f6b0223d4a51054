"""Per-trajectory GAE lambda schedules and the resolver of the ``gae_lambda`` option.

Counterpart of the reference's ``areal/trainer/ppo/lambda_fn.py:26-141``.  A schedule is any
callable ``fn(context, **kwargs)`` that maps the batch's length context (three ``[bs]`` integer
tensors, see :class:`GAELambdaContext`; built by ``areal_amd.ppo.gae._build_gae_lambda_context``)
to one fp32 lambda per trajectory.  ``compute_advantages`` hands the result to the GAE kernel as
its per-sequence lambda array, so these functions are plain tensor arithmetic on ``[bs]`` values
and run on whatever device the context lives on.

Three schedules are shipped, with ``L = context["timestep_lengths"]`` (generated tokens in token
mode, active turns in turn mode):

===============================  =======================================================
``constant_gae_lambda``          ``value`` for every trajectory
``vapo_length_adaptive_gae``     ``max(0, 1 - 1 / (alpha * L))``; 0 when ``L == 0``
``relative_position_gae_lambda`` ``q ** (1 / (L - 1))`` for ``L >= 2``; 1 for ``L == 1``;
                                 0 for ``L == 0``
===============================  =======================================================

With discount 1 the last schedule makes a terminal reward arrive at one-based step ``k`` scaled by
``q ** ((L - k) / (L - 1))``: ``q`` at the first step, 1 at the last, and the same factor at equal
relative positions of trajectories of different length.
"""

from __future__ import annotations

import importlib
import math
from collections.abc import Callable
from functools import partial
from numbers import Real
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
    """Lengths of the trajectories of one batch, each an integer tensor of shape ``[bs]``."""

    effective_token_lengths: torch.Tensor  # tokens under the loss mask
    turn_counts: torch.Tensor              # distinct active turn ids (token count without ids)
    timestep_lengths: torch.Tensor         # whichever of the two ``gae_timestep_unit`` selects


GAELambdaFn = Callable[..., torch.Tensor]


def _is_plain_number(x) -> bool:
    # bool is an int subclass; a flag passed by mistake must not be read as 0 or 1
    return isinstance(x, Real) and not isinstance(x, bool)


def constant_gae_lambda(context: GAELambdaContext, *, value: float) -> torch.Tensor:
    """The static option as a schedule: ``value`` for each trajectory (lambda_fn.py:37-47)."""
    n = context["timestep_lengths"]
    return torch.full(n.shape, float(value), dtype=torch.float32, device=n.device)


def vapo_length_adaptive_gae(context: GAELambdaContext, *, alpha: float) -> torch.Tensor:
    """VAPO's length-adaptive lambda ``1 - 1 / (alpha * L)``, floored at 0 (lambda_fn.py:50-69).

    Trajectories without a timestep, and those short enough for the formula to go negative, get
    lambda 0.  ``alpha`` must be a positive number; this is checked before looking at the batch.
    """
    if not _is_plain_number(alpha) or not alpha > 0:
        raise ValueError(f"alpha must be a positive number, got {alpha!r}")
    n = context["timestep_lengths"]
    steps = n.to(torch.float32)
    lam = (1.0 - 1.0 / (float(alpha) * steps.clamp(min=1.0))).clamp(min=0.0)
    return lam.masked_fill(n <= 0, 0.0)


def relative_position_gae_lambda(context: GAELambdaContext, *, q: float) -> torch.Tensor:
    """Lambda ``q ** (1 / (L - 1))``: a terminal reward keeps the fraction ``q`` at a trajectory's
    first step whatever its length (lambda_fn.py:72-112).

    ``q`` is the retained fraction, a finite number in (0, 1].  One timestep leaves nothing to
    decay over (lambda 1); no timestep gives lambda 0.
    """
    if not _is_plain_number(q) or not math.isfinite(q) or not 0 < q <= 1:
        raise ValueError(f"q must be a finite number in (0, 1], got {q!r}")
    n = context["timestep_lengths"]
    transitions = (n - 1).clamp(min=1).to(torch.float32)
    lam = torch.exp(math.log(float(q)) / transitions)
    lam = lam.masked_fill(n == 1, 1.0)
    return lam.masked_fill(n < 1, 0.0)


def _import_dotted(path: str):
    module_name, sep, attr = path.rpartition(".")
    if not sep or not module_name or not attr:
        raise ValueError(f"Invalid module path: {path!r}. Expected format 'module.path.ObjectName'.")
    try:
        module = importlib.import_module(module_name)
    except ImportError as err:
        raise ImportError(f"Failed to import module '{module_name}' from path '{path}': {err}") from err
    if not hasattr(module, attr):
        raise AttributeError(f"Module '{module_name}' has no attribute '{attr}'.")
    return getattr(module, attr)


def resolve_gae_lambda_fn(gae_lambda: float | str) -> tuple[GAELambdaFn, bool]:
    """Turn the ``gae_lambda`` option into ``(schedule, is_custom)`` (lambda_fn.py:115-141).

    A number becomes :func:`constant_gae_lambda` bound to it (``is_custom`` False, so callers can
    keep passing the number itself to the kernel); a non-empty string is imported as
    ``package.module.function`` (``is_custom`` True: the schedule has to be evaluated per batch,
    with the ``gae_lambda_kwargs`` of the configuration).  Anything else is a ``TypeError``.
    """
    if isinstance(gae_lambda, bool):
        raise TypeError("gae_lambda must be a float or dotted function path, not bool")
    if _is_plain_number(gae_lambda):
        return partial(constant_gae_lambda, value=float(gae_lambda)), False
    if not (isinstance(gae_lambda, str) and gae_lambda):
        raise TypeError(f"gae_lambda must be a float or a non-empty dotted function path, got {gae_lambda!r}")
    fn = _import_dotted(gae_lambda)
    if not callable(fn):
        raise TypeError(f"Imported gae_lambda object is not callable: {gae_lambda}")
    return fn, True
