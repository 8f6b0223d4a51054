"""Plain dataclass equivalents of the reference's config types used on the hot path.

Field names, defaults and validation follow ``areal/api/cli_args.py``: ``NormConfig``
(:43-96) and ``RejectionSamplingConfig`` (:1505-1668).  One deliberate difference:
``metric="binary_kl"`` is accepted, because the reference lists it among the field's choices
(:1565) and implements it (``functional.py:248-258``) while its ``__post_init__`` rejects it
(:1608).
"""

from __future__ import annotations

import warnings
from dataclasses import dataclass

_LEVELS = ("token", "sequence")
_ACTIONS = ("mask", "clamp")
_METRICS = ("ratio", "kl_k1", "kl_k2", "kl_k3", "binary_kl")
_AGGS = ("sum", "mean", "max")


@dataclass
class NormConfig:
    """Reward / advantage normalisation settings."""

    mean_level: str | None = "batch"
    mean_leave1out: bool = False
    std_level: str | None = "batch"
    std_unbiased: bool = True
    eps: float = 1e-5
    group_size: int = 1

    def __post_init__(self):
        levels = {"batch", "group", None}
        if self.mean_level not in levels:
            raise ValueError(f"mean_level must be 'batch', 'group' or None, got {self.mean_level}")
        if self.std_level not in levels:
            raise ValueError(f"std_level must be 'batch', 'group', or None, got {self.std_level}")
        if "group" in (self.mean_level, self.std_level) and self.group_size < 1:
            raise ValueError(
                "group_size must be a positive integer when using group normalization, "
                f"got {self.group_size}"
            )


@dataclass
class RejectionSamplingConfig:
    """Filtering of tokens / sequences by divergence between proximal and behaviour policy."""

    level: str = "token"
    action: str = "mask"
    metric: str = "ratio"
    agg: str = "mean"
    upper: float = 5.0
    lower: float | None = None

    def __post_init__(self):
        if self.level not in _LEVELS:
            raise ValueError(f"level must be one of {_LEVELS}, got '{self.level}'")
        if self.action not in _ACTIONS:
            raise ValueError(f"action must be one of {_ACTIONS}, got '{self.action}'")
        if self.metric not in _METRICS:
            raise ValueError(f"metric must be one of {_METRICS}, got '{self.metric}'")
        if self.agg not in _AGGS:
            raise ValueError(f"agg must be one of {_AGGS}, got '{self.agg}'")
        if self.lower is not None and self.lower > self.upper:
            raise ValueError(f"lower ({self.lower}) cannot be greater than upper ({self.upper})")
        if self.metric == "ratio":
            if self.upper <= 1.0:
                raise ValueError(
                    "upper must be > 1.0 for 'ratio' metric (otherwise all non-identical "
                    f"policy tokens will be filtered), got {self.upper}"
                )
            if self.lower is not None and self.lower <= 0:
                raise ValueError(f"lower must be positive for 'ratio' metric, got {self.lower}")
        if self.metric in ("kl_k2", "kl_k3", "binary_kl") and self.upper <= 0:
            raise ValueError(f"upper must be positive for '{self.metric}' metric, got {self.upper}")
        if self.action == "clamp" and self.metric != "ratio":
            raise ValueError(
                "action='clamp' only supports metric='ratio' (direct importance weight "
                f"truncation). Got metric='{self.metric}'. Use action='mask' for KL-based filtering."
            )
        if self.action == "clamp" and self.lower is None:
            self.lower = 0.0
        if self.level == "token" and self.agg != "mean":
            warnings.warn(
                f"agg='{self.agg}' is ignored when level='token'. "
                "Aggregation is only used for sequence-level filtering.",
                UserWarning,
                stacklevel=2,
            )
