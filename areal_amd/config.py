"""Configuration object of the rejection-sampling step (importance-weight cap).

Mirrors the fields, defaults and validation of ``RejectionSamplingConfig`` in
areal/api/cli_args.py:1223-1385, so that callers can pass either object (only
attribute access is used).
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass

LEVELS = ("token", "sequence")
ACTIONS = ("mask", "clamp")
METRICS = ("ratio", "kl_k1", "kl_k2", "kl_k3")
AGGS = ("sum", "mean", "max")


@dataclass
class RejectionSamplingConfig:
    level: str = "token"
    action: str = "mask"
    metric: str = "ratio"
    agg: str = "mean"
    upper: float = 5.0
    lower: float | None = None

    def __post_init__(self) -> None:
        for name, value, allowed in (
            ("level", self.level, LEVELS),
            ("action", self.action, ACTIONS),
            ("metric", self.metric, METRICS),
            ("agg", self.agg, AGGS),
        ):
            if value not in allowed:
                raise ValueError(f"{name} must be one of {allowed}, got '{value}'")
        if self.lower is not None and self.lower > self.upper:
            raise ValueError(f"lower ({self.lower}) cannot be greater than upper ({self.upper})")
        if self.metric == "ratio":
            if self.upper <= 1.0:
                raise ValueError(f"upper must be > 1.0 for 'ratio' metric, got {self.upper}")
            if self.lower is not None and self.lower <= 0:
                raise ValueError(f"lower must be positive for 'ratio' metric, got {self.lower}")
        if self.metric in ("kl_k2", "kl_k3") and self.upper <= 0:
            raise ValueError(f"upper must be positive for '{self.metric}' metric, got {self.upper}")
        if self.action == "clamp" and self.metric != "ratio":
            raise ValueError(
                f"action='clamp' only supports metric='ratio', got metric='{self.metric}'; "
                "use action='mask' for KL-based filtering"
            )
        if self.action == "clamp" and self.lower is None:
            self.lower = 0.0
        if self.level == "token" and self.agg != "mean":
            warnings.warn(
                f"agg='{self.agg}' is ignored when level='token'; it only applies to sequence-level filtering",
                UserWarning,
                stacklevel=2,
            )


@dataclass
class NormConfig:
    """Reward / advantage normalisation options; fields, defaults and validation texts of ``NormConfig`` in
    areal/api/cli_args.py:42-95."""

    mean_level: str | None = "batch"
    mean_leave1out: bool = False
    std_level: str | None = "batch"
    std_unbiased: bool = True
    eps: float = 1e-5
    group_size: int = 1

    def __post_init__(self) -> None:
        valid_levels = {"batch", "group", None}
        if self.mean_level not in valid_levels:
            raise ValueError(f"mean_level must be 'batch', 'group' or None, got {self.mean_level}")
        if self.std_level not in valid_levels:
            raise ValueError(f"std_level must be 'batch', 'group', or None, got {self.std_level}")
        if (self.mean_level == "group" or self.std_level == "group") and self.group_size < 1:
            raise ValueError(
                f"group_size must be a positive integer when using group normalization, got {self.group_size}"
            )
