"""Decides, per bucket and step, whether the stored residual is added to the gradient (``apply``) and
whether it is refreshed afterwards (``update``).  Policies and reason strings are those of the
reference (``ccdl_comm/quantization/error_feedback_policy.py:17-63``): ``none``, ``always``,
``large_bucket_only``, ``warmup_then_enable``, ``periodic``.
"""
from __future__ import annotations

from collections.abc import Hashable
from dataclasses import dataclass, field
from typing import Callable

from lowbit_comm_amd.config import CompressionConfig


@dataclass(frozen=True)
class ErrorFeedbackDecision:
    apply: bool
    update: bool
    reason: str


def _both(flag: bool, reason: str) -> ErrorFeedbackDecision:
    return ErrorFeedbackDecision(apply=flag, update=flag, reason=reason)


def _never(cfg: CompressionConfig, step: int, numel: int) -> ErrorFeedbackDecision:
    return _both(False, "error feedback disabled")


def _always(cfg: CompressionConfig, step: int, numel: int) -> ErrorFeedbackDecision:
    return _both(True, "error feedback policy always")


def _large_only(cfg: CompressionConfig, step: int, numel: int) -> ErrorFeedbackDecision:
    limit = cfg.error_feedback_min_numel
    relation = "below" if numel < limit else "reached"
    return _both(numel >= limit, f"bucket numel {numel} {relation} error feedback threshold {limit}")


def _after_warmup(cfg: CompressionConfig, step: int, numel: int) -> ErrorFeedbackDecision:
    warmup = cfg.error_feedback_warmup_steps
    relation = "before" if step < warmup else "reached"
    return _both(step >= warmup, f"bucket step {step} {relation} error feedback warmup {warmup}")


def _periodic(cfg: CompressionConfig, step: int, numel: int) -> ErrorFeedbackDecision:
    period = cfg.error_feedback_period
    if step % period:
        return ErrorFeedbackDecision(True, False, f"bucket step {step} skips error feedback update until period {period}")
    return ErrorFeedbackDecision(True, True, f"bucket step {step} updates error feedback every {period} steps")


_RULES: dict[str, Callable[[CompressionConfig, int, int], ErrorFeedbackDecision]] = {
    "none": _never, "always": _always, "large_bucket_only": _large_only,
    "warmup_then_enable": _after_warmup, "periodic": _periodic,
}


@dataclass
class ErrorFeedbackPolicy:
    """Step counters are per bucket key; ``advance`` is called once per processed bucket."""

    config: CompressionConfig
    _steps: dict[Hashable, int] = field(default_factory=dict)

    def decide(self, key: Hashable, *, numel: int) -> ErrorFeedbackDecision:
        name = self.config.effective_error_feedback_policy()
        rule = _RULES.get(name)
        if rule is None:
            raise ValueError(f"unsupported error feedback policy: {name}")
        return rule(self.config, self._steps.get(key, 0), numel)

    def advance(self, key: Hashable) -> None:
        self._steps[key] = 1 + self._steps.get(key, 0)
