"""When to apply and when to refresh the error-feedback residual of a bucket
(behaviour of ``ccdl_comm/quantization/error_feedback_policy.py:17-63``)."""
from __future__ import annotations

from collections.abc import Hashable
from dataclasses import dataclass, field

from lowbit_comm_amd.config import CompressionConfig


@dataclass(frozen=True)
class ErrorFeedbackDecision:
    apply: bool
    update: bool
    reason: str


@dataclass
class ErrorFeedbackPolicy:
    """Per-bucket step counters plus the rule set selected by ``config.error_feedback_policy``."""

    config: CompressionConfig
    _steps: dict[Hashable, int] = field(default_factory=dict)

    def decide(self, key: Hashable, *, numel: int) -> ErrorFeedbackDecision:
        rule = self.config.effective_error_feedback_policy()
        step = self._steps.get(key, 0)
        cfg = self.config
        if rule == "none":
            return ErrorFeedbackDecision(False, False, "error feedback disabled")
        if rule == "always":
            return ErrorFeedbackDecision(True, True, "error feedback policy always")
        if rule == "large_bucket_only":
            big = numel >= cfg.error_feedback_min_numel
            verb = "reached" if big else "below"
            return ErrorFeedbackDecision(
                big, big, f"bucket numel {numel} {verb} error feedback threshold {cfg.error_feedback_min_numel}")
        if rule == "warmup_then_enable":
            warm = step >= cfg.error_feedback_warmup_steps
            verb = "reached" if warm else "before"
            return ErrorFeedbackDecision(
                warm, warm, f"bucket step {step} {verb} error feedback warmup {cfg.error_feedback_warmup_steps}")
        if rule == "periodic":
            period = cfg.error_feedback_period
            if step % period == 0:
                return ErrorFeedbackDecision(True, True, f"bucket step {step} updates error feedback every {period} steps")
            return ErrorFeedbackDecision(True, False, f"bucket step {step} skips error feedback update until period {period}")
        raise ValueError(f"unsupported error feedback policy: {rule}")

    def advance(self, key: Hashable) -> None:
        self._steps[key] = self._steps.get(key, 0) + 1
