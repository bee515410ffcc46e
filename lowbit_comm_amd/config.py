"""Compression policy.  Field names, defaults and validation messages mirror the reference's
``ccdl_comm/config.py:22-77`` so configs move between the two packages unchanged."""
from __future__ import annotations

from dataclasses import dataclass

_CHOICES = {
    "bit": (4, 8),
    "group_size": (16, 32, 64),
    "topk": (0, 1, 2),
}
_NAMED_CHOICES = {
    "quant_type": ("e2m1", "e3m0", "linear", "normal", "uniform"),
    "target": ("collective", "ddp_gradient_bucket", "p2p", "tensor"),
    "error_feedback_policy": ("always", "large_bucket_only", "none", "periodic", "warmup_then_enable"),
}
_STABLE_BITS = (8,)


@dataclass(frozen=True)
class CompressionConfig:
    """User-facing compression policy; the default is linear 8-bit, group 64, error feedback on."""

    bit: int = 8
    group_size: int = 64
    topk: int = 0
    quant_type: str = "linear"
    stochastic: bool = False
    error_feedback: bool = True
    target: str = "tensor"
    warmup_steps: int = 0
    fallback: str = "bf16_compress"
    allow_experimental: bool = False
    compact: bool = False
    error_feedback_policy: str = "always"
    error_feedback_min_numel: int = 0
    error_feedback_warmup_steps: int = 0
    error_feedback_period: int = 1

    def __post_init__(self) -> None:
        for name, allowed in _CHOICES.items():
            value = getattr(self, name)
            if value not in allowed:
                raise ValueError(f"Unsupported {name}={value}; expected one of {sorted(allowed)}")
            if name == "bit" and value not in _STABLE_BITS and not self.allow_experimental:
                raise ValueError(f"bit={value} is experimental; set allow_experimental=True to opt in")
        for name, allowed in _NAMED_CHOICES.items():
            value = getattr(self, name)
            if value not in allowed:
                raise ValueError(f"Unsupported {name}={value!r}; expected one of {sorted(allowed)}")
        if self.error_feedback_min_numel < 0:
            raise ValueError("error_feedback_min_numel must be >= 0")
        if self.error_feedback_warmup_steps < 0:
            raise ValueError("error_feedback_warmup_steps must be >= 0")
        if self.error_feedback_period <= 0:
            raise ValueError("error_feedback_period must be > 0")

    def effective_error_feedback_policy(self) -> str:
        """``"none"`` when error feedback is switched off, else the configured policy."""
        return self.error_feedback_policy if self.error_feedback else "none"
