"""``CompressionConfig`` - the user-facing compression policy.

Fields, defaults and the wording of validation errors follow the reference's dataclass
(``ccdl_comm/config.py:22-77``), so a config written for either package constructs in both.  The HIP
kernels implement the default policy (linear, 8 bit, group 16/32/64, no top-k, deterministic
rounding); other valid policies are reported as unsupported by the codec, not rejected here.
"""
from __future__ import annotations

from dataclasses import dataclass

# field -> allowed values; the first table prints values bare, the second quoted (as the reference does)
_NUMERIC_DOMAINS = {"bit": (4, 8), "group_size": (16, 32, 64), "topk": (0, 1, 2)}
_NAMED_DOMAINS = {
    "quant_type": ("e2m1", "e3m0", "linear", "normal", "uniform"),
    "target": ("collective", "ddp_gradient_bucket", "p2p", "tensor"),
    "error_feedback_policy": ("always", "large_bucket_only", "none", "periodic", "warmup_then_enable"),
}
_NON_EXPERIMENTAL_BITS = frozenset({8})
_LOWER_BOUNDS = (("error_feedback_min_numel", 0, "must be >= 0"),
                 ("error_feedback_warmup_steps", 0, "must be >= 0"),
                 ("error_feedback_period", 1, "must be > 0"))


@dataclass(frozen=True)
class CompressionConfig:
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
        for name, domain in _NUMERIC_DOMAINS.items():
            value = getattr(self, name)
            if value not in domain:
                raise ValueError(f"Unsupported {name}={value}; expected one of {sorted(domain)}")
        if self.bit not in _NON_EXPERIMENTAL_BITS and not self.allow_experimental:
            raise ValueError(f"bit={self.bit} is experimental; set allow_experimental=True to opt in")
        for name, domain in _NAMED_DOMAINS.items():
            value = getattr(self, name)
            if value not in domain:
                raise ValueError(f"Unsupported {name}={value!r}; expected one of {sorted(domain)}")
        for name, minimum, rule in _LOWER_BOUNDS:
            if getattr(self, name) < minimum:
                raise ValueError(f"{name} {rule}")

    def effective_error_feedback_policy(self) -> str:
        """The configured policy, or ``"none"`` when ``error_feedback`` is off."""
        return self.error_feedback_policy if self.error_feedback else "none"
