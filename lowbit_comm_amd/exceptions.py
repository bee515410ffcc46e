"""Public error types (same names and hierarchy as the reference's ``ccdl_comm/exceptions.py``)."""
from __future__ import annotations


class CCDLError(RuntimeError):
    """Root of every error this package raises on purpose."""


class CCDLUnavailableError(CCDLError):
    """The native codec library (or a symbol of it) cannot be used."""


class UnsupportedCollective(CCDLError):
    """A collective or strategy that this runtime does not provide."""

    def __init__(self, collective: str, *, reason: str | None = None) -> None:
        text = f"unsupported CCDL collective or strategy: {collective}"
        super().__init__(f"{text} ({reason})" if reason else text)
        self.collective = collective
        self.reason = reason
