"""Error types raised on purpose by this package.  Names and hierarchy follow the reference
(``ccdl_comm/exceptions.py``) so ``except`` clauses written against it keep working."""
from __future__ import annotations


class CCDLError(RuntimeError):
    """Common base class."""


class CCDLUnavailableError(CCDLError):
    """The native codec library, one of its symbols, or a GPU is missing.  Never papered over with a
    CPU implementation."""


class UnsupportedCollective(CCDLError):
    """A collective, strategy or pipeline this runtime does not provide; ``collective`` names it and
    ``reason`` (optional) says why."""

    def __init__(self, collective: str, *, reason: str | None = None) -> None:
        self.collective, self.reason = collective, reason
        detail = f" ({reason})" if reason else ""
        super().__init__(f"unsupported CCDL collective or strategy: {collective}{detail}")
