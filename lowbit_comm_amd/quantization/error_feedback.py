"""Per-bucket error-feedback residuals (behaviour of ``ccdl_comm/quantization/error_feedback.py:22-54``).

The state is tensor-library agnostic: it only uses ``+``, ``-``, ``detach``, ``clone`` and ``shape``
of what it is given, so host frameworks can drive it with their own tensor types.  The fused GPU
path (quantize and residual update in one kernel) lives in ``lowbit_comm_amd.hip.codec`` and
stores its residuals in the same object through :meth:`put`.
"""
from __future__ import annotations

from collections.abc import Hashable
from typing import Any


def _detached_copy(value: Any) -> Any:
    if hasattr(value, "detach"):
        value = value.detach()
    return value.clone() if hasattr(value, "clone") else value


def _shapes_agree(a: Any, b: Any) -> bool:
    sa, sb = getattr(a, "shape", None), getattr(b, "shape", None)
    return sa is None or sb is None or tuple(sa) == tuple(sb)


class ErrorFeedbackState:
    """``residual[key]`` = what compression dropped from bucket ``key`` last time."""

    def __init__(self, _residuals: dict[Hashable, Any] | None = None) -> None:
        self._residuals: dict[Hashable, Any] = {} if _residuals is None else _residuals

    def compensate(self, key: Hashable, tensor: Any) -> Any:
        """``tensor + residual[key]``; the tensor itself when there is no residual.  A residual whose
        shape no longer matches the bucket is dropped."""
        residual = self._residuals.get(key)
        if residual is None:
            return tensor
        if not _shapes_agree(tensor, residual):
            self.clear(key)
            return tensor
        return tensor + residual

    def update(self, key: Hashable, *, original: Any, transmitted: Any) -> None:
        """Store a detached copy of ``original - transmitted``."""
        self._residuals[key] = _detached_copy(original - transmitted)

    def put(self, key: Hashable, residual: Any) -> None:
        """Adopt ``residual`` as is (used by fused kernels that wrote it in place)."""
        self._residuals[key] = residual

    def get(self, key: Hashable) -> Any | None:
        return self._residuals.get(key)

    def clear(self, key: Hashable | None = None) -> None:
        if key is None:
            self._residuals.clear()
        else:
            self._residuals.pop(key, None)

    def keys(self) -> list[Hashable]:
        """Bucket keys that currently hold a residual."""
        return list(self._residuals)

    def __len__(self) -> int:
        return len(self._residuals)

    def state_dict(self) -> dict[Hashable, Any]:
        """Residuals by bucket key, for the host framework's checkpoint (the tensors themselves, not copies)."""
        return dict(self._residuals)

    def load_state_dict(self, state: dict[Hashable, Any]) -> None:
        """Replace all residuals with ``state`` (as produced by :meth:`state_dict`)."""
        self._residuals.clear()
        self._residuals.update(state)

    def __eq__(self, other: object) -> bool:
        return isinstance(other, ErrorFeedbackState) and self._residuals == other._residuals

    def __repr__(self) -> str:
        return f"ErrorFeedbackState(keys={list(self._residuals)!r})"
