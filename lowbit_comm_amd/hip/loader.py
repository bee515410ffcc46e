"""Import-safe discovery of the native codec (role of ``ccdl_comm/cuda/loader.py:9-43``).

Planners may probe availability on machines without a GPU or without a built library: the outcome
is returned as data, never raised.  Nothing here substitutes a CPU implementation - an unavailable
status makes every codec call raise :class:`~lowbit_comm_amd.exceptions.CCDLUnavailableError`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable


@dataclass(frozen=True)
class HipExtensionStatus:
    """``available`` + the duck-typed native ``module`` (or ``None`` and the ``reason``)."""

    available: bool
    module: object | None
    reason: str | None = None


# The facade accepts any object with these three attributes; the reference's name is kept as an alias.
CudaExtensionStatus = HipExtensionStatus

_cached: HipExtensionStatus | None = None


def _default_factory() -> object:
    from lowbit_comm_amd.hip.native_module import HipNativeModule

    return HipNativeModule()


def load_hip_extension(*, factory: Callable[[], object] | None = None, require_gpu: bool = True) -> HipExtensionStatus:
    """Load ``liblbc_hip.so`` behind the native-module interface.

    ``factory`` lets tests inject a stand-in module.  With ``require_gpu`` the status is unavailable
    when torch sees no GPU, so callers do not find out at the first launch.
    """
    global _cached
    if factory is None and _cached is not None:
        return _cached
    try:
        module = (factory or _default_factory)()
    except Exception as exc:  # missing .so, missing symbol, ABI mismatch, torch import failure
        return HipExtensionStatus(available=False, module=None, reason=str(exc) or type(exc).__name__)
    if factory is None and require_gpu:
        try:
            import torch

            if not torch.cuda.is_available():
                return HipExtensionStatus(available=False, module=None, reason="no GPU is visible to torch")
        except ImportError as exc:
            return HipExtensionStatus(available=False, module=None, reason=str(exc))
    status = HipExtensionStatus(available=True, module=module)
    if factory is None:
        _cached = status
    return status


load_cuda_extension = load_hip_extension
