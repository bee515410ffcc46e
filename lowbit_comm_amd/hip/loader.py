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

_cached: dict[str, HipExtensionStatus] = {}

WIRE_FORMATS = ("portable", "native")


def _default_factory(wire_format: str) -> object:
    if wire_format == "native":
        from lowbit_comm_amd.hip.cuda_wire_module import HipCudaWireModule

        return HipCudaWireModule()
    from lowbit_comm_amd.hip.native_module import HipNativeModule

    return HipNativeModule()


def load_hip_extension(*, factory: Callable[[], object] | None = None, require_gpu: bool = True,
                       wire_format: str = "portable") -> HipExtensionStatus:
    """Load ``liblbc_hip.so`` behind the native-module interface.

    ``wire_format`` picks the payload bytes the module reads and writes: ``"portable"`` (the reference's
    torch codec: int8 codes then fp32 scales) or ``"native"`` (the bytes of the reference's CUDA extension,
    for jobs that mix both kinds of rank).  ``factory`` lets tests inject a stand-in module.  With
    ``require_gpu`` the status is unavailable when torch sees no GPU, so callers do not find out at the
    first launch.
    """
    if wire_format not in WIRE_FORMATS:
        raise ValueError(f"Unsupported wire_format={wire_format!r}; expected one of {list(WIRE_FORMATS)}")
    if factory is None and wire_format in _cached:
        return _cached[wire_format]
    try:
        module = factory() if factory is not None else _default_factory(wire_format)
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
        _cached[wire_format] = status
    return status


load_cuda_extension = load_hip_extension
