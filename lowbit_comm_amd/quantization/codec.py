"""Codec facade: translates a :class:`CompressionConfig` into calls on the duck-typed native module.

Function names, keyword arguments, return conventions and the positional argument tuples handed to
the native module are those of the reference's ``ccdl_comm/quantization/codec.py:39-480`` (the tuples
are pinned by its ``tests/test_quantization_codec.py``), so code written against that facade runs
unchanged.  What differs is underneath: ``extension_status`` defaults to the HIP module
(``lowbit_comm_amd.hip.loader``), buffers carry the portable wire format (fp32 scales: size them
with ``allocate_quantized_buffer``), and there is no CPU fallback - an unavailable module raises
:class:`CCDLUnavailableError`.
"""
from __future__ import annotations

from math import prod
from typing import Any

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.exceptions import CCDLUnavailableError
from lowbit_comm_amd.quantization.sizing import estimate_quantized_size

_QUANT_TYPE_MEMBER = {"linear": "Linear", "normal": "Normal", "uniform": "Uniform", "e3m0": "E3M0", "e2m1": "E2M1"}
_DTYPE_MEMBER = {"fp16": "FP16", "bf16": "BF16", "fp32": "FP32"}
_REDUCE_MODES = ("sum", "mean")
_MODULE_LABEL = "native codec module"


# --------------------------------------------------------------------------- #
# native-module resolution
# --------------------------------------------------------------------------- #
def _module_of(extension_status: Any | None) -> object:
    if extension_status is None:
        from lowbit_comm_amd.hip.loader import load_hip_extension

        extension_status = load_hip_extension()
    if not extension_status.available or extension_status.module is None:
        raise CCDLUnavailableError(extension_status.reason or f"{_MODULE_LABEL} is not available")
    return extension_status.module


def _symbol(owner: object, name: str) -> Any:
    if not hasattr(owner, name):
        raise CCDLUnavailableError(f"{_MODULE_LABEL} missing required symbol: {name}")
    return getattr(owner, name)


def _quant_type(module: object, config: CompressionConfig) -> Any:
    return _symbol(_symbol(module, "QuantType"), _QUANT_TYPE_MEMBER[config.quant_type])


def _dtype(module: object, dtype: str) -> Any:
    return _symbol(_symbol(module, "DType"), _DTYPE_MEMBER[dtype])


def _reduce_op(module: object, reduce_op: str) -> Any:
    return _symbol(_symbol(module, "ReduceOP"), reduce_op.upper())


def _wire_format(module: object) -> str:
    return getattr(module, "NATIVE_WIRE_FORMAT", "native")


def _check_reduce(buffers: list, reduce: str) -> None:
    if not buffers:
        raise ValueError("buffers must not be empty")
    if reduce not in _REDUCE_MODES:
        raise ValueError(f"unsupported dequantize-reduce mode: {reduce}")


def _padded_numel(numel: int, group_size: int) -> int:
    return -(-numel // group_size) * group_size if numel else 0


def _zero_padded(tensor: Any, group_size: int) -> Any:
    """Flat copy padded with zeros to a whole number of groups; the tensor itself when already whole."""
    if not (hasattr(tensor, "numel") and hasattr(tensor, "reshape")):
        return tensor
    missing = -tensor.numel() % group_size
    if missing == 0:
        return tensor
    import torch

    flat = tensor.reshape((-1,))
    return torch.cat((flat, flat.new_zeros((missing,))), dim=0)


def _divide(decoded: Any, count: int, *, in_place: bool, exact: bool = True) -> Any:
    """``decoded / count``.  ``exact``: a true division on GPU tensors, as the portable CPU codec computes it,
    instead of the reciprocal multiply torch uses there; the CUDA byte format keeps torch's own division because
    that is what a rank running the CUDA extension computes (ccdl_comm/quantization/codec.py:339-343)."""
    if exact and getattr(decoded, "is_cuda", False):
        from lowbit_comm_amd.hip.ops import true_divide_

        return true_divide_(decoded if in_place else decoded.clone(), count)
    if in_place:
        decoded.div_(count)
        return decoded
    return decoded / count


def _trim_to_shape(decoded: Any, shape: tuple[int, ...]) -> Any:
    if not hasattr(decoded, "reshape"):
        return decoded
    count = getattr(decoded, "numel", None)
    if callable(count) and count() == prod(shape):          # nothing to trim: one view instead of three
        return decoded.reshape(shape)
    flat = decoded.reshape((-1,))
    try:
        flat = flat[:prod(shape)]
    except TypeError:
        pass
    return flat.reshape(shape)


# --------------------------------------------------------------------------- #
# workspace helpers
# --------------------------------------------------------------------------- #
def allocate_quantized_buffer(tensor: Any, config: CompressionConfig, *, dtype: str, torch_module: Any | None = None,
                              wire_format: str = "portable") -> Any:
    """A ``uint8`` buffer sized for the quantized form of ``tensor`` (portable wire format by default)."""
    if torch_module is None:
        import torch as torch_module
    estimate = estimate_quantized_size(int(tensor.numel()), dtype=dtype, config=config, wire_format=wire_format)
    return tensor.new_empty((estimate.quantized_bytes,), dtype=torch_module.uint8)


def allocate_dequantized_buffer(tensor: Any, shape: tuple[int, ...], config: CompressionConfig, *,
                                torch_module: Any | None = None) -> Any:
    """A decode workspace of ``tensor``'s dtype, padded to a whole number of groups."""
    del torch_module
    padded = _padded_numel(prod(shape), config.group_size) if shape else 0
    return tensor.new_empty((padded,), dtype=getattr(tensor, "dtype"))


# --------------------------------------------------------------------------- #
# quantize
# --------------------------------------------------------------------------- #
def writes_prepared(extension_status: Any | None) -> bool:
    """Can the native module's fused quantize also write ``tensor + residual`` (``prepared_out=``)?  The reference's
    extension cannot; the HIP module says so with ``QUANTIZE_PACK_WRITES_PREPARED``."""
    module = getattr(extension_status, "module", None)
    return bool(getattr(extension_status, "available", False) and getattr(module, "QUANTIZE_PACK_WRITES_PREPARED", False))


def _try_quantize_pack(module: object, tensor: Any, output: Any, residual: Any | None, config: CompressionConfig,
                       metadata: dict[str, Any] | None, quant_type: Any, prepared_out: Any | None = None) -> bool:
    fused = False
    native = getattr(module, "inplace_quantize_pack", None)
    if native is not None:
        extra = {} if prepared_out is None else {"prepared_out": prepared_out}     # a keyword only this build's module has
        fused = bool(native(tensor, output, residual, config.group_size, config.topk, config.stochastic,
                            config.bit, quant_type, config.compact, **extra))
    if metadata is not None:
        numel = int(tensor.numel())
        padded = _padded_numel(numel, config.group_size)
        metadata.update(original_numel=numel, padded_numel=padded, padding_numel=padded - numel,
                        fused_quant_pack=fused)
    return fused


def quantize_tensor(tensor: object, config: CompressionConfig, *, extension_status: Any | None = None,
                    output: object | None = None, residual: object | None = None,
                    metadata: dict[str, Any] | None = None, prepared_out: object | None = None) -> object:
    """Quantize ``tensor`` (plus ``residual``) into ``output`` or a fresh buffer; returns the buffer.

    With ``output`` the fused allocation-free call is tried first; if the native module declines, the
    padded ``inplace_quantize`` chain runs.  Raises :class:`CCDLUnavailableError` when the native
    module is missing or incomplete.

    ``prepared_out`` (an addition to the reference's signature, needs ``output`` and a module for which
    :func:`writes_prepared` is true): receives ``tensor + residual`` from the quantize launch, for the caller that
    needs it after the collective (``ccdl_comm/communication/ddp_hook.py:196,224-241``).
    """
    module = _module_of(extension_status)
    quant_type = _quant_type(module, config)
    if prepared_out is not None:
        if output is None or not getattr(module, "QUANTIZE_PACK_WRITES_PREPARED", False):
            raise ValueError("prepared_out needs output= and a native module whose fused quantize writes it")
        if not _try_quantize_pack(module, tensor, output, residual, config, metadata, quant_type, prepared_out):
            raise ValueError("the fused quantize declined this policy; quantize without prepared_out")
        return output
    if output is not None and _try_quantize_pack(module, tensor, output, residual, config, metadata, quant_type):
        return output
    prepared = _zero_padded(tensor if residual is None else tensor + residual, config.group_size)
    policy = (config.group_size, config.topk, config.stochastic, config.bit, quant_type, config.compact)
    if output is not None:
        _symbol(module, "inplace_quantize")(prepared, output, *policy)
        return output
    return _symbol(module, "quantize")(prepared, *policy)


def inplace_quantize_pack(tensor: object, output: object, residual: object | None, config: CompressionConfig,
                          metadata: dict[str, Any] | None = None, *, extension_status: Any | None = None) -> bool:
    """Allocation-free fused quantize+pack; ``False`` when the policy is unsupported (take a fallback)."""
    module = _module_of(extension_status)
    return _try_quantize_pack(module, tensor, output, residual, config, metadata, _quant_type(module, config))


# --------------------------------------------------------------------------- #
# dequantize
# --------------------------------------------------------------------------- #
def dequantize_tensor(buffer: object, shape: tuple[int, ...], config: CompressionConfig, *, dtype: str,
                      extension_status: Any | None = None, output: object | None = None,
                      reduce_op: str = "none") -> object:
    """Decode ``buffer`` to ``dtype`` (``fp16``/``bf16``/``fp32``), trimmed and reshaped to ``shape``."""
    module = _module_of(extension_status)
    quant_type = _quant_type(module, config)
    dtype_member = _dtype(module, dtype)
    op = _reduce_op(module, reduce_op)
    if output is None:
        decoded = _symbol(module, "dequantize")(buffer, config.group_size, config.topk, config.bit, op, quant_type,
                                                dtype_member, config.compact)
    else:
        _symbol(module, "inplace_dequantize")(buffer, output, config.group_size, config.topk, config.bit, op,
                                              quant_type, config.compact)
        decoded = output
    return _trim_to_shape(decoded, shape)


def dequantize_reduce_tensors(buffers: list[object], shape: tuple[int, ...], config: CompressionConfig, *,
                              dtype: str, extension_status: Any | None = None, output: object | None = None,
                              reduce: str = "sum") -> object:
    """Decode every buffer and reduce them (list order) into one tensor; ``reduce`` is ``sum`` or ``mean``."""
    _check_reduce(buffers, reduce)
    module = _module_of(extension_status)
    quant_type = _quant_type(module, config)
    dtype_member = _dtype(module, dtype)
    fused = False
    if output is None:
        decoded = None
        one_launch = getattr(module, "dequantize_reduce_mean", None) if reduce == "mean" else None
        if one_launch is not None:      # an extension that divides in the reduce launch itself (same bits)
            decoded = one_launch(buffers, config.group_size, config.topk, config.bit, quant_type, dtype_member,
                                 config.compact, len(buffers))
            fused = decoded is not None
        if decoded is None:
            decoded = _symbol(module, "dequantize_reduce")(buffers, config.group_size, config.topk, config.bit,
                                                           quant_type, dtype_member, config.compact)
    else:
        if hasattr(module, "inplace_dequantize_reduce_mean"):
            fused = inplace_dequantize_reduce_mean(buffers, output, config, extension_status=extension_status,
                                                   reduce=reduce)
        if not fused:
            _symbol(module, "inplace_dequantize_reduce")(buffers, output, config.group_size, config.topk,
                                                         config.bit, quant_type, config.compact)
        decoded = output
    if reduce == "mean" and not fused:
        decoded = _divide(decoded, len(buffers), in_place=output is not None,
                          exact=_wire_format(module) == "portable")
    return _trim_to_shape(decoded, shape)


def inplace_dequantize_reduce_mean(buffers: list[object], output: object, config: CompressionConfig, *,
                                   extension_status: Any | None = None, reduce: str = "sum") -> bool:
    """Fused decode+reduce(+mean) into a caller-owned ``output``; ``False`` if the native module declines."""
    _check_reduce(buffers, reduce)
    module = _module_of(extension_status)
    native = _symbol(module, "inplace_dequantize_reduce_mean")
    divisor = len(buffers) if reduce == "mean" else 1
    return bool(native(buffers, output, config.group_size, config.topk, config.bit, _quant_type(module, config),
                       config.compact, divisor))


def dequantize_reduce_update_error_feedback(buffers: list[object], prepared: object, residual: object,
                                            shape: tuple[int, ...], config: CompressionConfig, *, dtype: str,
                                            extension_status: Any | None = None, reduce: str = "sum") -> object:
    """Decode+reduce and ``residual = prepared - restored`` in one native call; returns ``restored``."""
    _check_reduce(buffers, reduce)
    module = _module_of(extension_status)
    quant_type = _quant_type(module, config)
    dtype_member = _dtype(module, dtype)
    native = _symbol(module, "dequantize_reduce_update_error_feedback")
    divisor = len(buffers) if reduce == "mean" else 1
    restored = native(buffers, prepared, residual, config.group_size, config.topk, config.bit, quant_type,
                      dtype_member, config.compact, divisor)
    return _trim_to_shape(restored, shape)


def inplace_dequantize_reduce_mean_update_error_feedback(buffers: list[object], prepared: object, restored: object,
                                                         residual: object, config: CompressionConfig, *,
                                                         extension_status: Any | None = None,
                                                         reduce: str = "sum") -> bool:
    """Workspace-aware fused decode+reduce(+mean)+residual update; ``False`` if the native module declines."""
    _check_reduce(buffers, reduce)
    module = _module_of(extension_status)
    native = _symbol(module, "inplace_dequantize_reduce_mean_update_error_feedback")
    divisor = len(buffers) if reduce == "mean" else 1
    return bool(native(buffers, prepared, restored, residual, config.group_size, config.topk, config.bit,
                       _quant_type(module, config), config.compact, divisor))


def update_error_feedback_residual(prepared: object, restored: object, residual: object, *,
                                   extension_status: Any | None = None) -> object:
    """``residual <- prepared - restored`` on the device; returns ``residual``."""
    module = _module_of(extension_status)
    _symbol(module, "inplace_error_feedback_update")(prepared, restored, residual)
    return residual
