"""GPU codec callables with the calling convention of the reference's portable codec
(``quantize(tensor, config) -> CompressedPayload``, ``dequantize(payload, shape, config, dtype)``;
``ccdl_comm/quantization/torch_fallback.py:10-53``), to be injected wherever that codec is injected:
``create_ddp_comm_hook(quantize=, dequantize=)``, ``DDPBucketProcessor``, ``CompressedAllGatherReduce``.

Payloads are bit-identical to the portable codec's: ``buffer`` int8 codes in element order (tail group
zero padded), ``metadata["scales"]`` float32 per group, ``metadata["original_numel"]``.  Codes and
scales are adjacent views of one ``uint8`` allocation in wire order, so the fused-payload packer
ships them without a copy.
"""
from __future__ import annotations

from collections.abc import Hashable, Sequence
from typing import Any

import torch

from lowbit_comm_amd.communication.collectives import PackedPayload
from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip import ops
from lowbit_comm_amd.quantization.error_feedback import ErrorFeedbackState

_NAME_OF = ops.DTYPE_NAMES


def _check_policy(config: CompressionConfig) -> None:
    if config.quant_type != "linear":
        raise ValueError("the HIP codec supports only quant_type='linear'")
    if config.bit != 8:
        raise ValueError("the HIP codec only supports bit=8")
    if config.topk != 0 or config.stochastic:
        raise ValueError("the HIP codec supports neither top-k outliers nor stochastic rounding")


def ccdl_dtype(tensor: torch.Tensor) -> str:
    try:
        return _NAME_OF[tensor.dtype]
    except KeyError:
        raise ValueError(f"cannot infer CCDL dtype from tensor dtype: {tensor.dtype!r}") from None


def torch_dtype(name: str) -> torch.dtype:
    try:
        return ops.TORCH_DTYPES[name]
    except KeyError:
        raise ValueError(f"unsupported dtype: {name!r}") from None


def _flat(tensor: torch.Tensor) -> torch.Tensor:
    flat = tensor.reshape(-1)
    return flat if flat.is_contiguous() else flat.contiguous()


def _payload_views(payload: Any, group_size: int) -> tuple[torch.Tensor, torch.Tensor, int]:
    """``(codes, scales, original_numel)`` from a CompressedPayload, a dict, or a packed uint8 tensor."""
    if isinstance(payload, torch.Tensor):
        padded = payload.numel() // (group_size + 4) * group_size
        codes, scales = ops.split_payload(payload.reshape(-1), padded, group_size)
        return codes, scales, padded
    buffer = payload.buffer if hasattr(payload, "buffer") else payload["buffer"]
    metadata = payload.metadata if hasattr(payload, "metadata") else payload.get("metadata", {})
    codes = buffer.reshape(-1)
    if codes.dtype == torch.uint8:
        codes = codes.view(torch.int8)
    return codes, metadata["scales"], int(metadata.get("original_numel", codes.numel()))


def quantize_tensor_hip(tensor: torch.Tensor, config: CompressionConfig, *, out: torch.Tensor | None = None,
                        residual: torch.Tensor | None = None) -> PackedPayload:
    """Group-wise INT8 quantization on the GPU.  ``out``: optional packed ``uint8`` buffer of
    ``payload_nbytes(tensor.numel())`` bytes to write into (no allocation).  ``residual`` is added first."""
    _check_policy(config)
    flat = _flat(tensor)
    numel = flat.numel()
    g = config.group_size
    nbytes = ops.payload_nbytes(numel, g)
    packed = out if out is not None else torch.empty(nbytes, dtype=torch.uint8, device=flat.device)
    codes, scales = ops.split_payload(packed, numel, g)
    if numel and not ops.quant_pack_into(flat, codes, scales, group_size=g,
                                         residual=None if residual is None else _flat(residual)):
        raise ValueError(f"the HIP codec has no kernel for dtype {tensor.dtype} with this residual")
    return PackedPayload(buffer=codes, shape=tuple(tensor.shape), dtype=ccdl_dtype(tensor),
                         metadata={"scales": scales, "original_numel": numel}, packed=packed)


def dequantize_tensor_hip(payload: Any, shape: tuple[int, ...], config: CompressionConfig, dtype: str, *,
                          out: torch.Tensor | None = None) -> torch.Tensor:
    """Decode a payload of :func:`quantize_tensor_hip` (or of the portable codec) to ``dtype``."""
    codes, scales, numel = _payload_views(payload, config.group_size)
    target = out if out is not None else torch.empty(numel, dtype=torch_dtype(dtype), device=codes.device)
    if numel and not ops.dequant_into(codes, scales, target.reshape(-1), numel=numel, group_size=config.group_size):
        raise ValueError(f"the HIP codec cannot decode to {dtype}")
    return target.reshape(-1)[:numel].reshape(shape)


def dequantize_reduce_hip(payloads: Sequence[Any], shape: tuple[int, ...], config: CompressionConfig, dtype: str,
                          reduce: str = "sum", *, out: torch.Tensor | None = None) -> torch.Tensor | None:
    """Fused decode of all payloads and left-fold sum in list order (``mean`` divides by the count).

    Returns ``None`` when there are more than 8 payloads (the caller falls back to decode-then-add),
    so it can be passed as ``CompressedAllGatherReduce.fused_decompress_reduce``.
    """
    if not payloads:
        raise ValueError("cannot reduce an empty payload list")
    if reduce not in ("sum", "mean"):
        raise ValueError(f"unsupported gather-reduce mode: {reduce}")
    if len(payloads) > ops.MAX_PAYLOADS:
        return None
    views = [_payload_views(p, config.group_size) for p in payloads]
    numel = views[0][2]
    target = out if out is not None else torch.empty(numel, dtype=torch_dtype(dtype), device=views[0][0].device)
    pairs = [(codes, scales) for codes, scales, _ in views]
    divisor = float(len(payloads)) if reduce == "mean" else 1.0
    if numel and not ops.dequant_reduce_into(pairs, target.reshape(-1), numel=numel, group_size=config.group_size,
                                             divisor=divisor):
        return None
    return target.reshape(-1)[:numel].reshape(shape)


class FusedErrorFeedbackCodec:
    """Local bucket round trip with error feedback in ONE kernel per bucket.

    ``step(key, grad, dtype)`` computes ``p = grad + residual[key]``, quantizes ``p``, decodes it to
    ``dtype`` and stores ``residual[key] = p - restored`` - the sequence ``compensate -> quantize ->
    dequantize -> update`` of the reference's bucket processor (ccdl_comm/communication/ddp.py:69-97)
    without materialising ``p`` or re-reading the codes.  Residuals and workspaces are kept per key
    and reused, so a steady-state step allocates nothing.
    """

    def __init__(self, config: CompressionConfig, *, error_feedback: ErrorFeedbackState | None = None,
                 residual_dtype: torch.dtype | None = torch.float32) -> None:
        _check_policy(config)
        self.config = config
        self.error_feedback = error_feedback if error_feedback is not None else ErrorFeedbackState()
        self.residual_dtype = residual_dtype
        self._workspaces: dict[Hashable, dict[str, Any]] = {}

    def _workspace(self, key: Hashable, grad: torch.Tensor, restored_dtype: torch.dtype) -> dict[str, Any]:
        numel = grad.numel()
        signature = (numel, grad.dtype, restored_dtype, grad.device)
        ws = self._workspaces.get(key)
        if ws is None or ws["signature"] != signature:
            g = self.config.group_size
            packed = torch.empty(ops.payload_nbytes(numel, g), dtype=torch.uint8, device=grad.device)
            codes, scales = ops.split_payload(packed, numel, g)
            ws = {"signature": signature, "packed": packed, "codes": codes, "scales": scales,
                  "restored": torch.empty(numel, dtype=restored_dtype, device=grad.device), "bound": {}}
            self._workspaces[key] = ws
        return ws

    def step(self, key: Hashable, grad: torch.Tensor, dtype: str | None = None, *, update: bool = True,
             apply: bool = True) -> tuple[PackedPayload, torch.Tensor]:
        """Returns ``(payload, restored)``; ``restored`` has ``grad``'s shape and dtype ``dtype``."""
        flat = _flat(grad)
        restored_dtype = torch_dtype(dtype) if dtype is not None else grad.dtype
        ws = self._workspace(key, flat, restored_dtype)
        residual = self.error_feedback.get(key) if apply else None
        if residual is not None and (not isinstance(residual, torch.Tensor) or residual.numel() != flat.numel()
                                     or residual.device != flat.device):
            self.error_feedback.clear(key)
            residual = None
        if residual is not None:
            residual = residual.reshape(-1)
        p_dtype = flat.dtype if residual is None else ops.promote(flat.dtype, residual.dtype)
        new_dtype = ops.promote(p_dtype, restored_dtype)
        new_residual = None
        if update:
            if residual is not None and residual.dtype == new_dtype and residual.is_contiguous():
                new_residual = residual            # in place
            else:
                new_residual = torch.empty(flat.numel(), dtype=new_dtype, device=flat.device)
        signature = (flat.data_ptr(), None if residual is None else residual.data_ptr(),
                     None if new_residual is None else new_residual.data_ptr())
        bound = ws["bound"].get(signature)
        if bound is None:
            bound = ops.bind_quant_pack(flat, ws["codes"], ws["scales"], group_size=self.config.group_size,
                                        residual=residual, new_residual=new_residual, restored=ws["restored"])
            ws["bound"] = {signature: bound}
        if flat.numel() and not bound():
            raise ValueError(f"no fused error-feedback kernel for gradient {flat.dtype} / residual "
                             f"{None if residual is None else residual.dtype} / restored {restored_dtype}")
        if update:
            self.error_feedback.put(key, new_residual.reshape(grad.shape))
        payload = PackedPayload(buffer=ws["codes"], shape=tuple(grad.shape), dtype=ccdl_dtype(grad),
                                metadata={"scales": ws["scales"], "original_numel": flat.numel()},
                                packed=ws["packed"])
        return payload, ws["restored"].reshape(grad.shape)
