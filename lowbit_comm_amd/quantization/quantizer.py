"""``Quantizer``: a config, a dtype and the three codec entry points bound together, with the method
names of the reference's facade object (``ccdl_comm/quantization/quantizer.py:10-67``)."""
from __future__ import annotations

import dataclasses
from typing import Any, Callable

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.quantization import codec as _codec


class Quantizer:
    """Carries ``config``, the default ``dtype`` name (``"auto"``, ``"fp16"``, ``"bf16"``, ``"fp32"``) and an
    optional pre-resolved ``extension_status``; the codec functions can be replaced for testing."""

    def __init__(self, config: CompressionConfig | None = None, *, dtype: str = "auto",
                 extension_status: Any | None = None, quantize_fn: Callable[..., Any] | None = None,
                 dequantize_fn: Callable[..., Any] | None = None, allocate_fn: Callable[..., Any] | None = None) -> None:
        self.config = CompressionConfig() if config is None else config
        self.dtype = dtype
        self.extension_status = extension_status
        self._entry = {
            "quantize": quantize_fn or _codec.quantize_tensor,
            "dequantize": dequantize_fn or _codec.dequantize_tensor,
            "allocate": allocate_fn or _codec.allocate_quantized_buffer,
        }

    def _dtype(self, override: str | None) -> str:
        return override if override else self.dtype

    def quantize(self, tensor: Any, output: Any | None = None) -> Any:
        """Quantized buffer of ``tensor`` (written into ``output`` when given)."""
        return self._entry["quantize"](tensor, self.config, extension_status=self.extension_status, output=output)

    def dequantize(self, buffer: Any, shape: tuple[int, ...], output: Any | None = None, *,
                   reduce_op: str = "none", dtype: str | None = None) -> Any:
        """Decoded tensor of ``shape``; ``reduce_op`` combines with the content of ``output``."""
        options = dict(dtype=self._dtype(dtype), extension_status=self.extension_status, output=output,
                       reduce_op=reduce_op)
        return self._entry["dequantize"](buffer, shape, self.config, **options)

    def allocate_q(self, tensor: Any, *, dtype: str | None = None) -> Any:
        """A buffer large enough for the quantized form of ``tensor``."""
        return self._entry["allocate"](tensor, self.config, dtype=self._dtype(dtype))

    def payload_bytes(self, numel: int, *, dtype: str | None = None, wire_format: str = "portable") -> int:
        """Bytes of the quantized form of ``numel`` elements (``dtype`` defaults to this object's; an
        ``"auto"`` dtype is sized as fp32, which is exact for the portable wire format)."""
        from lowbit_comm_amd.quantization.sizing import estimate_quantized_size

        name = self._dtype(dtype)
        return estimate_quantized_size(numel, dtype="fp32" if name == "auto" else name, config=self.config,
                                       wire_format=wire_format).quantized_bytes

    def dequantize_reduce(self, buffers: list, shape: tuple[int, ...], output: Any | None = None, *,
                          reduce: str = "sum", dtype: str | None = None) -> Any:
        """Decode every buffer and reduce them in list order (``sum`` or ``mean``); fused on the GPU when an
        ``output`` workspace is given and there are at most eight buffers."""
        return _codec.dequantize_reduce_tensors(buffers, shape, self.config, dtype=self._dtype(dtype),
                                                extension_status=self.extension_status, output=output, reduce=reduce)

    def update_residual(self, prepared: Any, restored: Any, residual: Any) -> Any:
        """``residual <- prepared - restored`` on the device; returns ``residual``."""
        return _codec.update_error_feedback_residual(prepared, restored, residual,
                                                     extension_status=self.extension_status)

    def is_quantized(self) -> bool:
        return self.config.bit < 16

    def __repr__(self) -> str:
        c = self.config
        return (f"Quantizer(bit={c.bit}, group_size={c.group_size}, quant_type={c.quant_type!r}, "
                f"dtype={self.dtype!r})")

    def to_dict(self) -> dict[str, Any]:
        return {"config": dataclasses.asdict(self.config), "dtype": self.dtype}

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "Quantizer":
        return cls(CompressionConfig(**data["config"]), dtype=str(data.get("dtype", "auto")))
