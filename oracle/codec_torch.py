"""CPU oracle (torch ops) for the INT8 group codec.  TEST INFRASTRUCTURE ONLY.

The reference's portable codec is a short sequence of torch tensor ops; this
file restates that sequence on CPU tensors so parity tests can compare the HIP
path with "the same library ops the reference would have run" for every dtype
(fp32 / fp16 / bf16) without hand-written 16-bit rounding.  It is also the
thing timed as the CPU baseline.  Only tests, the smoke check and the
benchmark's CPU-baseline leg may import it.

Reference lines followed (paths under the upstream repository):

* ``quantize``         ccdl_comm/quantization/torch_fallback.py:24-36,56-61
* ``dequantize``       ccdl_comm/quantization/torch_fallback.py:48-53
* ``reduce_payloads``  ccdl_comm/communication/gather_reduce.py:27-45
* ``pack``             ccdl_comm/communication/payload_packing.py:63-68,190-193
* ``ef_round_trip``    ccdl_comm/communication/ddp.py:69-97 with
                       ccdl_comm/quantization/error_feedback.py:27-41

It is pinned against the numpy and scalar-C restatements and against
closed-form invariants in tests/test_oracle_pins.py.  The int8 cast of a NaN
quotient is undefined in the reference; here a NaN quotient is mapped to code
0 before the cast so all three restatements agree.
"""
from __future__ import annotations

import torch

_TORCH_DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}
_EPS = torch.finfo(torch.float32).eps


def torch_dtype(name: str) -> torch.dtype:
    try:
        return _TORCH_DTYPES[name]
    except KeyError:
        raise ValueError(f"unsupported dtype {name!r}") from None


def quantize(tensor: torch.Tensor, group_size: int = 64):
    """Return ``(codes int8[G*g], scales float32[G])`` for any-shape fp16/bf16/fp32 input."""
    values = tensor.reshape(-1)
    tail = values.numel() % group_size
    if tail:
        values = torch.cat([values, values.new_zeros(group_size - tail)])
    rows = values.reshape(-1, group_size).to(torch.float32)
    peak = rows.abs().amax(dim=1)
    scales = (peak / 127.0).clamp(min=_EPS)
    steps = (rows / scales.unsqueeze(1)).round().clamp(-127, 127)
    steps = torch.where(torch.isnan(steps), torch.zeros_like(steps), steps)
    return steps.to(torch.int8).reshape(-1), scales


def dequantize(codes: torch.Tensor, scales: torch.Tensor, numel: int, group_size: int = 64,
               dtype: str = "fp32") -> torch.Tensor:
    rows = codes.reshape(-1, group_size).to(torch.float32)
    decoded = rows * scales.unsqueeze(1)
    return decoded.reshape(-1)[:numel].to(torch_dtype(dtype))


def reduce_payloads(payloads, numel: int, group_size: int = 64, dtype: str = "fp32",
                    reduce: str = "sum") -> torch.Tensor:
    """Decode each payload to ``dtype``; add them left to right; ``mean`` divides by the count."""
    if not payloads:
        raise ValueError("cannot reduce an empty payload list")
    if reduce not in ("sum", "mean"):
        raise ValueError(f"unsupported gather-reduce mode: {reduce}")
    acc = None
    for codes, scales in payloads:
        term = dequantize(codes, scales, numel, group_size, dtype)
        acc = term if acc is None else acc + term
    return acc / len(payloads) if reduce == "mean" else acc


def pack(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    return torch.cat([codes.contiguous().view(torch.uint8).reshape(-1),
                      scales.contiguous().view(torch.uint8).reshape(-1)])


def ef_round_trip(grad: torch.Tensor, residual: torch.Tensor | None, group_size: int = 64,
                  restored_dtype: str = "fp32"):
    """p = g + r (torch promotion); q = quant(p); restored = dequant(q); r' = p - restored."""
    prepared = grad if residual is None else grad + residual
    codes, scales = quantize(prepared, group_size)
    restored = dequantize(codes, scales, prepared.numel(), group_size, restored_dtype)
    return codes, scales, restored, prepared - restored
