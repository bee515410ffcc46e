"""Tensor-level entry points for the payload format of the reference's CUDA extension.

A rank that runs ``ccdl_cuda_ops`` on an NVIDIA GPU produces and consumes flat ``uint8`` payloads whose
scales are group maxima in the tensor's own dtype and whose code bytes are swapped inside 2- or 4-byte
words (ccdl_comm/csrc/quantization/quant_pack_kernel.cu:101-162, dequant_reduce_kernel.cu:27-69).
These functions write and read exactly those bytes on a gfx950 GPU so both kinds of rank can sit in one
job.  Conventions are those of :mod:`lowbit_comm_amd.hip.ops`: ``*_into`` returns ``True`` (enqueued) or
``False`` (valid request without a kernel), contract violations raise ``RuntimeError``.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from lowbit_comm_amd.hip.library import load_library
from lowbit_comm_amd.hip.ops import (MAX_PAYLOADS, REDUCE_OPS, BoundLaunch, _device_tensor, _float_tensor, _ptr,
                                     _require, access_code, num_groups)


def payload_nbytes(numel: int, dtype: torch.dtype, group_size: int = 64, bit: int = 8) -> int:
    """``G * (g*bit/8 + element size)`` (ccdl_comm/csrc/quantization/quant_pack_kernel.cu:247-249)."""
    return num_groups(numel, group_size) * (group_size * bit // 8 + torch.empty((), dtype=dtype).element_size())


def _payload_rows(t: torch.Tensor, device: torch.device) -> None:
    _require(isinstance(t, torch.Tensor) and t.is_cuda and t.device == device, f"payloads must be a GPU tensor on {device}")
    _require(t.dtype == torch.uint8 and t.dim() == 2 and t.stride(1) == 1,
             "payloads must be a (world, stride) uint8 tensor with contiguous rows")


def _payload(t: torch.Tensor, name: str, device: torch.device, nbytes: int) -> None:
    _device_tensor(t, name, device)
    _require(t.dtype == torch.uint8, f"{name} must have uint8 dtype")
    _require(t.numel() == nbytes, f"{name} has an invalid quantized payload size: {t.numel()} bytes, expected {nbytes}")


def bind_quant_pack(x: torch.Tensor, payload: torch.Tensor, *, group_size: int = 64, compact: bool = True,
                    residual: torch.Tensor | None = None, bit: int = 8,
                    access: str | None = None) -> BoundLaunch:
    lib = load_library()
    code = _float_tensor(x, "input")
    _payload(payload, "output", x.device, payload_nbytes(x.numel(), x.dtype, group_size, bit))
    if residual is not None:
        _float_tensor(residual, "residual", x.device)
        _require(residual.dtype == x.dtype, "input and residual must have the same dtype")
        _require(residual.numel() == x.numel(), "input and residual must have the same number of elements")
    args = (_ptr(x), _ptr(residual), code, x.numel(), group_size, int(bit), int(compact), _ptr(payload))
    return BoundLaunch(lib.lbc_wire_quant_pack, args + (access_code(access),), x.device, lib, (x, residual, payload))


def quant_pack_into(x: torch.Tensor, payload: torch.Tensor, *, group_size: int = 64, compact: bool = True,
                    residual: torch.Tensor | None = None, bit: int = 8,
                    access: str | None = None) -> bool:
    """``payload = encode(x [+ residual])``; replaces native ``inplace_quantize_pack`` / ``inplace_quantize``."""
    return bind_quant_pack(x, payload, group_size=group_size, compact=compact, residual=residual, bit=bit,
                           access=access)()


def quant_pack(x: torch.Tensor, *, group_size: int = 64, compact: bool = True,
               residual: torch.Tensor | None = None, bit: int = 8, access: str | None = None) -> torch.Tensor:
    payload = torch.empty(payload_nbytes(x.numel(), x.dtype, group_size, bit), dtype=torch.uint8, device=x.device)
    if not quant_pack_into(x, payload, group_size=group_size, compact=compact, residual=residual, bit=bit,
                           access=access):
        raise RuntimeError(f"no kernel for group_size={group_size}, bit={bit}")
    return payload


def bind_quant_pack_chunks(x: torch.Tensor, payloads: torch.Tensor, world: int, *, group_size: int = 64,
                           compact: bool = True, residual: torch.Tensor | None = None, bit: int = 8,
                           access: str | None = None) -> BoundLaunch:
    """``payloads`` is a ``(world, stride)`` uint8 tensor; row d receives chunk d of ``ceil(numel/world)`` elements."""
    lib = load_library()
    code = _float_tensor(x, "input")
    _payload_rows(payloads, x.device)
    _require(payloads.shape[0] == world, "payloads must have one row per chunk")
    shard = -(-x.numel() // world) if x.numel() else 0
    _require(payloads.shape[1] >= payload_nbytes(shard, x.dtype, group_size, bit), "payload rows are too small")
    if residual is not None:
        _float_tensor(residual, "residual", x.device)
        _require(residual.dtype == x.dtype and residual.numel() == x.numel(),
                 "input and residual must have the same dtype and number of elements")
    args = (_ptr(x), _ptr(residual), code, x.numel(), world, group_size, int(bit), int(compact), _ptr(payloads),
            payloads.stride(0))
    return BoundLaunch(lib.lbc_wire_quant_pack_chunks, args + (access_code(access),), x.device, lib,
                       (x, residual, payloads))


def bind_dequant(payload: torch.Tensor, out: torch.Tensor, *, numel: int | None = None, group_size: int = 64,
                 compact: bool = True, reduce_op: str = "none", bit: int = 8,
                 access: str | None = None) -> BoundLaunch:
    lib = load_library()
    code = _float_tensor(out, "output")
    n = out.numel() if numel is None else int(numel)
    _require(0 <= n <= out.numel(), "numel exceeds the output size")
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    _payload(payload, "input", out.device, payload_nbytes(n, out.dtype, group_size, bit))
    args = (_ptr(payload), n, group_size, int(bit), int(compact), _ptr(out), code, REDUCE_OPS[reduce_op])
    return BoundLaunch(lib.lbc_wire_dequant, args + (access_code(access),), out.device, lib, (payload, out))


def dequant_into(payload: torch.Tensor, out: torch.Tensor, *, numel: int | None = None, group_size: int = 64,
                 compact: bool = True, reduce_op: str = "none", bit: int = 8,
                 access: str | None = None) -> bool:
    """Decode into ``out`` or combine with it (``sum``/``max``/``min``); replaces native ``inplace_dequantize``."""
    return bind_dequant(payload, out, numel=numel, group_size=group_size, compact=compact, reduce_op=reduce_op,
                        bit=bit, access=access)()


def bind_dequant_chunks(payloads: torch.Tensor, out: torch.Tensor, shard_numel: int, *, group_size: int = 64,
                        compact: bool = True, bit: int = 8, access: str | None = None) -> BoundLaunch:
    lib = load_library()
    code = _float_tensor(out, "output")
    _payload_rows(payloads, out.device)
    world = payloads.shape[0]
    _require(out.numel() <= world * shard_numel, "output is larger than world * shard_numel")
    _require(payloads.shape[1] >= payload_nbytes(shard_numel, out.dtype, group_size, bit), "payload rows are too small")
    args = (_ptr(payloads), payloads.stride(0), world, shard_numel, out.numel(), group_size, int(bit), int(compact),
            _ptr(out), code, REDUCE_OPS["none"])
    return BoundLaunch(lib.lbc_wire_dequant_chunks, args + (access_code(access),), out.device, lib, (payloads, out))


def bind_dequant_reduce(payloads: Sequence[torch.Tensor], out: torch.Tensor, *, numel: int | None = None,
                        group_size: int = 64, compact: bool = True, inv_divisor: float = 1.0,
                        fused_multiply_add: bool = True, prepared: torch.Tensor | None = None,
                        new_residual: torch.Tensor | None = None, access: str | None = None) -> BoundLaunch | None:
    """``None`` when the request has no kernel (more than 8 payloads, group size other than 64)."""
    lib = load_library()
    _require(len(payloads) > 0, "inputs must not be empty")
    _require(inv_divisor > 0, "inv_divisor must be > 0")
    code = _float_tensor(out, "output")
    device = out.device
    n = out.numel() if numel is None else int(numel)
    _require(0 <= n <= out.numel(), "numel exceeds the output size")
    if len(payloads) > MAX_PAYLOADS or group_size != 64:
        return None
    nbytes = payload_nbytes(n, out.dtype, group_size)
    pointers = (ctypes.c_void_p * len(payloads))()
    for r, payload in enumerate(payloads):
        _payload(payload, f"inputs[{r}]", device, nbytes)
        pointers[r] = payload.data_ptr()
    _require((prepared is None) == (new_residual is None), "prepared and new_residual must be given together")
    if prepared is not None:
        for name, t in (("prepared", prepared), ("residual", new_residual)):
            _float_tensor(t, name, device)
            _require(t.dtype == out.dtype, f"{name} and restored must have the same dtype")
            _require(t.numel() == n, f"{name} must have numel elements")
    args = (pointers, len(payloads), n, group_size, int(compact), float(inv_divisor), int(fused_multiply_add),
            _ptr(out), code, _ptr(prepared), _ptr(new_residual))
    return BoundLaunch(lib.lbc_wire_dequant_reduce, args + (access_code(access),), device, lib,
                       (tuple(payloads), out, prepared, new_residual))


def dequant_reduce_into(payloads: Sequence[torch.Tensor], out: torch.Tensor, **kwargs) -> bool:
    """``out = dtype(sum_r decode32(payload_r) * inv_divisor)``, optional ``new_residual = prepared - that``;
    replaces native ``try_inplace_dequantize_reduce_fused`` and
    ``inplace_dequantize_reduce_mean_update_error_feedback``."""
    bound = bind_dequant_reduce(payloads, out, **kwargs)
    return False if bound is None else bound()


# ---------------------------------------------------------------------------------------------------------
# the extension's remaining policies: non-linear 4-bit code books, stochastic rounding, top-k side channel
# ---------------------------------------------------------------------------------------------------------
QUANT_TYPES = {"linear": 0, "normal": 1, "uniform": 2, "e3m0": 3, "e2m1": 4}
_META_WORDS = {0: 1, 1: 3, 2: 4}


def bind_ring_step(received: torch.Tensor, chunk: torch.Tensor, send: torch.Tensor | None = None, *,
                   group_size: int = 64, compact: bool = True, reduce_op: str = "sum",
                   divisor: float = 1.0, access: str | None = None) -> BoundLaunch:
    """One ring / tree hop in this format: ``chunk (op)= decode(received)``, ``chunk *= 1/divisor`` (torch's device
    ``div_``), and - with ``send`` - the payload of the updated chunk, in one launch.  ``chunk`` holds whole groups."""
    lib = load_library()
    code = _float_tensor(chunk, "chunk")
    n = chunk.numel()
    _require(n % group_size == 0, "numel should be multiple of group_size")
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    _require(float(divisor) > 0.0, "divisor must be > 0")
    nbytes = payload_nbytes(n, chunk.dtype, group_size)
    _payload(received, "received payload", chunk.device, nbytes)
    if send is not None:
        _payload(send, "send payload", chunk.device, nbytes)
        _require(n == 0 or send.data_ptr() != received.data_ptr(), "the payload to send must not alias the received one")
    args = (_ptr(received), _ptr(chunk), code, n, group_size, int(compact), REDUCE_OPS[reduce_op], float(divisor),
            _ptr(send))
    return BoundLaunch(lib.lbc_wire_ring_step, args + (access_code(access),), chunk.device, lib,
                       (received, chunk, send))


def ring_step_into(received: torch.Tensor, chunk: torch.Tensor, send: torch.Tensor | None = None, **kwargs) -> bool:
    return bind_ring_step(received, chunk, send, **kwargs)()


def general_payload_nbytes(numel: int, dtype: torch.dtype, group_size: int = 64, bit: int = 8, topk: int = 0) -> int:
    """``G * (g*bit/8 + element size * (1 | 3 | 4))`` (ccdl_comm/csrc/quantization/gen_code_quant.py:167-178)."""
    _require(topk in _META_WORDS, f"topk must be 0, 1 or 2, got {topk}")
    item = torch.empty((), dtype=dtype).element_size()
    return num_groups(numel, group_size) * (group_size * bit // 8 + item * _META_WORDS[topk])


def _policy(quant_type: str, bit: int, topk: int) -> int:
    _require(quant_type in QUANT_TYPES, f"unsupported quant_type {quant_type!r}")
    _require(topk in _META_WORDS, f"topk must be 0, 1 or 2, got {topk}")
    _require(quant_type == "linear" or bit == 4, f"quant_type {quant_type!r} only supports 4-bit codes")
    return QUANT_TYPES[quant_type]


def bind_quant_general(x: torch.Tensor, payload: torch.Tensor, *, group_size: int = 64, bit: int = 8,
                       quant_type: str = "linear", topk: int = 0, stochastic: tuple[int, int] | None = None,
                       compact: bool = False) -> BoundLaunch:
    """``stochastic`` is the (seed, offset) pair of the Philox stream, ``None`` for round-to-nearest."""
    lib = load_library()
    code = _float_tensor(x, "input")
    kind = _policy(quant_type, bit, topk)
    _require(x.numel() % group_size == 0, "input numel should be multiple of group_size")
    _payload(payload, "output", x.device, general_payload_nbytes(x.numel(), x.dtype, group_size, bit, topk))
    seed, offset = (0, 0) if stochastic is None else (int(stochastic[0]), int(stochastic[1]))
    args = (_ptr(x), code, x.numel(), group_size, int(bit), kind, int(topk), int(stochastic is not None),
            seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF, int(compact), _ptr(payload))
    return BoundLaunch(lib.lbc_wire_quant_general, args, x.device, lib, (x, payload))


def quant_general_into(x: torch.Tensor, payload: torch.Tensor, **policy) -> bool:
    """Replaces native ``inplace_quantize`` for every policy of the reference's extension."""
    return bind_quant_general(x, payload, **policy)()


def bind_dequant_general(payload: torch.Tensor, out: torch.Tensor, *, group_size: int = 64, bit: int = 8,
                         quant_type: str = "linear", topk: int = 0, compact: bool = False,
                         reduce_op: str = "none") -> BoundLaunch:
    lib = load_library()
    code = _float_tensor(out, "output")
    kind = _policy(quant_type, bit, topk)
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    _require(out.numel() % group_size == 0, "output numel should be multiple of group_size")
    _payload(payload, "input", out.device, general_payload_nbytes(out.numel(), out.dtype, group_size, bit, topk))
    args = (_ptr(payload), out.numel(), group_size, int(bit), kind, int(topk), int(compact), _ptr(out), code,
            REDUCE_OPS[reduce_op])
    return BoundLaunch(lib.lbc_wire_dequant_general, args, out.device, lib, (payload, out))


def dequant_general_into(payload: torch.Tensor, out: torch.Tensor, **policy) -> bool:
    """Replaces native ``inplace_dequantize`` for every policy of the reference's extension."""
    return bind_dequant_general(payload, out, **policy)()
