"""Tensor-level entry points over the C ABI.

Every function takes torch tensors that already live on the GPU, checks the contract the C ABI
cannot see (device, contiguity, element counts), and enqueues on torch's current stream of the
tensors' device.  Functions named ``*_into`` write only into caller-owned tensors and return
``True`` (enqueued) or ``False`` (valid request this build has no kernel for - take a fallback),
mirroring the reference's native ``inplace_*`` functions (ccdl_comm/csrc/pybind.cpp:39-131);
contract violations raise ``RuntimeError`` like the reference's ``TORCH_CHECK``.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from lowbit_comm_amd.hip.library import LBC_OK, LBC_UNSUPPORTED, last_error, load_library

DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
DTYPE_NAMES = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}
TORCH_DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
REDUCE_OPS = {"none": 0, "sum": 1, "max": 2, "min": 3}
MAX_PAYLOADS = 8
_NONE = -1
ACCESS_MODES = {"auto": 0, "cached": 1, "stream": 2}
_default_access = "auto"


def access_code(access: str | None) -> int:
    """ABI code of an access mode; ``None`` means the module default (see :func:`access_mode`)."""
    name = _default_access if access is None else access
    if name not in ACCESS_MODES:
        raise RuntimeError(f"access must be one of {sorted(ACCESS_MODES)}; got {access!r}")
    return ACCESS_MODES[name]


class access_mode:
    """``with access_mode("cached"):`` - launches *bound* inside the block without an explicit ``access=`` use
    that mode ("auto": the library's rule, "cached": plain cached accesses for operands that are still in cache,
    "stream": non-temporal loads).  The mode is fixed when a launch is bound; replaying a :class:`BoundLaunch`
    later does not consult this default again.  Results never depend on the mode."""

    def __init__(self, mode: str) -> None:
        if mode not in ACCESS_MODES:
            raise RuntimeError(f"access must be one of {sorted(ACCESS_MODES)}; got {mode!r}")
        self._mode = mode
        self._previous = None

    def __enter__(self):
        global _default_access
        self._previous, _default_access = _default_access, self._mode
        return self

    def __exit__(self, *exc):
        global _default_access
        _default_access = self._previous
        return False


def num_groups(numel: int, group_size: int) -> int:
    return -(-numel // group_size) if numel else 0


def payload_nbytes(numel: int, group_size: int = 64) -> int:
    """Bytes of one packed payload ``[int8 codes || fp32 scales]``."""
    return num_groups(numel, group_size) * (group_size + 4)


def split_payload(payload: torch.Tensor, numel: int, group_size: int = 64):
    """Zero-copy ``(codes int8[G*g], scales float32[G])`` views of a packed uint8 payload."""
    groups = num_groups(numel, group_size)
    code_bytes = groups * group_size
    if payload.dtype != torch.uint8 or payload.dim() != 1 or payload.numel() != code_bytes + 4 * groups:
        raise RuntimeError(
            f"payload must be a flat uint8 tensor of {code_bytes + 4 * groups} bytes; got "
            f"{payload.dtype} with {payload.numel()} elements")
    return payload[:code_bytes].view(torch.int8), payload[code_bytes:].view(torch.float32)


def payload_addresses(payload: torch.Tensor, numel: int, group_size: int = 64, *, name: str = "payload",
                      device: torch.device | None = None) -> tuple[int, int]:
    """Device addresses ``(codes, scales)`` inside a packed uint8 payload, without creating tensor views (a view
    costs a few microseconds of host time; the hot callers hand over up to nine payloads per bucket)."""
    groups = num_groups(numel, group_size)
    code_bytes = groups * group_size
    # one combined test on the hot path; the separate tests below only run to name what is wrong
    if (isinstance(payload, torch.Tensor) and payload.dtype is torch.uint8 and payload.is_cuda
            and payload.numel() == code_bytes + 4 * groups and payload.is_contiguous()
            and (device is None or payload.device == device)):
        base = payload.data_ptr()
        return base, base + code_bytes
    if not isinstance(payload, torch.Tensor) or payload.dtype != torch.uint8:
        raise RuntimeError(f"{name} must be uint8")
    if not payload.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor")
    if not payload.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if device is not None and payload.device != device:
        raise RuntimeError(f"{name} must be on {device}")
    raise RuntimeError(f"{name} has an invalid quantized payload size")


def promote(a: torch.dtype, b: torch.dtype) -> torch.dtype:
    return a if a == b else torch.float32


def true_divide_(tensor: torch.Tensor, divisor: float) -> torch.Tensor:
    """In-place IEEE division by a scalar.  ``tensor.div_(python_number)`` on a GPU tensor multiplies by
    the reciprocal, which differs from the CPU codec's true division in the last bit for divisors that
    are not powers of two; dividing by a 0-dim device tensor takes the exact path."""
    if tensor.is_cuda:
        return tensor.div_(torch.full((), float(divisor), dtype=torch.float32, device=tensor.device))
    return tensor.div_(divisor)


# --------------------------------------------------------------------------- #
def _require(cond: bool, message: str) -> None:
    if not cond:
        raise RuntimeError(message)


def _device_tensor(t: torch.Tensor, name: str, device: torch.device | None = None) -> None:
    _require(isinstance(t, torch.Tensor), f"{name} must be a tensor")
    _require(t.is_cuda, f"{name} must be a GPU tensor")
    _require(t.is_contiguous(), f"{name} must be contiguous")
    if device is not None:
        _require(t.device == device, f"{name} must be on {device}")


def _float_tensor(t: torch.Tensor, name: str, device: torch.device | None = None) -> int:
    _device_tensor(t, name, device)
    _require(t.dtype in DTYPE_CODES, f"{name} must be fp16, bf16 or fp32; got {t.dtype}")
    return DTYPE_CODES[t.dtype]


def _ptr(t: torch.Tensor | None):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream_of = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_handle(device: torch.device) -> int:
    """Raw ``hipStream_t`` of torch's current stream on ``device`` (the direct binding when this torch has it: it
    skips building a ``torch.cuda.Stream`` object, a few microseconds per launch)."""
    if _raw_stream_of is not None:
        return _raw_stream_of(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _Launch:
    """Device guard + current stream of ``device`` for one ABI call."""

    def __init__(self, device: torch.device) -> None:
        self._guard = None if device.index in (None, torch.cuda.current_device()) else torch.cuda.device(device)
        self.device = device

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()
        return ctypes.c_void_p(current_stream_handle(self.device))

    def __exit__(self, *exc):
        if self._guard is not None:
            self._guard.__exit__(*exc)
        return False


class BoundLaunch:
    """One ABI call with every argument validated and marshalled ahead of time.

    Calling it enqueues the kernel on torch's current stream of the tensors' device and returns
    ``True``/``False`` like the ``*_into`` function it was made from.  The bound tensors are kept
    alive by the object; their addresses must not change (no resize, no reallocation).  This is
    the per-bucket fast path: a DDP hook binds once per bucket shape and replays every step.
    """

    __slots__ = ("_fn", "_args", "_device", "_lib", "_keep", "_kind", "_hold")

    def __init__(self, fn, args: tuple, device: torch.device, lib, keep: tuple, kind: str | None = None,
                 hold: tuple = ()) -> None:
        self._fn = fn
        self._args = args
        self._device = device
        self._lib = lib
        self._keep = keep
        self._kind = kind      # which entry point the arguments belong to, for launches that can share a grid
        self._hold = hold      # host memory the arguments point into (argument structures, pointer arrays)

    def forget_tensors(self) -> "BoundLaunch":
        """Stop keeping the bound tensors alive.  For a cache keyed by everything the binding depends on (addresses,
        dtypes, element counts) whose user passes the live tensors at every call anyway: the launch stays valid for
        any tensor that matches the key, and the cache pins no memory."""
        self._keep = ()
        return self

    def __call__(self, stream: int | None = None) -> bool:
        """Enqueue.  ``stream``: raw ``hipStream_t`` handle (``torch.cuda.Stream.cuda_stream``) of a stream on
        the tensors' device, which must be the current device; ``None`` looks up torch's current stream."""
        if stream is None:
            if self._device.index not in (None, torch.cuda.current_device()):
                with _Launch(self._device) as guarded:
                    return _finish(self._fn(*self._args, guarded), self._lib)
            stream = current_stream_handle(self._device)
        rc = self._fn(*self._args, stream)
        return True if rc == LBC_OK else _finish(rc, self._lib)


def _finish(rc: int, lib) -> bool:
    if rc == LBC_OK:
        return True
    if rc == LBC_UNSUPPORTED:
        return False
    raise RuntimeError(last_error(lib) or f"lbc call failed with code {rc}")


def _side_tensors(x: torch.Tensor, residual, new_residual, restored, restored_dtype, prepared_out=None):
    """Validate the optional error-feedback tensors of a quantize call; returns their dtype codes."""
    device, n = x.device, x.numel()
    r_code = _NONE
    if residual is not None:
        r_code = _float_tensor(residual, "residual", device)
        _require(residual.numel() == n, "input and residual must have the same number of elements")
    p_dtype = x.dtype if residual is None else promote(x.dtype, residual.dtype)
    d_dtype = restored.dtype if restored is not None else (restored_dtype or torch.float32)
    d_code = DTYPE_CODES.get(d_dtype)
    _require(d_code is not None, f"restored dtype must be fp16, bf16 or fp32; got {d_dtype}")
    n_code = _NONE
    if restored is not None:
        _float_tensor(restored, "restored", device)
        _require(restored.numel() >= n, "restored must have at least input.numel() elements")
    if new_residual is not None:
        n_code = _float_tensor(new_residual, "new_residual", device)
        _require(new_residual.numel() == n, "input and new_residual must have the same number of elements")
        _require(new_residual.dtype == promote(p_dtype, d_dtype),
                 f"new_residual must have dtype {promote(p_dtype, d_dtype)}")
    p_code = _NONE
    if prepared_out is not None:
        p_code = _float_tensor(prepared_out, "prepared_out", device)
        _require(prepared_out.numel() >= n, "prepared_out must have at least input.numel() elements")
        _require(prepared_out.dtype == p_dtype, f"prepared_out must have dtype {p_dtype}")
    return r_code, n_code, d_code, p_code



# --------------------------------------------------------------------------- #
# quantize + pack
# --------------------------------------------------------------------------- #
def quant_pack_into(x: torch.Tensor, codes: torch.Tensor, scales: torch.Tensor, *, group_size: int = 64,
                    residual: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                    restored: torch.Tensor | None = None, restored_dtype: torch.dtype | None = None,
                    prepared_out: torch.Tensor | None = None, access: str | None = None) -> bool:
    """``codes, scales <- quant(p)``, ``p = x + residual``; optionally ``restored``, ``new_residual = p - restored``
    and ``prepared_out = p``."""
    return bind_quant_pack(x, codes, scales, group_size=group_size, residual=residual, new_residual=new_residual,
                           restored=restored, restored_dtype=restored_dtype, prepared_out=prepared_out, access=access)()


def bind_quant_pack(x: torch.Tensor, codes: torch.Tensor, scales: torch.Tensor, *, group_size: int = 64,
                    residual: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                    restored: torch.Tensor | None = None, restored_dtype: torch.dtype | None = None,
                    prepared_out: torch.Tensor | None = None, access: str | None = None) -> BoundLaunch:
    """Validate once; the returned :class:`BoundLaunch` replays :func:`quant_pack_into` on the same tensors."""
    lib = load_library()
    x_code = _float_tensor(x, "input")
    device = x.device
    n = x.numel()
    groups = num_groups(n, group_size)
    _device_tensor(codes, "codes", device)
    _device_tensor(scales, "scales", device)
    _require(codes.dtype in (torch.int8, torch.uint8), "codes must have int8 or uint8 dtype")
    _require(scales.dtype == torch.float32, "scales must have float32 dtype")
    _require(codes.numel() == groups * group_size, "codes has an invalid quantized payload size")
    _require(scales.numel() == groups, "scales has an invalid group count")
    r_code, n_code, d_code, p_code = _side_tensors(x, residual, new_residual, restored, restored_dtype, prepared_out)
    args = (_ptr(x), x_code, _ptr(residual), r_code, n, group_size, _ptr(codes), _ptr(scales),
            _ptr(new_residual), n_code, _ptr(restored), d_code, _ptr(prepared_out), p_code)
    return BoundLaunch(lib.lbc_quant_pack, args + (access_code(access),), device, lib,
                       (x, codes, scales, residual, new_residual, restored, prepared_out))


def bind_quant_pack_payload(x: torch.Tensor, payload: torch.Tensor, *, group_size: int = 64,
                            residual: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                            restored: torch.Tensor | None = None,
                            restored_dtype: torch.dtype | None = None, prepared_out: torch.Tensor | None = None,
                            access: str | None = None) -> BoundLaunch:
    """:func:`bind_quant_pack` writing the packed ``uint8[codes || scales]`` wire layout into ``payload``."""
    lib = load_library()
    x_code = _float_tensor(x, "input")
    codes_at, scales_at = payload_addresses(payload, x.numel(), group_size, name="output", device=x.device)
    r_code, n_code, d_code, p_code = _side_tensors(x, residual, new_residual, restored, restored_dtype, prepared_out)
    args = (_ptr(x), x_code, _ptr(residual), r_code, x.numel(), group_size, ctypes.c_void_p(codes_at),
            ctypes.c_void_p(scales_at), _ptr(new_residual), n_code, _ptr(restored), d_code, _ptr(prepared_out), p_code)
    return BoundLaunch(lib.lbc_quant_pack, args + (access_code(access),), x.device, lib,
                       (x, payload, residual, new_residual, restored, prepared_out))


def quant_pack_payload_into(x: torch.Tensor, payload: torch.Tensor, *, group_size: int = 64, **kwargs) -> bool:
    """Same as :func:`quant_pack_into`, writing the packed ``uint8[codes || scales]`` wire layout."""
    return bind_quant_pack_payload(x, payload, group_size=group_size, **kwargs)()


def quant_pack(x: torch.Tensor, *, group_size: int = 64, residual: torch.Tensor | None = None):
    """Allocating convenience wrapper: returns ``(codes int8[G*g], scales float32[G])``."""
    groups = num_groups(x.numel(), group_size)
    codes = torch.empty(groups * group_size, dtype=torch.int8, device=x.device)
    scales = torch.empty(groups, dtype=torch.float32, device=x.device)
    if not quant_pack_into(x.contiguous().reshape(-1), codes, scales, group_size=group_size, residual=residual):
        raise RuntimeError(f"quant_pack has no kernel for dtype {x.dtype} / group_size {group_size}")
    return codes, scales


def quant_pack_chunks_into(x: torch.Tensor, payloads: torch.Tensor, world: int, *, group_size: int = 64,
                           residual: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                           restored: torch.Tensor | None = None, restored_dtype: torch.dtype | None = None,
                           prepared_out: torch.Tensor | None = None, access: str | None = None) -> bool:
    """Quantize the ``world`` destination chunks of ``x`` (+ ``residual``) into the rows of ``payloads``
    (uint8 ``[world, stride]``) in one launch; optional fused error-feedback outputs as in
    :func:`quant_pack_into`."""
    return bind_quant_pack_chunks(x, payloads, world, group_size=group_size, residual=residual,
                                  new_residual=new_residual, restored=restored, restored_dtype=restored_dtype,
                                  prepared_out=prepared_out, access=access)()


def bind_quant_pack_chunks(x: torch.Tensor, payloads: torch.Tensor, world: int, *, group_size: int = 64,
                           residual: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                           restored: torch.Tensor | None = None,
                           restored_dtype: torch.dtype | None = None, prepared_out: torch.Tensor | None = None,
                           access: str | None = None) -> BoundLaunch:
    lib = load_library()
    x_code = _float_tensor(x, "input")
    device = x.device
    n = x.numel()
    _device_tensor(payloads, "payloads", device)
    _require(payloads.dtype == torch.uint8 and payloads.dim() == 2, "payloads must be a 2-D uint8 tensor")
    _require(payloads.shape[0] == world, "payloads must have one row per destination rank")
    shard = -(-n // world)
    _require(payloads.shape[1] >= payload_nbytes(shard, group_size), "payload rows are too small")
    r_code, n_code, d_code, p_code = _side_tensors(x, residual, new_residual, restored, restored_dtype, prepared_out)
    args = (_ptr(x), x_code, _ptr(residual), r_code, n, world, group_size, _ptr(payloads), payloads.stride(0),
            _ptr(new_residual), n_code, _ptr(restored), d_code, _ptr(prepared_out), p_code)
    return BoundLaunch(lib.lbc_quant_pack_chunks, args + (access_code(access),), device, lib,
                       (x, payloads, residual, new_residual, restored, prepared_out), kind="quant_pack_chunks")


# --------------------------------------------------------------------------- #
# decode
# --------------------------------------------------------------------------- #
def dequant_into(codes: torch.Tensor, scales: torch.Tensor, out: torch.Tensor, *, numel: int | None = None,
                 group_size: int = 64, reduce_op: str = "none", access: str | None = None) -> bool:
    """``out[:numel] (op)= float(code) * scale``."""
    return bind_dequant(codes, scales, out, numel=numel, group_size=group_size, reduce_op=reduce_op, access=access)()


def bind_dequant(codes: torch.Tensor, scales: torch.Tensor, out: torch.Tensor, *, numel: int | None = None,
                 group_size: int = 64, reduce_op: str = "none", access: str | None = None) -> BoundLaunch:
    lib = load_library()
    o_code = _float_tensor(out, "output")
    device = out.device
    n = out.numel() if numel is None else int(numel)
    _require(0 <= n <= out.numel(), "numel exceeds the output size")
    groups = num_groups(n, group_size)
    _device_tensor(codes, "codes", device)
    _device_tensor(scales, "scales", device)
    _require(codes.dtype in (torch.int8, torch.uint8), "codes must have int8 or uint8 dtype")
    _require(scales.dtype == torch.float32, "scales must have float32 dtype")
    _require(codes.numel() >= groups * group_size, "codes is smaller than the padded element count")
    _require(scales.numel() >= groups, "scales is smaller than the group count")
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    args = (_ptr(codes), _ptr(scales), n, group_size, _ptr(out), o_code, REDUCE_OPS[reduce_op])
    return BoundLaunch(lib.lbc_dequant, args + (access_code(access),), device, lib, (codes, scales, out))


def dequant_payload_into(payload: torch.Tensor, out: torch.Tensor, *, numel: int | None = None, group_size: int = 64,
                         reduce_op: str = "none", access: str | None = None) -> bool:
    """:func:`dequant_into` reading a packed ``uint8[codes || scales]`` payload that covers ``numel`` elements."""
    lib = load_library()
    o_code = _float_tensor(out, "output")
    n = out.numel() if numel is None else int(numel)
    _require(0 <= n <= out.numel(), "numel exceeds the output size")
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    codes_at, scales_at = payload_addresses(payload, n, group_size, name="input", device=out.device)
    args = (ctypes.c_void_p(codes_at), ctypes.c_void_p(scales_at), n, group_size, _ptr(out), o_code,
            REDUCE_OPS[reduce_op])
    return BoundLaunch(lib.lbc_dequant, args + (access_code(access),), out.device, lib, (payload, out))()


def dequant(codes: torch.Tensor, scales: torch.Tensor, numel: int, *, group_size: int = 64,
            dtype: torch.dtype = torch.float32) -> torch.Tensor:
    out = torch.empty(numel, dtype=dtype, device=codes.device)
    if not dequant_into(codes, scales, out, group_size=group_size):
        raise RuntimeError(f"dequant has no kernel for dtype {dtype} / group_size {group_size}")
    return out


def dequant_chunks_into(payloads: torch.Tensor, out: torch.Tensor, shard_numel: int, *, group_size: int = 64,
                        access: str | None = None) -> bool:
    """Decode row ``d`` of ``payloads`` into ``out[d*shard : (d+1)*shard]`` (clipped to ``out.numel()``)."""
    return bind_dequant_chunks(payloads, out, shard_numel, group_size=group_size, access=access)()


def bind_dequant_chunks(payloads: torch.Tensor, out: torch.Tensor, shard_numel: int, *, group_size: int = 64,
                        access: str | None = None) -> BoundLaunch:
    lib = load_library()
    o_code = _float_tensor(out, "output")
    _device_tensor(payloads, "payloads", out.device)
    _require(payloads.dtype == torch.uint8 and payloads.dim() == 2, "payloads must be a 2-D uint8 tensor")
    world = payloads.shape[0]
    _require(payloads.shape[1] >= payload_nbytes(shard_numel, group_size), "payload rows are too small")
    _require(out.numel() <= world * shard_numel, "output is larger than world * shard_numel")
    args = (_ptr(payloads), payloads.stride(0), world, shard_numel, out.numel(), group_size, _ptr(out), o_code)
    return BoundLaunch(lib.lbc_dequant_chunks, args + (access_code(access),), out.device, lib, (payloads, out),
                       kind="dequant_chunks")


def dequant_reduce_into(payloads: Sequence[tuple[torch.Tensor, torch.Tensor]], out: torch.Tensor, *,
                        numel: int | None = None, group_size: int = 64, divisor: float = 1.0,
                        prepared: torch.Tensor | None = None, new_residual: torch.Tensor | None = None,
                        access: str | None = None) -> bool:
    """``out[:numel] = (sum_r decode(payload_r)) / divisor`` in list order; optional ``new_residual = prepared - out``.

    ``payloads`` is a sequence of ``(codes, scales)`` pairs or of packed ``uint8[codes || scales]`` tensors covering
    exactly ``numel`` elements.  More than 8 payloads returns ``False``.
    """
    bound = bind_dequant_reduce(payloads, out, numel=numel, group_size=group_size, divisor=divisor,
                                prepared=prepared, new_residual=new_residual, access=access)
    return False if bound is None else bound()


def bind_dequant_reduce(payloads: Sequence[tuple[torch.Tensor, torch.Tensor]], out: torch.Tensor, *,
                        numel: int | None = None, group_size: int = 64, divisor: float = 1.0,
                        prepared: torch.Tensor | None = None,
                        new_residual: torch.Tensor | None = None, access: str | None = None) -> BoundLaunch | None:
    """Bound form of :func:`dequant_reduce_into`; ``None`` when there are more than 8 payloads."""
    lib = load_library()
    _require(len(payloads) > 0, "inputs must not be empty")
    _require(divisor > 0, "divisor must be > 0")
    o_code = _float_tensor(out, "output")
    device = out.device
    n = out.numel() if numel is None else int(numel)
    _require(0 <= n <= out.numel(), "numel exceeds the output size")
    if len(payloads) > MAX_PAYLOADS:
        return None
    groups = num_groups(n, group_size)
    world = len(payloads)
    code_ptrs = (ctypes.c_void_p * world)()
    scale_ptrs = (ctypes.c_void_p * world)()
    for r, entry in enumerate(payloads):
        if isinstance(entry, torch.Tensor):          # a packed uint8[codes || scales] payload
            try:
                code_ptrs[r], scale_ptrs[r] = payload_addresses(entry, n, group_size, name="inputs", device=device)
            except RuntimeError as error:            # name the entry only when something is wrong with it
                raise RuntimeError(str(error).replace("inputs", f"inputs[{r}]", 1)) from None
            continue
        codes, scales = entry
        _device_tensor(codes, f"codes[{r}]", device)
        _device_tensor(scales, f"scales[{r}]", device)
        _require(codes.dtype in (torch.int8, torch.uint8), f"codes[{r}] must have int8 or uint8 dtype")
        _require(scales.dtype == torch.float32, f"scales[{r}] must have float32 dtype")
        _require(codes.numel() >= groups * group_size, f"codes[{r}] is smaller than the padded element count")
        _require(scales.numel() >= groups, f"scales[{r}] is smaller than the group count")
        code_ptrs[r] = codes.data_ptr()
        scale_ptrs[r] = scales.data_ptr()
    _require((prepared is None) == (new_residual is None), "prepared and new_residual must be given together")
    if prepared is not None:
        _float_tensor(prepared, "prepared", device)
        _float_tensor(new_residual, "residual", device)
        _require(prepared.dtype == out.dtype, "prepared and restored must have the same dtype")
        _require(new_residual.dtype == out.dtype, "prepared and residual must have the same dtype")
        _require(prepared.numel() == n, "prepared must have numel elements")
        _require(new_residual.numel() == n, "prepared and residual must have the same number of elements")
    args = (code_ptrs, scale_ptrs, world, n, group_size, float(divisor), _ptr(out), o_code,
            _ptr(prepared), _ptr(new_residual))
    keep = (tuple(payloads), out, prepared, new_residual)
    return BoundLaunch(lib.lbc_dequant_reduce, args + (access_code(access),), device, lib, keep, kind="dequant_reduce")


def bind_quant_chunks_and_reduce(quant: BoundLaunch, reduce: BoundLaunch) -> BoundLaunch:
    """One launch for the chunked quantize of one bucket and the fused reduce of the payloads that arrived for another
    bucket's shard (``lbc_quant_pack_chunks_and_dequant_reduce``).  ``quant`` comes from :func:`bind_quant_pack_chunks`
    (without ``restored``), ``reduce`` from :func:`bind_dequant_reduce`; the two must not touch the same memory, and
    the access mode is the quantize's.  Calling the result returns ``False`` when the combination has no shared grid
    (then call ``quant`` and ``reduce`` themselves); the results are bit-identical either way."""
    _require(isinstance(quant, BoundLaunch) and quant._kind == "quant_pack_chunks",
             "quant must come from bind_quant_pack_chunks")
    _require(isinstance(reduce, BoundLaunch) and reduce._kind == "dequant_reduce",
             "reduce must come from bind_dequant_reduce")
    _require(quant._device == reduce._device, "both launches must be on the same device")
    (x, x_code, residual, r_code, n, world, group_size, payloads, stride, new_residual, n_code, restored, _d_code,
     prepared_out, _p_code, access) = quant._args
    _require(restored is None and prepared_out is None, "the shared launch does not write `restored` or `prepared_out`")
    code_ptrs, scale_ptrs, r_world, r_n, r_group, divisor, out, o_code, prepared, r_new_residual, _r_access = reduce._args
    _require(group_size == r_group, "both launches must use the same group size")
    args = (x, x_code, residual, r_code, n, world, group_size, payloads, stride, new_residual, n_code,
            code_ptrs, scale_ptrs, r_world, r_n, divisor, out, o_code, prepared, r_new_residual, access)
    return BoundLaunch(quant._lib.lbc_quant_pack_chunks_and_dequant_reduce, args, quant._device, quant._lib,
                       (quant._keep, reduce._keep), kind="bucket_step")


def bind_dequant_reduce_quant(payloads: Sequence[tuple[torch.Tensor, torch.Tensor]], out_codes: torch.Tensor,
                              out_scales: torch.Tensor, numel: int, *, group_size: int = 64, divisor: float = 1.0,
                              mid_dtype: torch.dtype = torch.float32,
                              access: str | None = None) -> BoundLaunch | None:
    """Bound form of :func:`dequant_reduce_quant_into`; ``None`` when there are more than 8 payloads."""
    lib = load_library()
    _require(len(payloads) > 0, "inputs must not be empty")
    _require(divisor > 0, "divisor must be > 0")
    _require(mid_dtype in DTYPE_CODES, f"intermediate dtype must be fp16, bf16 or fp32; got {mid_dtype}")
    _device_tensor(out_codes, "out_codes")
    device = out_codes.device
    _device_tensor(out_scales, "out_scales", device)
    n = int(numel)
    groups = num_groups(n, group_size)
    _require(out_codes.dtype in (torch.int8, torch.uint8), "out_codes must have int8 or uint8 dtype")
    _require(out_scales.dtype == torch.float32, "out_scales must have float32 dtype")
    _require(out_codes.numel() >= groups * group_size, "out_codes is smaller than the padded element count")
    _require(out_scales.numel() >= groups, "out_scales is smaller than the group count")
    if len(payloads) > MAX_PAYLOADS:
        return None
    world = len(payloads)
    code_ptrs = (ctypes.c_void_p * world)()
    scale_ptrs = (ctypes.c_void_p * world)()
    for r, (codes, scales) in enumerate(payloads):
        _device_tensor(codes, f"codes[{r}]", device)
        _device_tensor(scales, f"scales[{r}]", device)
        _require(codes.dtype in (torch.int8, torch.uint8), f"codes[{r}] must have int8 or uint8 dtype")
        _require(scales.dtype == torch.float32, f"scales[{r}] must have float32 dtype")
        _require(codes.numel() >= groups * group_size, f"codes[{r}] is smaller than the padded element count")
        _require(scales.numel() >= groups, f"scales[{r}] is smaller than the group count")
        code_ptrs[r] = codes.data_ptr()
        scale_ptrs[r] = scales.data_ptr()
    args = (code_ptrs, scale_ptrs, world, n, group_size, float(divisor), DTYPE_CODES[mid_dtype], _ptr(out_codes),
            _ptr(out_scales))
    return BoundLaunch(lib.lbc_dequant_reduce_quant, args + (access_code(access),), device, lib,
                       (tuple(payloads), out_codes, out_scales), kind="dequant_reduce_quant")


def bind_bucket_pipeline_step(quant: BoundLaunch | None = None, reduce: BoundLaunch | None = None,
                              decode: BoundLaunch | None = None) -> BoundLaunch:
    """One launch for up to three stages of a bucket stream (``lbc_bucket_pipeline_step``): ``quant`` from
    :func:`bind_quant_pack_chunks` (bucket k, without ``restored`` / ``prepared_out``), ``reduce`` from
    :func:`bind_dequant_reduce_quant` (bucket k-1) and ``decode`` from :func:`bind_dequant_chunks` (bucket k-2); any
    may be ``None``.  The stages must not touch each other's outputs.  The access mode is that of the first stage
    given.  Calling the result returns ``False`` when the combination has no shared grid (then call the stages
    themselves); the results are bit-identical either way."""
    from lowbit_comm_amd.hip.library import DequantChunksStage, QuantChunksStage, ReduceQuantStage

    given = [stage for stage in (quant, reduce, decode) if stage is not None]
    _require(len(given) > 0, "at least one stage must be given")
    for stage, kind, maker in ((quant, "quant_pack_chunks", "bind_quant_pack_chunks"),
                               (reduce, "dequant_reduce_quant", "bind_dequant_reduce_quant"),
                               (decode, "dequant_chunks", "bind_dequant_chunks")):
        _require(stage is None or (isinstance(stage, BoundLaunch) and stage._kind == kind),
                 f"the {kind} stage must come from {maker}")
    _require(all(stage._device == given[0]._device for stage in given), "all stages must be on the same device")
    value = lambda p: None if p is None else (p.value if isinstance(p, ctypes.c_void_p) else p)  # noqa: E731
    hold: list = []
    group_size = None
    q_ref = r_ref = d_ref = None
    if quant is not None:
        (x, x_code, residual, r_code, n, world, group_size, payloads, stride, new_residual, n_code, restored, _d_code,
         prepared_out, _p_code, _access) = quant._args
        _require(restored is None and prepared_out is None,
                 "the shared launch does not write `restored` or `prepared_out`")
        q_stage = QuantChunksStage(value(x), value(residual), value(payloads), value(new_residual), n, stride,
                                   x_code, r_code, n_code, world)
        hold.append(q_stage)
        q_ref = ctypes.c_void_p(ctypes.addressof(q_stage))
    if reduce is not None:
        code_ptrs, scale_ptrs, r_world, r_n, r_group, divisor, mid_code, out_codes, out_scales, _r_access = reduce._args
        _require(group_size in (None, r_group), "all stages must use the same group size")
        group_size = r_group
        r_stage = ReduceQuantStage(ctypes.addressof(code_ptrs), ctypes.addressof(scale_ptrs), value(out_codes),
                                   value(out_scales), r_n, divisor, r_world, mid_code)
        hold.extend((r_stage, code_ptrs, scale_ptrs))
        r_ref = ctypes.c_void_p(ctypes.addressof(r_stage))
    if decode is not None:
        d_payloads, d_stride, d_world, d_shard, d_total, d_group, d_out, o_code, _d_access = decode._args
        _require(group_size in (None, d_group), "all stages must use the same group size")
        group_size = d_group
        d_stage = DequantChunksStage(value(d_payloads), value(d_out), d_stride, d_shard, d_total, d_world, o_code)
        hold.append(d_stage)
        d_ref = ctypes.c_void_p(ctypes.addressof(d_stage))
    lib = given[0]._lib
    args = (q_ref, r_ref, d_ref, group_size, given[0]._args[-1])
    return BoundLaunch(lib.lbc_bucket_pipeline_step, args, given[0]._device, lib, tuple(stage._keep for stage in given),
                       kind="bucket_pipeline_step", hold=tuple(hold))


def dequant_reduce_quant_into(payloads: Sequence[tuple[torch.Tensor, torch.Tensor]], out_codes: torch.Tensor,
                              out_scales: torch.Tensor, numel: int, **kwargs) -> bool:
    """``(out_codes, out_scales) = quantize((sum_r decode(payload_r)) / divisor)`` in one launch, the reduce carried
    out in ``mid_dtype`` exactly as :func:`dequant_reduce_into` would for an output of that dtype."""
    bound = bind_dequant_reduce_quant(payloads, out_codes, out_scales, numel, **kwargs)
    return False if bound is None else bound()


# --------------------------------------------------------------------------- #
# ring step: chunk (op)= decode(received) [/ divisor], then quantize+pack of the updated chunk
# --------------------------------------------------------------------------- #
def bind_ring_step(received: torch.Tensor, chunk: torch.Tensor, send: torch.Tensor | None = None, *,
                   group_size: int = 64, reduce_op: str = "sum", divisor: float = 1.0,
                   access: str | None = None) -> BoundLaunch:
    """``received`` and ``send`` are packed ``uint8[codes || scales]`` payloads covering ``chunk.numel()``
    elements; ``chunk`` is updated in place and, when ``send`` is given, quantized into it in the same launch."""
    lib = load_library()
    code = _float_tensor(chunk, "chunk")
    device = chunk.device
    n = chunk.numel()
    _require(reduce_op in REDUCE_OPS, f"unsupported reduce op {reduce_op!r}")
    _require(float(divisor) > 0.0, "divisor must be > 0")
    recv_codes, recv_scales = payload_addresses(received, n, group_size, name="received payload", device=device)
    send_codes = send_scales = None
    if send is not None:
        send_codes, send_scales = payload_addresses(send, n, group_size, name="send payload", device=device)
        _require(n == 0 or send.data_ptr() != received.data_ptr(), "the payload to send must not alias the received one")
    args = (ctypes.c_void_p(recv_codes), ctypes.c_void_p(recv_scales), _ptr(chunk), code, n, group_size,
            REDUCE_OPS[reduce_op], float(divisor),
            None if send is None else ctypes.c_void_p(send_codes), None if send is None else ctypes.c_void_p(send_scales))
    return BoundLaunch(lib.lbc_ring_step, args + (access_code(access),), device, lib, (received, chunk, send))


def ring_step_into(received: torch.Tensor, chunk: torch.Tensor, send: torch.Tensor | None = None, *,
                   group_size: int = 64, reduce_op: str = "sum", divisor: float = 1.0,
                   access: str | None = None) -> bool:
    return bind_ring_step(received, chunk, send, group_size=group_size, reduce_op=reduce_op, divisor=divisor,
    access=access)()


def ef_update_into(prepared: torch.Tensor, restored: torch.Tensor, residual: torch.Tensor, *,
                   access: str | None = None) -> bool:
    """``residual = prepared - restored`` (fp32 subtraction, rounded to the residual's dtype)."""
    lib = load_library()
    p_code = _float_tensor(prepared, "prepared")
    t_code = _float_tensor(restored, "restored", prepared.device)
    r_code = _float_tensor(residual, "residual", prepared.device)
    _require(prepared.numel() == restored.numel(), "prepared and restored must have the same number of elements")
    _require(prepared.numel() == residual.numel(), "prepared and residual must have the same number of elements")
    args = (_ptr(prepared), p_code, _ptr(restored), t_code, _ptr(residual), r_code, prepared.numel())
    return BoundLaunch(lib.lbc_ef_update, args + (access_code(access),), prepared.device, lib,
                       (prepared, restored, residual))()
