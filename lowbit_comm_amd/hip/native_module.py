"""The duck-typed native module the codec facade talks to.

It exposes the names and positional argument orders of the reference's pybind module
(``ccdl_comm/csrc/pybind.cpp:133-166``; orders from ``ccdl_comm/csrc/quantization/quant_api.cuh:5-17``
and ``dequant_api.cuh:5-12``) over this package's C ABI.  Buffers are flat ``uint8`` tensors holding
the portable wire format ``[int8 codes || fp32 scales]`` (68 bytes per group of 64 for every source
dtype; size them with ``estimate_payload_size``).

Conventions kept from the reference: ``inplace_*`` never allocate and never touch their inputs;
unsupported *policy* (4-bit, top-k, stochastic, non-linear, more than 8 payloads for the fused calls)
returns ``False`` so the caller can fall back; contract violations raise ``RuntimeError``; launches go
to torch's current stream of the tensors' device and do not synchronise.  ``compact`` is accepted
and ignored: the portable format has a single layout.
"""
from __future__ import annotations

import enum
import operator
import threading
from collections import OrderedDict
from typing import Sequence

import torch

from lowbit_comm_amd.hip import ops
from lowbit_comm_amd.hip.library import load_library


class QuantType(enum.IntEnum):
    Linear = 0
    Normal = 1
    Uniform = 2
    E3M0 = 3
    E2M1 = 4


class DType(enum.IntEnum):
    FP16 = 1
    BF16 = 2
    FP32 = 0


class ReduceOP(enum.IntEnum):
    NONE = 0
    SUM = 1
    MAX = 2
    MIN = 3


_IS_CUDA = operator.attrgetter("is_cuda")
_DTYPE = operator.attrgetter("dtype")
_TORCH_OF = {DType.FP16: torch.float16, DType.BF16: torch.bfloat16, DType.FP32: torch.float32}
_OP_NAME = {ReduceOP.NONE: "none", ReduceOP.SUM: "sum", ReduceOP.MAX: "max", ReduceOP.MIN: "min"}


def _policy_supported(group_size: int, topk: int, stochastic: bool, bit: int, quant_type) -> bool:
    return (group_size in (16, 32, 64) and topk == 0 and not stochastic and bit == 8
            and int(quant_type) == int(QuantType.Linear))


def _require_policy(group_size, topk, stochastic, bit, quant_type) -> None:
    if not _policy_supported(group_size, topk, stochastic, bit, quant_type):
        raise RuntimeError(
            "the HIP codec supports linear 8-bit quantization with group_size 16/32/64, topk=0, no stochastic "
            f"rounding; got group_size={group_size} topk={topk} stochastic={stochastic} bit={bit} "
            f"quant_type={getattr(quant_type, 'name', quant_type)}")


def _check_payload(buffer: torch.Tensor, name: str) -> None:
    if not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.uint8:
        raise RuntimeError(f"{name} must be uint8")
    if not buffer.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor")
    if not buffer.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _padded_numel_of(buffer: torch.Tensor, group_size: int, name: str = "input") -> int:
    nbytes = buffer.numel()
    if nbytes % (group_size + 4) != 0:
        raise RuntimeError(f"{name} has an invalid quantized payload size")
    return nbytes // (group_size + 4) * group_size


def _views(buffer: torch.Tensor, group_size: int):
    padded = _padded_numel_of(buffer, group_size)
    flat = buffer.reshape(-1)
    return flat[:padded].view(torch.int8), flat[padded:].view(torch.float32)


class HipNativeModule:
    """Instance with the reference extension's symbols; constructing it loads (and type-checks) the library."""

    QuantType = QuantType
    DType = DType
    ReduceOP = ReduceOP
    NATIVE_WIRE_FORMAT = "portable"

    def __init__(self) -> None:
        self._lib = load_library()
        # Launches of the allocation-free entry points, bound to the addresses they were last called with.  A DDP
        # hook presents the same bucket, payload and workspace addresses every step, so from the second step on a
        # call is one key lookup and one ABI call.  The key holds everything a binding depends on (addresses,
        # dtypes, element counts, policy), the entries do not keep the tensors alive, least recently used go first.
        self._launches: OrderedDict = OrderedDict()
        # DistributedDataParallel calls its hook from the autograd thread while the training script may call the
        # codec from its own (the reference guards its pool and caches the same way, ccdl_comm/cuda/workspace.py:294).
        self._launches_lock = threading.Lock()
        self.launch_memo_entries = self.LAUNCH_MEMO_ENTRIES

    # One pass over a model's buckets must fit: an 8 B-parameter model in 25 MiB buckets has 613 of them, each with
    # a quantize and a reduce.  A smaller cache, walked cyclically, would miss on every call.  An entry is a few
    # hundred bytes of host memory; ``launch_memo_entries`` can be raised per instance.
    LAUNCH_MEMO_ENTRIES = 4096

    def _recall(self, key: tuple | None):
        """The launch remembered under ``key`` for the access mode in force, or ``None``."""
        if key is None:
            return None
        key = key + (ops.access_code(None),)
        with self._launches_lock:
            bound = self._launches.get(key)
            if bound is not None:
                self._launches.move_to_end(key)
        return bound

    def _memoized(self, key: tuple, bind):
        """The launch remembered under ``key``, else ``bind()`` (which validates and may raise; nothing is then
        stored).  ``bind`` may return ``None`` for a call that has no single launch.  The key is completed with the
        access mode in force: a launch bound under one mode is not replayed for a call made under another."""
        bound = self._recall(key)
        if bound is not None:
            return bound
        key = key + (ops.access_code(None),)
        launches = self._launches
        bound = bind()                       # validates tensors and marshals arguments: outside the lock
        if bound is not None:
            with self._launches_lock:
                bound = launches.setdefault(key, bound.forget_tensors())
                launches.move_to_end(key)
                while len(launches) > self.launch_memo_entries:
                    launches.popitem(last=False)
        return bound

    @staticmethod
    def _spec(tensor):
        """What a binding depends on, for a contiguous GPU tensor; ``None`` for anything else (the caller then takes
        the validating path, which names what is wrong)."""
        if tensor is None:
            return ()
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or not tensor.is_contiguous():
            return None
        return (tensor.data_ptr(), tensor.dtype, tensor.numel())

    def _reduce_key(self, tag, inputs, tensors, policy):
        """Memo key of a fused reduce: payload addresses and sizes, the other tensors' specs, the policy."""
        if not isinstance(inputs, (list, tuple)) or not 1 <= len(inputs) <= ops.MAX_PAYLOADS:
            return None
        specs = []
        for tensor in tensors:
            spec = self._spec(tensor)
            if spec is None:
                return None
            specs.append(spec)
        try:        # loops that stay in C: this runs for every bucket
            if not (all(map(_IS_CUDA, inputs)) and all(map(torch.Tensor.is_contiguous, inputs))):
                return None
            return (tag, tuple(map(torch.Tensor.data_ptr, inputs)), tuple(map(torch.Tensor.numel, inputs)),
                    tuple(map(_DTYPE, inputs)), tuple(specs), policy)
        except (TypeError, AttributeError):      # something in the list is not a tensor
            return None

    # ---- quantize ------------------------------------------------------------------------------
    def quantize(self, input, group_size, topk, stochastic, bit, quant_type, compact):
        _require_policy(group_size, topk, stochastic, bit, quant_type)
        output = torch.empty(ops.payload_nbytes(input.numel(), group_size), dtype=torch.uint8, device=input.device)
        self.inplace_quantize(input, output, group_size, topk, stochastic, bit, quant_type, compact)
        return output

    def inplace_quantize(self, input, output, group_size, topk, stochastic, bit, quant_type, compact) -> None:
        _require_policy(group_size, topk, stochastic, bit, quant_type)
        if not self.inplace_quantize_pack(input, output, None, group_size, topk, stochastic, bit, quant_type, compact):
            raise RuntimeError(f"no HIP quantize kernel for input dtype {input.dtype}")

    # The fused quantize can also hand back ``input + residual`` (keyword ``prepared_out``); the codec facade looks
    # for this flag before it passes the keyword, which the reference's extension does not know.
    QUANTIZE_PACK_WRITES_PREPARED = True

    def inplace_quantize_pack(self, input, output, residual, group_size, topk, stochastic, bit, quant_type,
                              compact, *, prepared_out=None) -> bool:
        """Fused ``(input + residual) -> quantize -> pack`` into ``output``; ``False`` for unsupported policy.

        ``prepared_out`` (no counterpart in the reference's extension): a tensor of the promoted type of input and
        residual that receives ``input + residual`` from the same launch - what ``ErrorFeedbackState.compensate``
        would have computed in a kernel of its own (ccdl_comm/quantization/error_feedback.py:27-36)."""
        if not _policy_supported(group_size, topk, stochastic, bit, quant_type):
            return False
        if not isinstance(input, torch.Tensor) or not input.is_cuda:
            raise RuntimeError("input must be a GPU tensor")
        if not input.is_contiguous():
            raise RuntimeError("input must be contiguous")
        if isinstance(output, torch.Tensor) and output.device != input.device:
            raise RuntimeError("input and output must be on the same device")
        if residual is not None and residual.numel() != input.numel():
            raise RuntimeError("input and residual must have the same number of elements")
        if input.numel() == 0:
            _check_payload(output, "output")
            if output.numel() != 0:
                raise RuntimeError("output has an invalid quantized payload size")
            return True
        # payload dtype / contiguity / size are checked where the addresses are taken
        bind = lambda: ops.bind_quant_pack_payload(input.reshape(-1), output, group_size=group_size,  # noqa: E731
                                                   residual=None if residual is None else residual.reshape(-1),
                                                   prepared_out=None if prepared_out is None else prepared_out.reshape(-1))
        out_spec, r_spec, p_spec = self._spec(output), self._spec(residual), self._spec(prepared_out)
        if out_spec is None or r_spec is None or p_spec is None:
            return bind()()
        key = ("quant_pack", input.data_ptr(), input.dtype, input.numel(), out_spec, r_spec, p_spec, group_size)
        return self._memoized(key, bind)()

    # ---- dequantize -----------------------------------------------------------------------------
    def dequantize(self, input, group_size, topk, bit, reduce_op, quant_type, dtype, compact):
        _require_policy(group_size, topk, False, bit, quant_type)
        _check_payload(input, "input")
        output = torch.empty(_padded_numel_of(input, group_size), dtype=_TORCH_OF[DType(int(dtype))],
                             device=input.device)
        if int(reduce_op) != int(ReduceOP.NONE):
            output.zero_()
        self.inplace_dequantize(input, output, group_size, topk, bit, reduce_op, quant_type, compact)
        return output

    def inplace_dequantize(self, input, output, group_size, topk, bit, reduce_op, quant_type, compact) -> None:
        _require_policy(group_size, topk, False, bit, quant_type)
        _check_payload(input, "input")
        padded = _padded_numel_of(input, group_size)
        flat = output.reshape(-1)
        if flat.numel() >= padded:        # the payload's own size decides; the usual workspace is padded
            done = ops.dequant_payload_into(input, flat, numel=padded, group_size=group_size,
                                            reduce_op=_OP_NAME[ReduceOP(int(reduce_op))])
        else:                             # a trimmed output: codes and scales sit at offsets the payload size fixes
            codes, scales = _views(input, group_size)
            done = ops.dequant_into(codes, scales, flat, numel=flat.numel(), group_size=group_size,
                                    reduce_op=_OP_NAME[ReduceOP(int(reduce_op))])
        if not done:
            raise RuntimeError(f"no HIP dequantize kernel for output dtype {output.dtype}")

    # ---- dequantize + reduce ------------------------------------------------------------------
    def _entries(self, inputs: Sequence[torch.Tensor], numel: int, group_size: int):
        """The payloads as the ops layer takes them: the packed tensors themselves when they cover exactly ``numel``
        elements' worth of groups (addresses are then computed without tensor views), (codes, scales) views when the
        caller decodes fewer groups than the payloads hold."""
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        for i, buffer in enumerate(inputs):
            _check_payload(buffer, f"inputs[{i}]" if i else "input")
        if all(buffer.numel() == ops.payload_nbytes(numel, group_size) for buffer in inputs):
            return [buffer.reshape(-1) for buffer in inputs]
        return [_views(buffer, group_size) for buffer in inputs]

    def dequantize_reduce(self, inputs, group_size, topk, bit, quant_type, dtype, compact):
        _require_policy(group_size, topk, False, bit, quant_type)
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        _check_payload(inputs[0], "input")
        output = torch.empty(_padded_numel_of(inputs[0], group_size), dtype=_TORCH_OF[DType(int(dtype))],
                             device=inputs[0].device)
        self.inplace_dequantize_reduce(inputs, output, group_size, topk, bit, quant_type, compact)
        return output

    def dequantize_reduce_mean(self, inputs, group_size, topk, bit, quant_type, dtype, compact, divisor):
        """``dequantize_reduce`` with the division by ``divisor`` in the same launch (no counterpart in the
        reference's module: its facade divides the sum afterwards, which costs a copy and a second pass; the bits
        are the same).  ``None`` when the fused launch does not apply: the caller then sums and divides."""
        _require_policy(group_size, topk, False, bit, quant_type)
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        _check_payload(inputs[0], "input")
        output = torch.empty(_padded_numel_of(inputs[0], group_size), dtype=_TORCH_OF[DType(int(dtype))],
                             device=inputs[0].device)
        if self.inplace_dequantize_reduce_mean(inputs, output, group_size, topk, bit, quant_type, compact, divisor):
            return output
        return None

    def inplace_dequantize_reduce(self, inputs, output, group_size, topk, bit, quant_type, compact) -> None:
        """Sum of all payloads into ``output`` in list order; any number of payloads (8 per fused launch)."""
        _require_policy(group_size, topk, False, bit, quant_type)
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        _check_payload(inputs[0], "input")
        flat = output.reshape(-1)
        numel = min(flat.numel(), _padded_numel_of(inputs[0], group_size))
        key = self._reduce_key("reduce", inputs, (flat,), (group_size, topk, bit, int(quant_type), numel))
        bound = self._recall(key)
        if bound is not None:
            if not bound():
                raise RuntimeError(f"no HIP dequantize-reduce kernel for output dtype {output.dtype}")
            return
        entries = self._entries(inputs, numel, group_size)
        if len(entries) <= ops.MAX_PAYLOADS:
            bind = lambda: ops.bind_dequant_reduce(entries, flat, numel=numel, group_size=group_size)  # noqa: E731
            if not (self._memoized(key, bind) if key is not None else bind())():
                raise RuntimeError(f"no HIP dequantize-reduce kernel for output dtype {output.dtype}")
            return
        # More than 8 payloads: keep the left fold exact by chaining decode-and-add one payload at a time.
        for r, buffer in enumerate(inputs):
            codes, scales = _views(buffer, group_size)
            if not ops.dequant_into(codes, scales, flat, numel=numel, group_size=group_size,
                                    reduce_op="none" if r == 0 else "sum"):
                raise RuntimeError(f"no HIP dequantize kernel for output dtype {output.dtype}")

    def _fused_eligible(self, inputs, output, group_size, topk, bit, quant_type) -> bool:
        if not _policy_supported(group_size, topk, False, bit, quant_type):
            return False
        if not 1 <= len(inputs) <= ops.MAX_PAYLOADS:
            return False
        if not isinstance(output, torch.Tensor) or not output.is_cuda or not output.is_contiguous():
            return False
        if output.dtype not in ops.DTYPE_CODES or output.numel() == 0:
            return False
        expected = ops.payload_nbytes(output.numel(), group_size)
        for buffer in inputs:
            if not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.uint8 or not buffer.is_cuda:
                return False
            if not buffer.is_contiguous() or buffer.device != output.device or buffer.numel() != expected:
                return False
        return True

    def inplace_dequantize_reduce_mean(self, inputs, output, group_size, topk, bit, quant_type, compact,
                                       divisor) -> bool:
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
        key = self._reduce_key("reduce_mean", inputs, (output,),
                               (group_size, topk, bit, int(quant_type), float(divisor)))
        bound = self._recall(key)
        if bound is None:
            if not self._fused_eligible(inputs, output, group_size, topk, bit, quant_type):
                return False
            bind = lambda: ops.bind_dequant_reduce(list(inputs), output.reshape(-1), group_size=group_size,  # noqa: E731
                                                   divisor=float(divisor))
            bound = self._memoized(key, bind) if key is not None else bind()
        return bound()

    # ---- error feedback -------------------------------------------------------------------------
    def inplace_error_feedback_update(self, prepared, restored, residual) -> None:
        if prepared.numel() != restored.numel():
            raise RuntimeError("prepared and restored must have the same number of elements")
        if prepared.numel() != residual.numel():
            raise RuntimeError("prepared and residual must have the same number of elements")
        if not ops.ef_update_into(prepared.reshape(-1), restored.reshape(-1), residual.reshape(-1)):
            raise RuntimeError("unsupported dtype for inplace_error_feedback_update")

    def dequantize_reduce_update_error_feedback(self, inputs, prepared, residual, group_size, topk, bit, quant_type,
                                                dtype, compact, divisor):
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
        restored = torch.empty(_padded_numel_of(inputs[0], group_size), dtype=_TORCH_OF[DType(int(dtype))],
                               device=inputs[0].device)
        trimmed = restored[:prepared.numel()]
        if not self.inplace_dequantize_reduce_mean_update_error_feedback(
                inputs, prepared, trimmed, residual, group_size, topk, bit, quant_type, compact, divisor):
            self.inplace_dequantize_reduce(inputs, trimmed, group_size, topk, bit, quant_type, compact)
            if divisor != 1:
                ops.true_divide_(trimmed, divisor)
            self.inplace_error_feedback_update(prepared, trimmed, residual)
        return restored

    def inplace_dequantize_reduce_mean_update_error_feedback(self, inputs, prepared, restored, residual, group_size,
                                                             topk, bit, quant_type, compact, divisor) -> bool:
        """One launch: ``restored = mean/sum of payloads``, ``residual = prepared - restored``."""
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
        key = self._reduce_key("reduce_mean_feedback", inputs, (prepared, restored, residual),
                               (group_size, topk, bit, int(quant_type), float(divisor)))
        bound = self._recall(key)
        if bound is not None:
            return bound()
        for name, t in (("prepared", prepared), ("restored", restored), ("residual", residual)):
            if not isinstance(t, torch.Tensor) or not t.is_cuda:
                raise RuntimeError(f"{name} must be a GPU tensor")
            if not t.is_contiguous():
                raise RuntimeError(f"{name} must be contiguous")
        if prepared.numel() != residual.numel():
            raise RuntimeError("prepared and residual must have the same number of elements")
        if restored.numel() < prepared.numel():
            raise RuntimeError("restored must have at least prepared.numel() elements")
        if prepared.dtype != restored.dtype:
            raise RuntimeError("prepared and restored must have the same dtype")
        if prepared.dtype != residual.dtype:
            raise RuntimeError("prepared and residual must have the same dtype")
        if prepared.device != restored.device or prepared.device != residual.device:
            raise RuntimeError("prepared, restored and residual must be on the same device")
        numel = prepared.numel()
        if not _policy_supported(group_size, topk, False, bit, quant_type):
            return False
        if not 1 <= len(inputs) <= ops.MAX_PAYLOADS or numel == 0:
            return False
        expected = ops.payload_nbytes(numel, group_size)
        for buffer in inputs:
            if (not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.uint8 or not buffer.is_cuda
                    or not buffer.is_contiguous() or buffer.device != prepared.device or buffer.numel() != expected):
                return False
        bind = lambda: ops.bind_dequant_reduce(list(inputs), restored.reshape(-1), numel=numel,  # noqa: E731
                                               group_size=group_size, divisor=float(divisor),
                                               prepared=prepared.reshape(-1), new_residual=residual.reshape(-1))
        return (self._memoized(key, bind) if key is not None else bind())()
