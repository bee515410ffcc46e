"""A stand-in for the reference's CUDA extension module that speaks its byte format.

Same names and positional argument orders as ``ccdl_cuda_ops`` (``ccdl_comm/csrc/pybind.cpp:133-166``),
and the same payload bytes: scales are group maxima in the tensor's dtype, codes are byte-swapped in
2- or 4-byte words, ``compact`` chooses between interleaved and appended scales
(``ccdl_comm/csrc/quantization/quant_pack_kernel.cu:101-162``).  A job can therefore mix ranks that
load this module on gfx950 with ranks that load the CUDA extension.  The portable-format twin is
:class:`lowbit_comm_amd.hip.native_module.HipNativeModule`.

Kept from the reference: the fused reduce runs only for group size 64, at most 8 payloads and an element
count that is a multiple of 64 (``dequant_reduce_kernel.cu:243-262``); otherwise payloads are decoded one
by one and added in the tensor dtype (``pybind.cpp:39-56``), which rounds differently, so eligibility is
mirrored exactly.  Every policy of the extension is implemented: linear 8- and 4-bit codes, the non-linear 4-bit
code books, stochastic rounding (seed and offset come from torch's generator of the device, as in
``gen_code_quant.py:27-36``) and the top-k side channel.  As in the reference the fused calls
(``inplace_quantize_pack``, the fused reduces) serve the plain policy only (linear, top-k 0, no stochastic
rounding, ``quant_pack_kernel.cu:231``) and return ``False`` otherwise; the other policies run through
``quantize`` / ``dequantize`` and the decode-and-add chain, and need whole groups (``gen_code_quant.py:164``).
"""
from __future__ import annotations

from typing import Sequence

import torch

from lowbit_comm_amd.hip import cuda_wire, ops
from lowbit_comm_amd.hip.library import load_library
from lowbit_comm_amd.hip.native_module import DType, QuantType, ReduceOP, _OP_NAME, _TORCH_OF, _check_payload

FUSED_GROUP_SIZE = 64
FUSED_BIT = 8


_KIND = {int(QuantType.Linear): "linear", int(QuantType.Normal): "normal", int(QuantType.Uniform): "uniform",
         int(QuantType.E3M0): "e3m0", int(QuantType.E2M1): "e2m1"}
_META_WORDS = {0: 1, 1: 3, 2: 4}


def _policy_supported(group_size: int, topk: int, stochastic: bool, bit: int, quant_type) -> bool:
    """The combinations the reference instantiates (gen_code_quant.py:42-48,243-245)."""
    return (group_size in (16, 32, 64) and topk in (0, 1, 2) and bit in (4, 8) and int(quant_type) in _KIND
            and (int(quant_type) == int(QuantType.Linear) or bit == 4))


def _plain(topk: int, stochastic: bool, quant_type) -> bool:
    """The policy the fused pack and reduce kernels serve (quant_pack_kernel.cu:231, dequant_reduce_kernel.cu:243-262)."""
    return topk == 0 and not stochastic and int(quant_type) == int(QuantType.Linear)


def _require_policy(group_size, topk, stochastic, bit, quant_type) -> None:
    if not _policy_supported(group_size, topk, stochastic, bit, quant_type):
        raise RuntimeError(
            "the HIP codec for the CUDA byte format supports group_size 16/32/64, topk 0/1/2, 8-bit linear and "
            f"4-bit linear/normal/uniform/e3m0/e2m1 codes; got group_size={group_size} topk={topk} "
            f"stochastic={stochastic} bit={bit} quant_type={getattr(quant_type, 'name', quant_type)}")


def _item(dtype: torch.dtype) -> int:
    return 4 if dtype == torch.float32 else 2


def _padded_numel(buffer: torch.Tensor, group_size: int, dtype: torch.dtype, bit: int = 8, name: str = "input",
                  topk: int = 0) -> int:
    per_group = group_size * bit // 8 + _item(dtype) * _META_WORDS[topk]
    if buffer.numel() % per_group != 0:
        raise RuntimeError(f"{name} has an invalid quantized payload size")
    return buffer.numel() // per_group * group_size


class HipCudaWireModule:
    """Instance with the reference extension's symbols over the CUDA byte format."""

    QuantType = QuantType
    DType = DType
    ReduceOP = ReduceOP
    NATIVE_WIRE_FORMAT = "native"

    def __init__(self, fused_multiply_add: bool = True) -> None:
        """``fused_multiply_add``: accumulate the fused reduce as ``fma(code, step, sum)`` (what nvcc's default
        contraction makes of the reference source) or with a separately rounded product."""
        self._lib = load_library()
        self.fused_multiply_add = bool(fused_multiply_add)

    # ---- quantize ------------------------------------------------------------------------------
    def quantize(self, input, group_size, topk, stochastic, bit, quant_type, compact):
        _require_policy(group_size, topk, stochastic, bit, quant_type)
        nbytes = cuda_wire.general_payload_nbytes(input.numel(), input.dtype, group_size, bit, topk)
        output = torch.empty(nbytes, dtype=torch.uint8, device=input.device)
        self.inplace_quantize(input, output, group_size, topk, stochastic, bit, quant_type, compact)
        return output

    def inplace_quantize(self, input, output, group_size, topk, stochastic, bit, quant_type, compact) -> None:
        _require_policy(group_size, topk, stochastic, bit, quant_type)
        if _plain(topk, stochastic, quant_type):
            done = self._quantize(input, output, None, group_size, compact, bit)
        else:
            done = self._quantize_general(input, output, group_size, topk, stochastic, bit, quant_type, compact)
        if not done:
            raise RuntimeError(f"no HIP quantize kernel for input dtype {input.dtype}")

    @staticmethod
    def philox_engine_inputs(device: torch.device, increment: int) -> tuple[int, int]:
        """(seed, offset) of the device's default generator, advanced past ``increment`` draws rounded up to a
        multiple of four: what ``CUDAGeneratorImpl::philox_engine_inputs`` hands the reference's kernels."""
        index = device.index if device.index is not None else torch.cuda.current_device()
        generator = torch.cuda.default_generators[index]
        offset = int(generator.get_offset())
        generator.set_offset(offset + (int(increment) + 3) // 4 * 4)
        return int(generator.initial_seed()), offset

    def _quantize_general(self, input, output, group_size, topk, stochastic, bit, quant_type, compact) -> bool:
        _check_payload(output, "output")
        if not isinstance(input, torch.Tensor) or not input.is_cuda:
            raise RuntimeError("input must be a GPU tensor")
        if not input.is_contiguous():
            raise RuntimeError("input must be contiguous")
        if output.device != input.device:
            raise RuntimeError("input and output must be on the same device")
        if input.numel() % group_size != 0:
            raise RuntimeError("input numel should be multiple of group_size")
        if output.numel() != cuda_wire.general_payload_nbytes(input.numel(), input.dtype, group_size, bit, topk):
            raise RuntimeError("Output tensor must have the same number of elements as the quantized tensor")
        if input.dtype not in ops.DTYPE_CODES:
            return False
        if input.numel() == 0:
            return True
        seeds = self.philox_engine_inputs(input.device, input.numel()) if stochastic else None
        return cuda_wire.quant_general_into(input.reshape(-1), output.reshape(-1), group_size=group_size, bit=bit,
                                            quant_type=_KIND[int(quant_type)], topk=topk, stochastic=seeds,
                                            compact=bool(compact))

    def inplace_quantize_pack(self, input, output, residual, group_size, topk, stochastic, bit, quant_type,
                              compact) -> bool:
        if not compact or not _plain(topk, stochastic, quant_type) or \
                not _policy_supported(group_size, topk, stochastic, bit, quant_type):
            return False                                        # quant_pack_kernel.cu:231-236
        if input.dtype not in ops.DTYPE_CODES:
            return False
        if residual is not None:
            if residual.dtype != input.dtype:
                raise RuntimeError("input and residual must have the same dtype")
            if residual.numel() != input.numel():
                raise RuntimeError("input and residual must have the same number of elements")
        return self._quantize(input, output, residual, group_size, True, bit)

    def _quantize(self, input, output, residual, group_size, compact, bit) -> bool:
        _check_payload(output, "output")
        if not isinstance(input, torch.Tensor) or not input.is_cuda:
            raise RuntimeError("input must be a GPU tensor")
        if not input.is_contiguous():
            raise RuntimeError("input must be contiguous")
        if output.device != input.device:
            raise RuntimeError("input and output must be on the same device")
        if output.numel() != cuda_wire.payload_nbytes(input.numel(), input.dtype, group_size, bit):
            raise RuntimeError("output has an invalid quantized payload size")
        if input.numel() == 0:
            return True
        flat_residual = None if residual is None else residual.reshape(-1)
        return cuda_wire.quant_pack_into(input.reshape(-1), output.reshape(-1), group_size=group_size,
                                         compact=bool(compact), residual=flat_residual, bit=bit)

    # ---- dequantize -----------------------------------------------------------------------------
    def dequantize(self, input, group_size, topk, bit, reduce_op, quant_type, dtype, compact):
        _require_policy(group_size, topk, False, bit, quant_type)
        _check_payload(input, "input")
        torch_dtype = _TORCH_OF[DType(int(dtype))]
        output = torch.empty(_padded_numel(input, group_size, torch_dtype, bit, topk=topk), dtype=torch_dtype,
                             device=input.device)
        if int(reduce_op) != int(ReduceOP.NONE):
            output.zero_()
        self.inplace_dequantize(input, output, group_size, topk, bit, reduce_op, quant_type, compact)
        return output

    def inplace_dequantize(self, input, output, group_size, topk, bit, reduce_op, quant_type, compact) -> None:
        _require_policy(group_size, topk, False, bit, quant_type)
        _check_payload(input, "input")
        flat = output.reshape(-1)
        if not _plain(topk, False, quant_type):
            if flat.numel() % group_size != 0 or \
                    input.numel() != cuda_wire.general_payload_nbytes(flat.numel(), output.dtype, group_size, bit, topk):
                raise RuntimeError("input has an invalid quantized payload size")
            if not cuda_wire.dequant_general_into(input.reshape(-1), flat, group_size=group_size, bit=bit,
                                                  quant_type=_KIND[int(quant_type)], topk=topk, compact=bool(compact),
                                                  reduce_op=_OP_NAME[ReduceOP(int(reduce_op))]):
                raise RuntimeError(f"no HIP dequantize kernel for output dtype {output.dtype}")
            return
        numel = min(flat.numel(), _padded_numel(input, group_size, output.dtype, bit))
        payload = input.reshape(-1)
        expected = cuda_wire.payload_nbytes(numel, output.dtype, group_size, bit)
        if payload.numel() != expected:
            raise RuntimeError("input has an invalid quantized payload size")
        if not cuda_wire.dequant_into(payload, flat, numel=numel, group_size=group_size, compact=bool(compact),
                                      reduce_op=_OP_NAME[ReduceOP(int(reduce_op))], bit=bit):
            raise RuntimeError(f"no HIP dequantize kernel for output dtype {output.dtype}")

    # ---- dequantize + reduce ------------------------------------------------------------------
    def _fused_eligible(self, inputs, output, group_size, topk, bit, quant_type) -> bool:
        """``can_use_fused_dequant_reduce`` (dequant_reduce_kernel.cu:243-262)."""
        if not 1 <= len(inputs) <= ops.MAX_PAYLOADS:
            return False
        if group_size != FUSED_GROUP_SIZE or bit != FUSED_BIT or not _plain(topk, False, quant_type):
            return False
        if not isinstance(output, torch.Tensor) or not output.is_cuda or not output.is_contiguous():
            return False
        if output.dtype not in ops.DTYPE_CODES or output.numel() == 0 or output.numel() % FUSED_GROUP_SIZE != 0:
            return False
        expected = cuda_wire.payload_nbytes(output.numel(), output.dtype, group_size)
        for buffer in inputs:
            if not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.uint8 or not buffer.is_cuda:
                return False
            if not buffer.is_contiguous() or buffer.device != output.device or buffer.numel() != expected:
                return False
        return True

    def _fused(self, inputs, output, compact, inv_divisor, prepared=None, residual=None) -> bool:
        numel = output.numel() if prepared is None else prepared.numel()
        return cuda_wire.dequant_reduce_into(
            [buffer.reshape(-1) for buffer in inputs], output.reshape(-1), numel=numel,
            group_size=FUSED_GROUP_SIZE, compact=bool(compact), inv_divisor=inv_divisor,
            fused_multiply_add=self.fused_multiply_add,
            prepared=None if prepared is None else prepared.reshape(-1),
            new_residual=None if residual is None else residual.reshape(-1))

    def inplace_dequantize_reduce(self, inputs: Sequence[torch.Tensor], output, group_size, topk, bit, quant_type,
                                  compact) -> None:
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        if self._fused_eligible(inputs, output, group_size, topk, bit, quant_type) and \
                self._fused(inputs, output, compact, 1.0):
            return
        for i, buffer in enumerate(inputs):                      # pybind.cpp:44-55
            self.inplace_dequantize(buffer, output, group_size, topk, bit,
                                    ReduceOP.NONE if i == 0 else ReduceOP.SUM, quant_type, compact)

    def dequantize_reduce(self, inputs, group_size, topk, bit, quant_type, dtype, compact):
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        _check_payload(inputs[0], "input")
        torch_dtype = _TORCH_OF[DType(int(dtype))]
        output = torch.empty(_padded_numel(inputs[0], group_size, torch_dtype, bit, topk=topk), dtype=torch_dtype,
                             device=inputs[0].device)
        self.inplace_dequantize_reduce(inputs, output, group_size, topk, bit, quant_type, compact)
        return output

    def inplace_dequantize_reduce_mean(self, inputs, output, group_size, topk, bit, quant_type, compact,
                                       divisor) -> bool:
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
        if not self._fused_eligible(inputs, output, group_size, topk, bit, quant_type):
            return False
        inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(divisor), dtype=torch.float32))
        return self._fused(inputs, output, compact, inv)

    # ---- error feedback -------------------------------------------------------------------------
    def inplace_error_feedback_update(self, prepared, restored, residual) -> None:
        for name, t in (("prepared", prepared), ("restored", restored), ("residual", residual)):
            if not isinstance(t, torch.Tensor) or not t.is_cuda:
                raise RuntimeError(f"{name} must be a GPU tensor")
            if not t.is_contiguous():
                raise RuntimeError(f"{name} must be contiguous")
        if prepared.numel() != restored.numel():
            raise RuntimeError("prepared and restored must have the same number of elements")
        if prepared.numel() != residual.numel():
            raise RuntimeError("prepared and residual must have the same number of elements")
        if prepared.dtype != restored.dtype:
            raise RuntimeError("prepared and restored must have the same dtype")
        if prepared.dtype != residual.dtype:
            raise RuntimeError("prepared and residual must have the same dtype")
        if not ops.ef_update_into(prepared.reshape(-1), restored.reshape(-1), residual.reshape(-1)):
            raise RuntimeError("unsupported dtype for inplace_error_feedback_update")

    def inplace_dequantize_reduce_mean_update_error_feedback(self, inputs, prepared, restored, residual, group_size,
                                                             topk, bit, quant_type, compact, divisor) -> bool:
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
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
        if not self._fused_eligible(inputs, restored, group_size, topk, bit, quant_type):
            return False                                        # eligibility is judged on `restored` (:381)
        if -(-prepared.numel() // FUSED_GROUP_SIZE) * FUSED_GROUP_SIZE != restored.numel():
            return False           # the kernel derives the group count from prepared.numel() (:387, :170)
        inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(divisor), dtype=torch.float32))
        return self._fused(inputs, restored, compact, inv, prepared, residual)

    def dequantize_reduce_update_error_feedback(self, inputs, prepared, residual, group_size, topk, bit, quant_type,
                                                dtype, compact, divisor):
        if len(inputs) == 0:
            raise RuntimeError("inputs must not be empty")
        if divisor <= 0:
            raise RuntimeError("divisor must be > 0")
        torch_dtype = _TORCH_OF[DType(int(dtype))]
        restored = torch.empty(_padded_numel(inputs[0], group_size, torch_dtype, bit, topk=topk), dtype=torch_dtype,
                               device=inputs[0].device)
        if self.inplace_dequantize_reduce_mean_update_error_feedback(
                inputs, prepared, restored, residual, group_size, topk, bit, quant_type, compact, divisor):
            return restored
        self.inplace_dequantize_reduce(inputs, restored, group_size, topk, bit, quant_type, compact)
        if divisor != 1:
            restored = restored / divisor                        # pybind.cpp:126-128: torch's own scalar division
        self.inplace_error_feedback_update(prepared, restored, residual)
        return restored
