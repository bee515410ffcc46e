"""Host-side checks for the general policies of the CUDA byte format that need no GPU: payload sizes, the policy
matrix the module accepts, and argument validation of the C entry points (which happens before any device work)."""
import ctypes
import itertools

import pytest
import torch

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip import cuda_wire, library
from lowbit_comm_amd.hip import cuda_wire_module as module
from lowbit_comm_amd.quantization.sizing import estimate_quantized_size
from oracle import cuda_wire_general_np as general

TORCH = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.mark.parametrize("name", list(TORCH))
def test_payload_sizes_agree_between_binding_library_oracle_and_sizing(name):
    lib = library.load_library()
    code = {"fp32": 0, "fp16": 1, "bf16": 2}[name]
    for g, bit, topk, numel in itertools.product((16, 32, 64), (4, 8), (0, 1, 2), (0, 64, 640, 64 * 1001)):
        want = general.payload_nbytes(numel, g, name, bit, topk)
        assert cuda_wire.general_payload_nbytes(numel, TORCH[name], g, bit, topk) == want
        assert lib.lbc_wire_general_payload_nbytes(numel, g, code, bit, topk) == want
        config = CompressionConfig(bit=bit, group_size=g, topk=topk, allow_experimental=True)
        assert estimate_quantized_size(numel, dtype=name, config=config, wire_format="native").quantized_bytes == want
    assert lib.lbc_wire_general_payload_nbytes(64, 64, code, 8, 3) == -1
    assert lib.lbc_wire_general_payload_nbytes(64, 48, code, 8, 0) == -1
    assert lib.lbc_wire_general_payload_nbytes(-1, 64, code, 8, 0) == -1
    # without a side channel the size is the plain format's
    assert lib.lbc_wire_general_payload_nbytes(6400, 64, code, 8, 0) == lib.lbc_wire_payload_nbytes(6400, 64, code, 8)


def test_policy_matrix_is_what_the_reference_instantiates():
    """gen_code_quant.py:42-48,243-245: groups 16/32/64, top-k 0/1/2, 8-bit linear, 4-bit linear and the four code
    books, each with and without stochastic rounding."""
    kinds = list(module.QuantType)
    accepted = [(g, k, s, b, q) for g, k, s, b, q in itertools.product((8, 16, 32, 64, 128), (0, 1, 2, 3), (False, True),
                                                                         (2, 4, 8, 16), kinds)
                if module._policy_supported(g, k, s, b, q)]
    assert len(accepted) == 3 * 3 * 2 * (1 + 5)
    assert all(b == 4 or q == module.QuantType.Linear for _, _, _, b, q in accepted)
    plain = [p for p in accepted if module._plain(p[1], p[2], p[4])]
    assert len(plain) == 3 * 2 and all(k == 0 and not s for _, k, s, _, _ in plain)
    assert module._KIND == {0: "linear", 1: "normal", 2: "uniform", 3: "e3m0", 4: "e2m1"}
    assert cuda_wire.QUANT_TYPES == {name: index for index, name in enumerate(general.QUANT_TYPES)}


def test_general_entry_points_validate_before_any_device_work():
    lib = library.load_library()
    none = ctypes.c_void_p(None)
    quant, decode = lib.lbc_wire_quant_general, lib.lbc_wire_dequant_general
    assert quant(none, 0, 0, 64, 8, 0, 2, 1, 5, 8, 1, none, none) == 0                   # empty: no-op
    assert quant(none, 0, 100, 64, 8, 0, 0, 0, 0, 0, 0, none, none) == -1
    assert library.last_error(lib) == "input numel should be multiple of group_size"
    assert quant(none, 0, 128, 64, 8, 1, 0, 0, 0, 0, 0, none, none) == 1                 # code book needs 4-bit codes
    assert quant(none, 0, 128, 64, 4, 5, 0, 0, 0, 0, 0, none, none) == 1                 # no such quant type
    assert quant(none, 0, 128, 64, 8, 0, 3, 0, 0, 0, 0, none, none) == 1                 # top-k 3
    assert quant(none, 0, 128, 48, 8, 0, 0, 0, 0, 0, 0, none, none) == 1                 # group size
    assert quant(none, 9, 128, 64, 8, 0, 0, 0, 0, 0, 0, none, none) == -1
    assert "unsupported dtype" in library.last_error(lib)
    assert quant(none, 0, 128, 64, 8, 0, 0, 0, 0, 0, 0, none, none) == -1
    assert library.last_error(lib) == "input and payload must not be null"
    assert decode(none, 0, 64, 8, 0, 1, 0, none, 0, 0, none) == 0
    assert decode(none, 70, 64, 8, 0, 1, 0, none, 0, 0, none) == -1
    assert decode(none, 128, 64, 8, 0, 1, 0, none, 0, 7, none) == -1
    assert "unsupported reduce op" in library.last_error(lib)
    assert decode(none, 128, 64, 8, 2, 0, 0, none, 0, 0, none) == 1
    assert decode(none, 128, 64, 4, 2, 0, 0, none, 0, 0, none) == -1
    assert library.last_error(lib) == "payload and out must not be null"


def test_tensor_level_binding_rejects_bad_policies_without_a_gpu():
    x = torch.zeros(128)
    payload = torch.zeros(136, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        cuda_wire.quant_general_into(x, payload)
    with pytest.raises(RuntimeError, match="topk must be"):
        cuda_wire.general_payload_nbytes(128, torch.float32, 64, 8, 5)
