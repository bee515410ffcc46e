"""CPU tests of the host-side mirror of the reference interface: config, sizing, error feedback, policy,
payload packing, codec facade argument marshalling, quantizer, chunk plan, shard metadata, caches, hooks.

They restate the behaviours the reference's own tests pin (cited per test) against this package.
"""
import dataclasses

import pytest
import torch

from lowbit_comm_amd import CCDLUnavailableError, CompressionConfig, ReducedShard, UnsupportedCollective
from lowbit_comm_amd.communication import (
    CompressedPayload,
    FusedPayloadPacker,
    GatheredPayloads,
    make_fused_payload_all_gather,
    make_payload_all_gather,
    should_fuse_payload,
)
from lowbit_comm_amd.communication.ddp import DDPBucketProcessor
from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
from lowbit_comm_amd.communication.workspace import DequantizedWorkspaceCache, ShardCommunicationWorkspaceCache
from lowbit_comm_amd.hip.chunk_plan import ChunkPlan, ChunkRange, compile_chunk_plan
from lowbit_comm_amd.hip.loader import HipExtensionStatus, load_hip_extension
from lowbit_comm_amd.quantization import ErrorFeedbackState, Quantizer, estimate_payload_size, estimate_quantized_size
from lowbit_comm_amd.quantization import codec
from lowbit_comm_amd.quantization.error_feedback_policy import ErrorFeedbackPolicy


# --------------------------------------------------------------------------- #
# config (reference tests/test_config.py)
# --------------------------------------------------------------------------- #
def test_config_defaults_and_validation():
    cfg = CompressionConfig()
    assert (cfg.bit, cfg.group_size, cfg.topk, cfg.quant_type, cfg.error_feedback) == (8, 64, 0, "linear", True)
    assert cfg.effective_error_feedback_policy() == "always"
    assert CompressionConfig(error_feedback=False).effective_error_feedback_policy() == "none"
    with pytest.raises(ValueError, match="Unsupported target"):
        CompressionConfig(target="gpu")
    with pytest.raises(ValueError, match="bit"):
        CompressionConfig(bit=3)
    with pytest.raises(ValueError, match="experimental"):
        CompressionConfig(bit=4)
    assert CompressionConfig(bit=4, allow_experimental=True).bit == 4
    with pytest.raises(ValueError, match="Unsupported group_size"):
        CompressionConfig(group_size=128)
    with pytest.raises(ValueError, match="Unsupported error_feedback_policy"):
        CompressionConfig(error_feedback_policy="sometimes")
    for field, bad in (("error_feedback_min_numel", -1), ("error_feedback_warmup_steps", -1), ("error_feedback_period", 0)):
        with pytest.raises(ValueError, match=field):
            CompressionConfig(**{field: bad})
    with pytest.raises(dataclasses.FrozenInstanceError):
        cfg.bit = 4


# --------------------------------------------------------------------------- #
# sizing (reference tests/test_quantization_sizing.py:7-51)
# --------------------------------------------------------------------------- #
def test_native_sizing_matches_the_reference_fixture(golden_vectors):
    for case in golden_vectors["sizing"]["cases"]:
        estimate = estimate_quantized_size(case["numel"], dtype=case["dtype"], config=CompressionConfig(**case["config"]))
        for field, want in case.items():
            if field not in ("numel", "dtype", "config"):
                assert getattr(estimate, field) == want, (case, field)


def test_native_sizing_matches_the_reference_numbers():
    cfg = CompressionConfig()
    e = estimate_quantized_size(128, dtype="fp16", config=cfg)
    assert (e.num_groups, e.padded_numel, e.padding_numel, e.original_bytes, e.quantized_bytes) == (2, 128, 0, 256, 132)
    e = estimate_quantized_size(65, dtype="fp16", config=cfg)
    assert (e.num_groups, e.padded_numel, e.padding_numel, e.quantized_bytes) == (2, 128, 63, 132)
    assert estimate_quantized_size(64, dtype="fp32", config=cfg).quantized_bytes == 68
    assert estimate_quantized_size(64, dtype="fp16", config=CompressionConfig(topk=2)).quantized_bytes == 72
    four = CompressionConfig(bit=4, allow_experimental=True)
    assert estimate_quantized_size(64, dtype="fp16", config=four).quantized_bytes == 34
    assert estimate_quantized_size(0, dtype="fp16", config=cfg).compression_ratio == 0.0
    with pytest.raises(ValueError, match="dtype"):
        estimate_quantized_size(64, dtype="fp64", config=cfg)
    with pytest.raises(ValueError, match="non-negative"):
        estimate_quantized_size(-1, dtype="fp16", config=cfg)


def test_portable_wire_format_is_68_bytes_per_group_for_every_dtype():
    cfg = CompressionConfig()
    for dtype in ("fp16", "bf16", "fp32"):
        assert estimate_payload_size(128, dtype=dtype, config=cfg).quantized_bytes == 136
        assert estimate_payload_size(65, dtype=dtype, config=cfg).quantized_bytes == 136
    assert estimate_payload_size(6_553_600, dtype="fp32", config=cfg).quantized_bytes == 6_963_200
    assert estimate_payload_size(64, dtype="bf16", config=CompressionConfig(group_size=16)).quantized_bytes == 4 * 20
    with pytest.raises(ValueError, match="wire_format"):
        estimate_quantized_size(64, dtype="fp16", config=cfg, wire_format="compact")


# --------------------------------------------------------------------------- #
# error feedback (reference tests/test_error_feedback.py:36-95)
# --------------------------------------------------------------------------- #
class Vec:
    """Minimal tensor stand-in: +, -, detach, clone, shape."""

    def __init__(self, values, detached=False, cloned=False):
        self.values = tuple(values)
        self.detached, self.cloned = detached, cloned

    shape = property(lambda self: (len(self.values),))

    def __add__(self, other):
        if self.shape != other.shape:
            raise RuntimeError("shape mismatch")
        return Vec(a + b for a, b in zip(self.values, other.values))

    def __sub__(self, other):
        if self.shape != other.shape:
            raise RuntimeError("shape mismatch")
        return Vec(a - b for a, b in zip(self.values, other.values))

    def detach(self):
        return Vec(self.values, True, self.cloned)

    def clone(self):
        return Vec(self.values, self.detached, True)

    def __eq__(self, other):
        return isinstance(other, Vec) and (self.values, self.detached, self.cloned) == (
            other.values, other.detached, other.cloned)


def test_error_feedback_state_literal_cycle():
    state = ErrorFeedbackState()
    first = Vec([1.0, 2.0])
    assert state.compensate("b0", first) is first
    state.update("b0", original=first, transmitted=Vec([0.75, 1.5]))
    assert state.get("b0") == Vec([0.25, 0.5], True, True)
    assert state.compensate("b0", Vec([10.0, 20.0])) == Vec([10.25, 20.5])
    state.update("b1", original=Vec([4.0]), transmitted=Vec([3.0]))
    compensated = state.compensate("b1", Vec([10.0]))
    state.update("b1", original=compensated, transmitted=Vec([10.25]))
    assert compensated == Vec([11.0]) and state.get("b1") == Vec([0.75], True, True)
    state.clear("b0")
    assert state.get("b0") is None and state.get("b1") is not None
    state.clear()
    assert state.get("b1") is None


def test_error_feedback_drops_a_residual_whose_shape_changed():
    state = ErrorFeedbackState()
    state.update("b", original=Vec([4.0, 5.0]), transmitted=Vec([3.0, 4.0]))
    other = Vec([10.0])
    assert state.compensate("b", other) is other
    assert state.get("b") is None


def test_bf16_plus_fp32_residual_promotes_to_fp32():
    state = ErrorFeedbackState()
    state.put("b", torch.full((4,), 1e-5))
    out = state.compensate("b", torch.ones(4, dtype=torch.bfloat16))
    assert out.dtype == torch.float32


# --------------------------------------------------------------------------- #
# policy (reference tests/test_error_feedback_policy.py:5-86)
# --------------------------------------------------------------------------- #
def test_error_feedback_policies():
    d = ErrorFeedbackPolicy(CompressionConfig(error_feedback=False)).decide("b", numel=10)
    assert (d.apply, d.update, d.reason) == (False, False, "error feedback disabled")
    d = ErrorFeedbackPolicy(CompressionConfig()).decide("b", numel=10)
    assert (d.apply, d.update, d.reason) == (True, True, "error feedback policy always")
    p = ErrorFeedbackPolicy(CompressionConfig(error_feedback_policy="large_bucket_only", error_feedback_min_numel=4096))
    assert p.decide("a", numel=1024).reason == "bucket numel 1024 below error feedback threshold 4096"
    big = p.decide("a", numel=4096)
    assert big.apply and big.update and big.reason == "bucket numel 4096 reached error feedback threshold 4096"
    p = ErrorFeedbackPolicy(CompressionConfig(error_feedback_policy="warmup_then_enable", error_feedback_warmup_steps=2))
    seen = []
    for _ in range(3):
        seen.append(p.decide("a", numel=1))
        p.advance("a")
    assert [s.apply for s in seen] == [False, False, True]
    assert seen[1].reason == "bucket step 1 before error feedback warmup 2"
    assert seen[2].reason == "bucket step 2 reached error feedback warmup 2"
    assert not p.decide("other", numel=1).apply          # counters are per bucket
    p = ErrorFeedbackPolicy(CompressionConfig(error_feedback_policy="periodic", error_feedback_period=3))
    seen = []
    for _ in range(4):
        seen.append(p.decide("a", numel=1))
        p.advance("a")
    assert [s.apply for s in seen] == [True] * 4
    assert [s.update for s in seen] == [True, False, False, True]
    assert seen[1].reason == "bucket step 1 skips error feedback update until period 3"


# --------------------------------------------------------------------------- #
# payload packing (reference tests/test_payload_packing.py:12-76)
# --------------------------------------------------------------------------- #
def _payload(codes, scales, dtype=torch.float16):
    return CompressedPayload(buffer=torch.tensor(codes, dtype=torch.int8), shape=(len(codes),), dtype="fp16",
                             metadata={"scales": torch.tensor(scales, dtype=dtype), "original_numel": len(codes)})


def test_fused_payload_all_gather_packs_once_and_round_trips(golden_vectors):
    """The reference's own packer case (tests/test_payload_packing.py:12-57): float16 scales, a round trip, one byte
    collective; it asserts no packed bytes."""
    case = golden_vectors["packer"]
    assert case["scales_dtype"] == "float16"
    assert (case["local"]["codes"], case["local"]["scales"]) == ([-2, 3, 7, 11], [0.25, 0.5])
    assert (case["remote"]["codes"], case["remote"]["scales"]) == ([1, 2, 3, 4], [1.0, 2.0])
    local = _payload(case["local"]["codes"], case["local"]["scales"])
    remote = _payload(case["remote"]["codes"], case["remote"]["scales"])
    calls = []

    def byte_all_gather(packed):
        calls.append((packed.dtype, tuple(packed.shape)))
        return GatheredPayloads(payloads=[packed, fused.packer.pack(remote)], world_size=2)

    fused = make_fused_payload_all_gather(byte_all_gather)
    gathered = fused(local)
    assert calls == [(torch.uint8, (case["packed_numel"],))]
    assert gathered.world_size == 2
    assert [p.buffer.tolist() for p in gathered.payloads] == [[-2, 3, 7, 11], [1, 2, 3, 4]]
    assert [p.metadata["scales"].tolist() for p in gathered.payloads] == [[0.25, 0.5], [1.0, 2.0]]
    assert [p.metadata["original_numel"] for p in gathered.payloads] == [4, 4]


def test_packed_bytes_are_codes_then_little_endian_fp32_scales():
    payload = _payload([-2, 3, 7, 11], [0.25, 1.0], dtype=torch.float32)
    packer = FusedPayloadPacker.from_payload(payload)
    assert packer.pack(payload).tolist() == [254, 3, 7, 11, 0, 0, 128, 62, 0, 0, 128, 63]
    assert packer.packed_bytes == 12 and packer.metadata_schemas[0].offset == 4
    back = packer.unpack(packer.pack(payload), shape=(4,), dtype="fp32")
    assert back.buffer.dtype == torch.int8 and back.metadata["scales"].dtype == torch.float32


def test_packed_payload_is_shipped_as_is_only_while_its_pieces_are_still_views_of_it():
    from lowbit_comm_amd.communication import PackedPayload

    packed = torch.tensor([254, 3, 7, 11, 0, 0, 128, 62, 0, 0, 128, 63], dtype=torch.uint8)
    codes, scales = packed[:4].view(torch.int8), packed[4:].view(torch.float32)
    payload = PackedPayload(buffer=codes, shape=(4,), dtype="fp32", metadata={"scales": scales, "original_numel": 4},
                            packed=packed)
    packer = FusedPayloadPacker.from_payload(payload)
    assert packer.pack(payload) is packed                              # no copy
    swapped = dataclasses.replace(payload, buffer=torch.tensor([1, 2, 3, 4], dtype=torch.int8))
    assert packer.pack(swapped).tolist() == [1, 2, 3, 4, 0, 0, 128, 62, 0, 0, 128, 63]
    edited = dataclasses.replace(payload, metadata={"scales": torch.tensor([2.0, 4.0]), "original_numel": 4})
    assert packer.pack(edited).tolist() == [254, 3, 7, 11, 0, 0, 0, 64, 0, 0, 128, 64]
    shifted = dataclasses.replace(payload, metadata={"scales": packed[0:8].view(torch.float32), "original_numel": 4})
    assert packer.pack(shifted) is not packed                          # a view of the allocation, at the wrong offset


def test_fused_packer_rejects_payloads_without_tensor_metadata():
    fused = make_fused_payload_all_gather(lambda packed: GatheredPayloads([packed], 1))
    bare = CompressedPayload(buffer=torch.tensor([1, 2, 3], dtype=torch.int8), shape=(3,), dtype="fp16",
                             metadata={"original_numel": 3})
    with pytest.raises(ValueError, match="requires tensor metadata"):
        fused(bare)


def test_unfused_gather_moves_buffer_and_each_tensor_item():
    sent = []

    def gather(tensor):
        sent.append(tuple(tensor.shape))
        return GatheredPayloads([tensor, tensor + 1], 2)

    out = make_payload_all_gather(gather)(_payload([1, 2, 3, 4], [1.0, 2.0]))
    assert sent == [(4,), (2,)]
    assert out.payloads[1].buffer.tolist() == [2, 3, 4, 5] and out.payloads[1].metadata["scales"].tolist() == [2.0, 3.0]
    assert out.payloads[1].metadata["original_numel"] == 4


def test_should_fuse_payload_threshold():
    t = torch.zeros(10)
    assert not should_fuse_payload(t, enabled=False)
    assert should_fuse_payload(t, enabled=True, min_numel=0)
    assert should_fuse_payload(t, enabled=True, min_numel=10)
    assert not should_fuse_payload(t, enabled=True, min_numel=11)
    assert not should_fuse_payload(t, enabled=True)          # default 4,000,000


# --------------------------------------------------------------------------- #
# codec facade argument marshalling (reference tests/test_quantization_codec.py)
# --------------------------------------------------------------------------- #
class Enum:
    def __init__(self, *names):
        for n in names:
            setattr(self, n, f"<{n}>")


class RecordingModule:
    QuantType = Enum("Linear", "Normal", "Uniform", "E3M0", "E2M1")
    DType = Enum("FP16", "BF16", "FP32")
    ReduceOP = Enum("SUM", "NONE", "MIN", "MAX")

    def __init__(self, pack_result=True, fused_result=True):
        self.calls = []
        self.pack_result, self.fused_result = pack_result, fused_result

    def _rec(self, name, result=None):
        def call(*args):
            self.calls.append((name,) + args)
            return result
        return call

    def __getattr__(self, name):
        table = {"quantize": "Q", "dequantize": torch.arange(128.0), "inplace_quantize": None,
                 "inplace_dequantize": None, "dequantize_reduce": torch.arange(128.0),
                 "inplace_dequantize_reduce": None, "inplace_error_feedback_update": None,
                 "dequantize_reduce_update_error_feedback": torch.arange(128.0)}
        if name == "inplace_quantize_pack":
            return self._rec(name, self.pack_result)
        if name in ("inplace_dequantize_reduce_mean", "inplace_dequantize_reduce_mean_update_error_feedback"):
            return self._rec(name, self.fused_result)
        if name in table:
            return self._rec(name, table[name])
        raise AttributeError(name)


def status(module):
    return HipExtensionStatus(available=True, module=module)


CFG = CompressionConfig(group_size=64)


def test_quantize_tensor_pads_and_forwards_the_policy_tuple():
    m = RecordingModule()
    x = torch.ones(100)
    assert codec.quantize_tensor(x, CFG, extension_status=status(m)) == "Q"
    name, padded, *policy = m.calls[0]
    assert name == "quantize" and padded.numel() == 128 and padded[100:].abs().sum() == 0
    assert policy == [64, 0, False, 8, "<Linear>", False]


def test_quantize_with_output_prefers_the_fused_pack_call_and_reports_metadata():
    m = RecordingModule(pack_result=True)
    x, out, res, meta = torch.ones(100), torch.empty(136, dtype=torch.uint8), torch.zeros(100), {}
    assert codec.quantize_tensor(x, CFG, extension_status=status(m), output=out, residual=res, metadata=meta) is out
    assert m.calls == [("inplace_quantize_pack", x, out, res, 64, 0, False, 8, "<Linear>", False)]
    assert meta == {"original_numel": 100, "padded_numel": 128, "padding_numel": 28, "fused_quant_pack": True}


def test_quantize_with_output_falls_back_to_inplace_quantize_when_fused_declines():
    m = RecordingModule(pack_result=False)
    x, out, res = torch.ones(64), torch.empty(68, dtype=torch.uint8), torch.full((64,), 2.0)
    codec.quantize_tensor(x, CFG, extension_status=status(m), output=out, residual=res)
    assert [c[0] for c in m.calls] == ["inplace_quantize_pack", "inplace_quantize"]
    _, prepared, got_out, *policy = m.calls[1]
    assert torch.equal(prepared, torch.full((64,), 3.0)) and got_out is out
    assert policy == [64, 0, False, 8, "<Linear>", False]
    assert codec.inplace_quantize_pack(x, out, None, CFG, extension_status=status(m)) is False


def test_dequantize_tensor_forwards_enums_and_trims_to_shape():
    m = RecordingModule()
    out = codec.dequantize_tensor("buf", (10, 10), CFG, dtype="bf16", extension_status=status(m))
    assert m.calls == [("dequantize", "buf", 64, 0, 8, "<NONE>", "<Linear>", "<BF16>", False)]
    assert tuple(out.shape) == (10, 10) and out[9, 9] == 99
    ws = torch.zeros(128)
    codec.dequantize_tensor("buf", (100,), CFG, dtype="fp32", extension_status=status(m), output=ws, reduce_op="sum")
    assert m.calls[1] == ("inplace_dequantize", "buf", ws, 64, 0, 8, "<SUM>", "<Linear>", False)


def test_dequantize_reduce_tensors_paths():
    m = RecordingModule(fused_result=True)
    ws = torch.full((128,), 6.0)
    out = codec.dequantize_reduce_tensors(["a", "b", "c"], (100,), CFG, dtype="fp32", extension_status=status(m),
                                          output=ws, reduce="mean")
    assert m.calls == [("inplace_dequantize_reduce_mean", ["a", "b", "c"], ws, 64, 0, 8, "<Linear>", False, 3)]
    assert out.numel() == 100 and out[0] == 6.0          # fused call already applied the mean
    m = RecordingModule(fused_result=False)
    out = codec.dequantize_reduce_tensors(["a", "b", "c"], (100,), CFG, dtype="fp32", extension_status=status(m),
                                          output=ws, reduce="mean")
    assert [c[0] for c in m.calls] == ["inplace_dequantize_reduce_mean", "inplace_dequantize_reduce"]
    assert m.calls[1] == ("inplace_dequantize_reduce", ["a", "b", "c"], ws, 64, 0, 8, "<Linear>", False)
    assert out[0] == 2.0                                  # div_ in place on the fallback
    m = RecordingModule()
    out = codec.dequantize_reduce_tensors(["a", "b"], (128,), CFG, dtype="fp16", extension_status=status(m), reduce="mean")
    assert m.calls == [("dequantize_reduce", ["a", "b"], 64, 0, 8, "<Linear>", "<FP16>", False)]
    assert out[4] == 2.0
    with pytest.raises(ValueError, match="unsupported dequantize-reduce mode"):
        codec.dequantize_reduce_tensors(["a"], (1,), CFG, dtype="fp32", extension_status=status(m), reduce="max")
    with pytest.raises(ValueError, match="must not be empty"):
        codec.dequantize_reduce_tensors([], (1,), CFG, dtype="fp32", extension_status=status(m))


def test_error_feedback_facade_calls():
    m = RecordingModule()
    assert codec.inplace_dequantize_reduce_mean_update_error_feedback(
        ["a", "b"], "P", "R", "E", CFG, extension_status=status(m), reduce="mean") is True
    assert m.calls[0] == ("inplace_dequantize_reduce_mean_update_error_feedback", ["a", "b"], "P", "R", "E",
                          64, 0, 8, "<Linear>", False, 2)
    out = codec.dequantize_reduce_update_error_feedback(["a", "b"], "P", "E", (100,), CFG, dtype="fp32",
                                                        extension_status=status(m), reduce="sum")
    assert m.calls[1] == ("dequantize_reduce_update_error_feedback", ["a", "b"], "P", "E", 64, 0, 8, "<Linear>",
                          "<FP32>", False, 1)
    assert out.numel() == 100
    assert codec.update_error_feedback_residual("P", "R", "E", extension_status=status(m)) == "E"
    assert m.calls[2] == ("inplace_error_feedback_update", "P", "R", "E")
    with pytest.raises(ValueError, match="unsupported dequantize-reduce mode"):
        codec.inplace_dequantize_reduce_mean(["a"], "O", CFG, extension_status=status(m), reduce="max")


def test_unavailable_or_incomplete_native_module_raises():
    with pytest.raises(CCDLUnavailableError, match="no GPU here"):
        codec.quantize_tensor(torch.ones(64), CFG, extension_status=HipExtensionStatus(False, None, "no GPU here"))

    class NoQuantize:
        QuantType = Enum("Linear")

    with pytest.raises(CCDLUnavailableError, match="missing required symbol: quantize"):
        codec.quantize_tensor(torch.ones(64), CFG, extension_status=status(NoQuantize()))
    with pytest.raises(CCDLUnavailableError, match="inplace_error_feedback_update"):
        codec.update_error_feedback_residual(1, 2, 3, extension_status=status(NoQuantize()))
    with pytest.raises(CCDLUnavailableError, match="missing required symbol: QuantType"):
        codec.quantize_tensor(torch.ones(64), CFG, extension_status=status(object()))


def test_default_extension_status_is_unavailable_without_a_gpu_and_never_falls_back():
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    found = load_hip_extension()
    assert not found.available and found.module is None and "GPU" in found.reason
    with pytest.raises(CCDLUnavailableError):
        codec.quantize_tensor(torch.ones(64), CFG)
    broken = load_hip_extension(factory=lambda: (_ for _ in ()).throw(OSError("cannot load liblbc_hip.so")))
    assert not broken.available and "cannot load" in broken.reason


def test_loader_wire_format_choice():
    with pytest.raises(ValueError, match="wire_format"):
        load_hip_extension(wire_format="format-b")
    if not torch.cuda.is_available():
        assert not load_hip_extension(wire_format="native").available
    from lowbit_comm_amd.hip.cuda_wire_module import HipCudaWireModule
    from lowbit_comm_amd.hip.native_module import HipNativeModule

    portable = load_hip_extension(factory=HipNativeModule)      # constructing only loads the library
    native = load_hip_extension(factory=HipCudaWireModule)
    assert portable.module.NATIVE_WIRE_FORMAT == "portable" and native.module.NATIVE_WIRE_FORMAT == "native"
    names = [n for n in dir(HipNativeModule) if not n.startswith("_")]
    # same surface as the reference's pybind module, plus what the facade probes for - the portable format's
    # sum-and-divide in one launch (the CUDA byte format divides the way torch does instead) and the flag that the
    # fused quantize also writes bucket + residual - and the size of the launch memo
    assert set(names) - set(dir(HipCudaWireModule)) == {"dequantize_reduce_mean", "QUANTIZE_PACK_WRITES_PREPARED",
                                                        "LAUNCH_MEMO_ENTRIES"}


def test_workspace_allocators():
    x = torch.ones(100, dtype=torch.bfloat16)
    assert codec.allocate_quantized_buffer(x, CFG, dtype="bf16").shape == (136,)
    assert codec.allocate_quantized_buffer(x, CFG, dtype="bf16", wire_format="native").shape == (132,)
    ws = codec.allocate_dequantized_buffer(x, (10, 10), CFG)
    assert ws.shape == (128,) and ws.dtype == torch.bfloat16
    assert codec.allocate_dequantized_buffer(x, (), CFG).shape == (0,)


def test_quantizer_facade_round_trips_through_dict():
    seen = []
    q = Quantizer(CompressionConfig(group_size=32), dtype="bf16", extension_status="S",
                  quantize_fn=lambda *a, **k: seen.append(("q", a, k)) or "QB",
                  dequantize_fn=lambda *a, **k: seen.append(("d", a, k)) or "T",
                  allocate_fn=lambda *a, **k: seen.append(("a", a, k)) or "B")
    assert q.quantize("x", output="o") == "QB" and seen[-1] == ("q", ("x", q.config), {"extension_status": "S", "output": "o"})
    assert q.dequantize("b", (4,), dtype="fp16", reduce_op="sum") == "T"
    assert seen[-1][2] == {"dtype": "fp16", "extension_status": "S", "output": None, "reduce_op": "sum"}
    assert q.allocate_q("x") == "B" and seen[-1] == ("a", ("x", q.config), {"dtype": "bf16"})
    assert q.is_quantized()
    clone = Quantizer.from_dict(q.to_dict())
    assert clone.config == q.config and clone.dtype == "bf16"


# --------------------------------------------------------------------------- #
# chunk plan + shard (reference tests/cuda/test_compressed_reduce_scatter.py)
# --------------------------------------------------------------------------- #
def test_chunk_plan():
    plan = compile_chunk_plan(original_numel=10, world_size=4)
    assert (plan.shard_numel, plan.padded_numel) == (3, 12)
    assert plan.chunks == (ChunkRange(0, 3), ChunkRange(3, 6), ChunkRange(6, 9), ChunkRange(9, 12))
    assert plan.owner_by_chunk == (0, 1, 2, 3) and plan.chunk_for_rank(2).numel == 3
    assert compile_chunk_plan(original_numel=0, world_size=2).shard_numel == 0
    with pytest.raises(ValueError, match="rank"):
        plan.chunk_for_rank(4)
    with pytest.raises(TypeError, match="rank must be an integer"):
        plan.chunk_for_rank(True)
    with pytest.raises(TypeError, match="must be an integer"):
        compile_chunk_plan(original_numel=1.5, world_size=2)
    with pytest.raises(ValueError, match="world_size"):
        compile_chunk_plan(original_numel=4, world_size=0)
    with pytest.raises(ValueError, match="padded_numel"):
        dataclasses.replace(plan, padded_numel=13)
    with pytest.raises(ValueError, match="chunks"):
        dataclasses.replace(plan, chunks=plan.chunks[::-1])
    with pytest.raises(ValueError, match="owner_by_chunk"):
        dataclasses.replace(plan, owner_by_chunk=(3, 2, 1, 0))
    with pytest.raises(TypeError, match="owner_by_chunk"):
        dataclasses.replace(plan, owner_by_chunk=(0, 1, 2, "3"))
    assert isinstance(plan, ChunkPlan)


def test_reduced_shard_geometry():
    s = ReducedShard(shard="T", shard_index=3, shard_numel=3, original_shape=(10,), original_numel=10, world_size=4,
                     reduce="sum", metadata={"k": 1})
    assert (s.shard_offset, s.shard_end, s.valid_numel, s.padding_numel, s.padded_numel) == (9, 10, 1, 2, 12)
    assert s.has_padding and not s.is_padding_only and s.logical_range == (9, 10)
    assert s.to_metadata()["metadata"] == {"k": 1}
    with pytest.raises(TypeError):
        s.metadata["k"] = 2
    with pytest.raises(ValueError, match="shard_index must be < world_size"):
        ReducedShard(shard=0, shard_index=4, shard_numel=3, original_shape=(10,), original_numel=10, world_size=4, reduce="sum")
    with pytest.raises(ValueError, match="padded_numel"):
        ReducedShard(shard=0, shard_index=0, shard_numel=2, original_shape=(10,), original_numel=10, world_size=4, reduce="sum")


# --------------------------------------------------------------------------- #
# caches (reference tests/test_workspace_cache.py)
# --------------------------------------------------------------------------- #
def test_dequantized_workspace_cache_reuses_and_evicts():
    made = []

    def allocator(tensor, shape, config):
        made.append(shape)
        return torch.empty(128)

    cache = DequantizedWorkspaceCache(allocator=allocator, max_entries=1)
    x = torch.ones(100)
    a = cache.get("k0", x, (100,), CFG)
    assert cache.get("k0", x, (100,), CFG) is a and len(made) == 1
    assert cache.get("k0", x, (50, 2), CFG) is not a and len(made) == 2      # layout changed
    cache.get("k1", x, (100,), CFG)
    assert len(cache) == 1
    cache.get("k0", x, (50, 2), CFG)
    assert len(made) == 4                                                    # k0 had been evicted
    with pytest.raises(ValueError):
        DequantizedWorkspaceCache(max_entries=0)
    byte_cache = DequantizedWorkspaceCache(allocator=allocator, max_cached_bytes=600)
    byte_cache.get("a", x, (100,), CFG)
    byte_cache.get("b", x, (100,), CFG)
    assert len(byte_cache) == 1 and byte_cache.cached_bytes == 512


def test_shard_workspace_cache_keys_on_kind_bucket_index_and_layout():
    cache = ShardCommunicationWorkspaceCache(
        quantized_allocator=lambda t, c, d: torch.empty(68, dtype=torch.uint8),
        reduced_allocator=lambda t, s, c: torch.empty(64))
    x = torch.ones(64)
    send0 = cache.get_quantized_chunk("b", 0, x, CFG, dtype="fp32", world_size=2)
    assert cache.get_quantized_chunk("b", 0, x, CFG, dtype="fp32", world_size=2) is send0
    assert cache.get_quantized_chunk("b", 1, x, CFG, dtype="fp32", world_size=2) is not send0
    recv = cache.get_received_payload("b", send0, 0, world_size=2, config=CFG)
    assert recv is not send0 and recv.shape == send0.shape
    red = cache.get_reduced_shard("b", x, (64,), CFG, dtype="fp32", world_size=2, rank=1)
    assert cache.get_reduced_shard("b", x, (64,), CFG, dtype="fp32", world_size=2, rank=1) is red
    assert len(cache) == 4
    cache.clear()
    assert len(cache) == 0 and cache.cached_bytes == 0


# --------------------------------------------------------------------------- #
# bucket processor and hook (reference tests/test_ddp_hook_scaffold.py, tests/test_ddp_comm_hook.py)
# --------------------------------------------------------------------------- #
class Bucket:
    def __init__(self, tensor, index=0):
        self._tensor, self._index = tensor, index

    def buffer(self):
        return self._tensor

    def index(self):
        return self._index


class Future:
    def __init__(self):
        self.value = None

    def set_result(self, value):
        self.value = value


def test_processor_compensates_then_updates_the_residual():
    seen = []

    def quantize(tensor, config):
        seen.append(tensor.values)
        return tensor

    def dequantize(payload, shape, config, dtype):
        return Vec(v - 0.25 for v in payload.values)

    proc = DDPBucketProcessor(config=CompressionConfig(), quantize=quantize, dequantize=dequantize)
    proc.error_feedback.update(0, original=Vec([4.0]), transmitted=Vec([3.25]))
    out = proc.process(Bucket(Vec([10.0])), dtype="fp32")
    assert seen == [(10.75,)] and out == Vec([10.5])
    assert proc.error_feedback.get(0) == Vec([0.25], True, True)
    with pytest.raises(TypeError, match="buffer"):
        proc.process(object(), dtype="fp32")
    plain = DDPBucketProcessor(config=CompressionConfig(error_feedback=False), quantize=quantize, dequantize=dequantize)
    plain.process(Bucket(Vec([1.0])), dtype="fp32")
    assert plain.error_feedback.get(0) is None


def test_all_reduce_hook_wraps_the_result_in_a_future():
    def all_reduce(payload, op):
        assert op == "sum"
        return payload

    hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), dtype="fp32", all_reduce=all_reduce,
                                quantize=lambda t, c: t, dequantize=lambda p, s, c, d: p, future_factory=Future,
                                annotation_provider=lambda: {"state": object})
    fut = hook(None, Bucket(Vec([1.0, 2.0])))
    assert isinstance(fut, Future) and fut.value == Vec([1.0, 2.0])
    assert hook._ccdl_effective_strategy == "all_reduce" and hook.__annotations__ == {"state": object}


def test_all_gather_hook_reduces_in_rank_order_with_error_feedback():
    order = []

    def quantize(tensor, config):
        return {"buffer": tensor, "metadata": {}}

    def all_gather(payload):
        return GatheredPayloads([payload.buffer, torch.full((4,), 3.0)], 2)

    def dequantize(payload, shape, config, dtype):
        order.append(float(payload[0]))
        return payload.reshape(shape)

    state = ErrorFeedbackState()
    hook = create_ddp_comm_hook(CompressionConfig(), strategy="all_gather", reduce="mean", quantize=quantize,
                                dequantize=dequantize, all_gather=all_gather, error_feedback=state,
                                future_factory=Future, annotation_provider=dict)
    out = hook(None, Bucket(torch.full((4,), 1.0), index=7)).value
    assert order == [1.0, 3.0] and torch.equal(out, torch.full((4,), 2.0))
    assert torch.equal(state.get(7), torch.full((4,), -1.0))          # prepared - restored
    out = hook(None, Bucket(torch.full((4,), 1.0), index=7)).value      # residual now applied: prepared = 0
    assert torch.equal(out, torch.full((4,), 1.5))


def test_small_buckets_bypass_compression():
    hook = create_ddp_comm_hook(CompressionConfig(), strategy="all_gather", all_gather=lambda p: 1 / 0,
                                min_compress_numel=100, bypass_all_reduce=lambda t, op: ("raw", op, t),
                                future_factory=Future, annotation_provider=dict)
    tag, op, tensor = hook(None, Bucket(torch.ones(10))).value
    assert (tag, op) == ("raw", "mean") and torch.equal(tensor, torch.ones(10))


def test_strategies_without_an_injected_transport_are_unsupported():
    for name in ("reduce_scatter", "hierarchical", "topology"):
        with pytest.raises(UnsupportedCollective, match=name):
            create_ddp_comm_hook(CompressionConfig(), strategy=name)
    with pytest.raises(UnsupportedCollective, match="ring"):
        create_ddp_comm_hook(CompressionConfig(), strategy="ring")
    with pytest.raises(UnsupportedCollective, match="all_gather"):
        create_ddp_comm_hook(CompressionConfig(), strategy="all_gather")
    with pytest.raises(UnsupportedCollective, match="async_gather"):
        create_ddp_comm_hook(CompressionConfig(), strategy="all_gather", all_gather=lambda p: p, async_gather=True)
    calls = []
    hook = create_ddp_comm_hook(CompressionConfig(), strategy="auto", future_factory=Future, annotation_provider=dict,
                                reduce_scatter_all_gather=lambda t, **kw: calls.append(kw) or "RS")
    assert hook._ccdl_effective_strategy == "reduce_scatter"
    assert hook(None, Bucket(torch.ones(4))).value == "RS"
    assert calls[0]["op"] == "mean" and calls[0]["dtype"] == "fp32" and calls[0]["async_op"] is False


def test_error_feedback_state_checkpoint_round_trip():
    state = ErrorFeedbackState()
    state.put("a", torch.ones(3))
    state.put(7, torch.zeros(2))
    saved = state.state_dict()
    assert sorted(map(str, state.keys())) == ["7", "a"] and len(state) == 2
    other = ErrorFeedbackState()
    other.load_state_dict(saved)
    assert torch.equal(other.get("a"), torch.ones(3)) and other.get(7) is saved[7]


def test_payload_conveniences():
    p = _payload([1, 2, 3, 4], [1.0, 2.0])
    assert p.original_numel == 4
    assert CompressedPayload(buffer=None, shape=(2, 3), dtype="fp32").original_numel == 6
    q = Quantizer(CompressionConfig(), dtype="bf16")
    assert q.payload_bytes(128) == 136 and q.payload_bytes(128, wire_format="native") == 132
    assert "group_size=64" in repr(q)


# --------------------------------------------------------------------------- #
# the native module's launch memo under two threads
# --------------------------------------------------------------------------- #
def test_launch_memo_survives_two_threads_on_a_four_entry_cache():
    """DistributedDataParallel calls the hook from the autograd thread while the script may use the codec from its
    own: lookups, insertions and evictions of the launch memo interleave.  The reference guards its caches with a lock
    (ccdl_comm/cuda/workspace.py:84,149,294; two-thread release test tests/cuda/test_cuda_workspace_pool.py:413-450);
    without one, ``get`` followed by ``move_to_end`` raises KeyError when the other thread's eviction lands between."""
    import threading

    from lowbit_comm_amd.hip.native_module import HipNativeModule

    module = HipNativeModule()
    module.launch_memo_entries = 4

    class Launch:
        def __init__(self, key):
            self.key = key

        def forget_tensors(self):
            return self

    failures, served = [], [0, 0]

    def hammer(who, keys):
        try:
            for i in range(20_000):
                key = ("k", keys[i % len(keys)])
                got = module._memoized(key, lambda key=key: Launch(key))
                assert got.key == key
                served[who] += 1
        except BaseException as failure:      # noqa: BLE001
            failures.append(failure)

    threads = [threading.Thread(target=hammer, args=(0, list(range(7)))),
               threading.Thread(target=hammer, args=(1, list(range(3, 12))))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert failures == [] and served == [20_000, 20_000]
    assert len(module._launches) <= 4
    # a binder that declines (no single launch) stores nothing, one that raises stores nothing either
    before = dict(module._launches)
    assert module._memoized(("none",), lambda: None) is None

    def refuse():
        raise RuntimeError("bad tensor")

    with pytest.raises(RuntimeError, match="bad tensor"):
        module._memoized(("raises",), refuse)
    assert dict(module._launches) == before


def test_reduce_scatter_plan_memo_is_locked_and_sized_for_a_model():
    """The plan's cache of bound launches: same guard, and room for every bucket of a large model (three stages each)."""
    import threading

    from lowbit_comm_amd.hip.reduce_scatter import ReduceScatterPlan

    assert ReduceScatterPlan._BOUND_LAUNCHES >= 3 * 613
    plan = ReduceScatterPlan(64 * 8, torch.float32, world_size=8, rank=0, config=CompressionConfig(), device="cpu")
    plan._BOUND_LAUNCHES = 4

    class Launch:
        def forget_tensors(self):
            return self

    failures = []

    def hammer(keys):
        try:
            for i in range(20_000):
                plan._remember(("q", keys[i % len(keys)]), Launch)
        except BaseException as failure:      # noqa: BLE001
            failures.append(failure)

    threads = [threading.Thread(target=hammer, args=(list(range(7)),)), threading.Thread(target=hammer, args=(list(range(3, 12)),))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert failures == [] and len(plan._bound) <= 4
