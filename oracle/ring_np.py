"""CPU oracle (numpy) for the quantized ring and tree all-reduce.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this module; the product never
routes through it.

Reference lines each function follows (paths under the upstream repository):

* ``ring_step``        ccdl_comm/cuda/transports/torch_topology.py:262-316 (``fused_reduce``: dequantize with
                       reduce_op "sum" into the chunk view, ``div_(world_size)`` once all other ranks have
                       contributed; ``apply_broadcast``: dequantize with reduce_op "none") followed by
                       ``quant_pack`` of the same view (:236-240, the codec of
                       ccdl_comm/quantization/torch_fallback.py:24-36)
* ``PortableCodec`` / ``CudaWireCodec``
                       what ``quantize_tensor`` / ``dequantize_tensor`` compute in the two payload formats (the
                       restatements of oracle/codec_np.py and oracle/cuda_wire_general_np.py)
* ``ring_all_reduce``  ccdl_comm/cuda/transports/pipelined_ring.py:216-275 (the order of quantize, exchange and
                       reduce on every rank) with chunk views ``tensor.reshape(-1)[start:stop]``
                       (torch_topology.py:418-419) of the plan of
                       ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94

* ``tree_edges`` / ``tree_all_reduce``
                       ccdl_comm/cuda/transports/tree.py:196-306 and torch_topology.py:319-415

``ring_all_reduce`` does not restate the schedule compiler's index formulas (pipelined_ring.py:298-331).  It
passes messages: every rank sends to its successor the chunk it has just received into, starting with the
chunk of its predecessor's index, which is the one rule under which rank r ends the first W-1 steps holding the
complete chunk r.  The product's compiled schedule is tested against this simulation.

Pinning (tests/test_ring_oracle.py): ``ring_step`` against Python-float brute force on tiny inputs and against
the composition of the separately pinned ``dequantize`` / ``quantize``; ``ring_all_reduce`` on inputs built so
that every quantization on the way is lossless, where the result must equal the exact mean on every rank (a
wrong peer, chunk, contributor count or a second division fails it), on world sizes 1 to 8 with ragged and
empty chunks, and against the error bound of W-1 successive quantizations on random inputs; ``tree_edges`` against
the edge list the reference's test spells out for five ranks and the properties it states for every root (each
rank once, connected, acyclic), ``tree_all_reduce`` on the same lossless construction and by following the mean
down the levels.
"""
from __future__ import annotations

import numpy as np

from oracle import codec_np


class PortableCodec:
    """The portable payload ``(int8 codes, fp32 scales)`` and the CPU codec's arithmetic: decode rounded to the
    chunk's type, sum in that type, true division (ccdl_comm/quantization/torch_fallback.py:24-53)."""

    def __init__(self, group_size: int = 64) -> None:
        self.group_size = group_size

    def quantize(self, chunk: np.ndarray, dtype: str):
        return codec_np.quantize(codec_np.widen(chunk, dtype), self.group_size)

    def decode_into(self, payload, chunk: np.ndarray, dtype: str, reduce_op: str) -> np.ndarray:
        decoded = codec_np.widen(codec_np.dequantize(payload[0], payload[1], int(chunk.size), self.group_size, dtype),
                                 dtype)
        if reduce_op == "none":
            return codec_np.narrow(decoded, dtype)
        with np.errstate(invalid="ignore", over="ignore"):
            return codec_np.narrow(codec_np.widen(chunk, dtype) + decoded, dtype)

    def divide(self, chunk: np.ndarray, dtype: str, divisor: float) -> np.ndarray:
        with np.errstate(invalid="ignore", over="ignore"):
            return codec_np.narrow(codec_np.widen(chunk, dtype) / np.float32(divisor), dtype)


class CudaWireCodec:
    """The byte format and arithmetic of the reference's CUDA extension for any of its policies
    (oracle/cuda_wire_general_np.py); the in-place division is the one ``tensor.div_(int)`` performs on a GPU
    tensor, a multiplication by the float32 reciprocal (torch_topology.py:287-289 runs it on the device)."""

    def __init__(self, group_size: int = 64, *, bit: int = 8, quant_type: str = "linear", topk: int = 0,
                 compact: bool = False) -> None:
        self.group_size, self.bit, self.quant_type, self.topk, self.compact = group_size, bit, quant_type, topk, compact

    def quantize(self, chunk: np.ndarray, dtype: str):
        from oracle import cuda_wire_general_np as general

        return general.quantize(chunk, dtype, self.group_size, self.bit, self.quant_type, self.topk, None,
                                self.compact)

    def decode_into(self, payload, chunk: np.ndarray, dtype: str, reduce_op: str) -> np.ndarray:
        from oracle import cuda_wire_general_np as general

        return general.dequantize(payload, int(chunk.size), dtype, self.group_size, self.bit, self.quant_type,
                                  self.topk, self.compact, reduce_op=reduce_op, out=chunk)

    def divide(self, chunk: np.ndarray, dtype: str, divisor: float) -> np.ndarray:
        reciprocal = np.float32(1.0) / np.float32(divisor)
        with np.errstate(invalid="ignore", over="ignore"):
            return codec_np.narrow(codec_np.widen(chunk, dtype) * reciprocal, dtype)


def ring_step(received, chunk: np.ndarray, dtype: str, group_size: int = 64, *, reduce_op: str = "sum",
              divisor: float = 1.0, emit: bool = True, codec=None):
    """One compute step on one chunk.  ``received`` is a payload of ``codec`` (portable: ``(codes, scales)``)
    covering ``chunk.size`` elements; ``chunk`` holds values of ``dtype`` (bf16 as uint16 bit patterns).
    Returns ``(new_chunk, payload | None)``."""
    if reduce_op not in ("sum", "none"):
        raise ValueError(f"unsupported reduce op {reduce_op!r}")
    codec = codec or PortableCodec(group_size)
    value = codec.decode_into(received, chunk, dtype, reduce_op)
    if divisor != 1.0:
        value = codec.divide(value, dtype, divisor)
    return value, (codec.quantize(value, dtype) if emit else None)


def ring_all_reduce(buckets, dtype: str, group_size: int = 64, trace: list | None = None, codec=None):
    """Mean all-reduce of ``W = len(buckets)`` equally sized flat buckets of ``dtype`` over a ring, every rank
    simulated on the host.  Returns the W result buckets (they differ between ranks: a rank keeps the unquantized
    mean of its own chunk and the decoded payloads of the others).  ``trace``, when given, receives one
    ``(phase, step, rank, sent_chunk, received_from, received_chunk)`` tuple per rank and step."""
    codec = codec or PortableCodec(group_size)
    world = len(buckets)
    tensors = [np.array(b, copy=True).reshape(-1) for b in buckets]
    n = int(tensors[0].size)
    shard, _padded, ranges = codec_np.chunk_plan(n, world)
    views = [(min(a, n), min(b, n)) for a, b in ranges]          # slicing clamps to the tensor's end

    def quantize_chunk(rank: int, index: int):
        a, b = views[index]
        return codec.quantize(tensors[rank][a:b], dtype)

    carried = [(rank - 1) % world for rank in range(world)]       # chunk each rank sends next
    for phase in ("reduce", "gather"):
        for step in range(world - 1):
            sent = [(carried[rank], quantize_chunk(rank, carried[rank])) for rank in range(world)]
            for rank in range(world):
                source = (rank - 1) % world
                index, payload = sent[source]
                a, b = views[index]
                last_reduce = phase == "reduce" and step == world - 2
                new_chunk, _ = ring_step(payload, tensors[rank][a:b], dtype, group_size,
                                         reduce_op="sum" if phase == "reduce" else "none",
                                         divisor=float(world) if last_reduce else 1.0, emit=False, codec=codec)
                tensors[rank][a:b] = new_chunk
                if trace is not None:
                    trace.append((phase, step, rank, sent[rank][0], source, index))
                carried[rank] = index
    return tensors


def tree_edges(world: int, root: int = 0):
    """``(child, parent)`` pairs of the reference's tree (ccdl_comm/cuda/transports/tree.py:297-306): the ranks
    form a binary heap counted from the root, and the edges are listed from the last heap position up to the
    root's first child, so a rank's own children come before its edge to its parent."""
    at = [(root + position) % world for position in range(world)]
    return [(at[position], at[(position - 1) // 2]) for position in range(world - 1, 0, -1)]


def tree_all_reduce(buckets, dtype: str, group_size: int = 64, codec=None, root: int = 0):
    """Mean all-reduce over that tree, every rank simulated on the host (TreeExecutor,
    ccdl_comm/cuda/transports/tree.py:196-281, with TorchTreeRuntime, torch_topology.py:319-415): each edge carries
    the child's whole bucket, quantized, to the parent, which adds it in the bucket's type; the root divides by W
    before its first send down; the mean descends the edges in reverse order, quantized again at every level.
    The root keeps the unquantized mean."""
    codec = codec or PortableCodec(group_size)
    world = len(buckets)
    tensors = [np.array(b, copy=True).reshape(-1) for b in buckets]
    edges = tree_edges(world, root)
    for child, parent in edges:
        tensors[parent] = codec.decode_into(codec.quantize(tensors[child], dtype), tensors[parent], dtype, "sum")
    if edges:
        tensors[root] = codec.divide(tensors[root], dtype, float(world))
    for child, parent in reversed(edges):
        tensors[child] = codec.decode_into(codec.quantize(tensors[parent], dtype), tensors[child], dtype, "none")
    return tensors
