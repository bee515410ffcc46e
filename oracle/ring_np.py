"""CPU oracle (numpy) for the quantized ring all-reduce.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this module; the product never
routes through it.

Reference lines each function follows (paths under the upstream repository):

* ``ring_step``        ccdl_comm/cuda/transports/torch_topology.py:262-316 (``fused_reduce``: dequantize with
                       reduce_op "sum" into the chunk view, ``div_(world_size)`` once all other ranks have
                       contributed; ``apply_broadcast``: dequantize with reduce_op "none") followed by
                       ``quant_pack`` of the same view (:236-240, the codec of
                       ccdl_comm/quantization/torch_fallback.py:24-36)
* ``ring_all_reduce``  ccdl_comm/cuda/transports/pipelined_ring.py:216-275 (the order of quantize, exchange and
                       reduce on every rank) with chunk views ``tensor.reshape(-1)[start:stop]``
                       (torch_topology.py:418-419) of the plan of
                       ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94

``ring_all_reduce`` does not restate the schedule compiler's index formulas (pipelined_ring.py:298-331).  It
passes messages: every rank sends to its successor the chunk it has just received into, starting with the
chunk of its predecessor's index, which is the one rule under which rank r ends the first W-1 steps holding the
complete chunk r.  The product's compiled schedule is tested against this simulation.

Pinning (tests/test_ring_oracle.py): ``ring_step`` against Python-float brute force on tiny inputs and against
the composition of the separately pinned ``dequantize`` / ``quantize``; ``ring_all_reduce`` on inputs built so
that every quantization on the way is lossless, where the result must equal the exact mean on every rank (a
wrong peer, chunk, contributor count or a second division fails it), on world sizes 1 to 8 with ragged and
empty chunks, and against the error bound of W-1 successive quantizations on random inputs.
"""
from __future__ import annotations

import numpy as np

from oracle import codec_np


def ring_step(received, chunk: np.ndarray, dtype: str, group_size: int = 64, *, reduce_op: str = "sum",
              divisor: float = 1.0, emit: bool = True):
    """One compute step on one chunk.  ``received`` = ``(codes, scales)`` covering ``chunk.size`` elements;
    ``chunk`` holds values of ``dtype`` (bf16 as uint16 bit patterns).  Returns ``(new_chunk, payload | None)``."""
    if reduce_op not in ("sum", "none"):
        raise ValueError(f"unsupported reduce op {reduce_op!r}")
    n = int(chunk.size)
    decoded = codec_np.widen(codec_np.dequantize(received[0], received[1], n, group_size, dtype), dtype)
    with np.errstate(invalid="ignore", over="ignore"):
        if reduce_op == "sum":
            value = codec_np._round_through(codec_np.widen(chunk, dtype) + decoded, dtype)
        else:
            value = decoded
        if divisor != 1.0:
            value = codec_np._round_through(value / np.float32(divisor), dtype)
    payload = codec_np.quantize(value, group_size) if emit else None
    return codec_np.narrow(value, dtype), payload


def ring_all_reduce(buckets, dtype: str, group_size: int = 64, trace: list | None = None):
    """Mean all-reduce of ``W = len(buckets)`` equally sized flat buckets of ``dtype`` over a ring, every rank
    simulated on the host.  Returns the W result buckets (they differ between ranks: a rank keeps the unquantized
    mean of its own chunk and the decoded payloads of the others).  ``trace``, when given, receives one
    ``(phase, step, rank, sent_chunk, received_from, received_chunk)`` tuple per rank and step."""
    world = len(buckets)
    tensors = [np.array(b, copy=True).reshape(-1) for b in buckets]
    n = int(tensors[0].size)
    shard, _padded, ranges = codec_np.chunk_plan(n, world)
    views = [(min(a, n), min(b, n)) for a, b in ranges]          # slicing clamps to the tensor's end

    def quantize_chunk(rank: int, index: int):
        a, b = views[index]
        return codec_np.quantize(codec_np.widen(tensors[rank][a:b], dtype), group_size)

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
                                         divisor=float(world) if last_reduce else 1.0, emit=False)
                tensors[rank][a:b] = new_chunk
                if trace is not None:
                    trace.append((phase, step, rank, sent[rank][0], source, index))
                carried[rank] = index
    return tensors
