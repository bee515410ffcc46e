"""One flat ``uint8`` tensor per payload: buffer bytes first, then tensor-valued metadata in sorted key
order (layout of ``ccdl_comm/communication/payload_packing.py:26-75``).  For the linear INT8 codec
that is ``[int8 codes || fp32 scales]`` - exactly what the HIP quantizer writes when handed a packed
buffer, so packing a payload produced that way is a view, not a copy.
"""
from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass
from typing import Any

from lowbit_comm_amd.communication.collectives import CompressedPayload
from lowbit_comm_amd.communication.gather_reduce import GatheredPayloads

DEFAULT_FUSED_PAYLOAD_MIN_NUMEL = 4_000_000


@dataclass(frozen=True)
class TensorFieldSchema:
    """Where one tensor lives inside the packed bytes."""

    name: str
    dtype: Any
    shape: tuple[int, ...]
    numel: int
    byte_count: int
    offset: int


def _looks_like_tensor(value: Any) -> bool:
    return all(hasattr(value, attr) for attr in ("shape", "dtype", "numel"))


def _field(name: str, tensor: Any, offset: int) -> TensorFieldSchema:
    flat = tensor.contiguous() if callable(getattr(tensor, "contiguous", None)) else tensor
    count = int(flat.numel())
    return TensorFieldSchema(name=name, dtype=flat.dtype, shape=tuple(flat.shape), numel=count,
                             byte_count=count * int(flat.element_size()), offset=offset)


def _bytes_of(tensor: Any) -> Any:
    import torch

    flat = tensor.contiguous() if callable(getattr(tensor, "contiguous", None)) else tensor
    return flat.view(torch.uint8).reshape(-1)


def _is_view_of_packed(payload: CompressedPayload, fields: tuple[TensorFieldSchema, ...]) -> Any | None:
    """The packed tensor itself when buffer and metadata are adjacent views of that one allocation, each at its
    offset in the schema (a :class:`~lowbit_comm_amd.communication.collectives.PackedPayload` as the quantizer made
    it).  A payload whose buffer or metadata were replaced since (``dataclasses.replace``, an edited metadata
    dict) no longer passes and is packed by copying."""
    packed = getattr(payload, "packed", None)
    if packed is None or int(packed.numel()) != sum(f.byte_count for f in fields):
        return None
    base = packed.data_ptr()
    for f in fields:
        piece = payload.buffer if f.name == "buffer" else payload.metadata.get(f.name)
        if not _looks_like_tensor(piece) or not callable(getattr(piece, "data_ptr", None)):
            return None
        contiguous = getattr(piece, "is_contiguous", None)
        if callable(contiguous) and not contiguous():
            return None
        if piece.data_ptr() != base + f.offset or int(piece.numel()) * int(piece.element_size()) != f.byte_count:
            return None
    return packed


@dataclass(frozen=True)
class FusedPayloadPacker:
    """Pack / unpack against a schema frozen from the first payload seen."""

    buffer_schema: TensorFieldSchema
    metadata_schemas: tuple[TensorFieldSchema, ...]
    scalar_metadata: dict[str, Any]

    @classmethod
    def from_payload(cls, payload: CompressedPayload) -> "FusedPayloadPacker":
        items = dict(payload.metadata)
        tensors = {k: v for k, v in items.items() if _looks_like_tensor(v)}
        if not tensors:
            raise ValueError("fused payload all-gather requires tensor metadata")
        head = _field("buffer", payload.buffer, 0)
        cursor = head.byte_count
        fields = []
        for key in sorted(tensors):
            fields.append(_field(key, tensors[key], cursor))
            cursor += fields[-1].byte_count
        scalars = {k: v for k, v in items.items() if k not in tensors}
        return cls(buffer_schema=head, metadata_schemas=tuple(fields), scalar_metadata=scalars)

    @property
    def packed_bytes(self) -> int:
        return self.buffer_schema.byte_count + sum(f.byte_count for f in self.metadata_schemas)

    def pack(self, payload: CompressedPayload) -> Any:
        already = _is_view_of_packed(payload, (self.buffer_schema,) + self.metadata_schemas)
        if already is not None:
            return already
        import torch

        pieces = [_bytes_of(payload.buffer)]
        pieces += [_bytes_of(payload.metadata[f.name]) for f in self.metadata_schemas]
        return torch.cat(pieces, dim=0)

    def unpack(self, packed: Any, *, shape: tuple[int, ...], dtype: str) -> CompressedPayload:
        def piece(f: TensorFieldSchema) -> Any:
            return packed.narrow(0, f.offset, f.byte_count).view(f.dtype).reshape(f.shape)

        metadata = dict(self.scalar_metadata)
        for f in self.metadata_schemas:
            metadata[f.name] = piece(f)
        return CompressedPayload(buffer=piece(self.buffer_schema), shape=shape, dtype=dtype, metadata=metadata)


@dataclass(frozen=True)
class FusedPayloadAllGather:
    """``payload -> pack -> byte all-gather -> unpack each``."""

    byte_all_gather: Callable[[Any], GatheredPayloads]
    packer: FusedPayloadPacker
    shape: tuple[int, ...]
    dtype: str

    def __call__(self, payload: CompressedPayload) -> GatheredPayloads:
        gathered = self.byte_all_gather(self.packer.pack(payload))
        return GatheredPayloads(
            payloads=[self.packer.unpack(p, shape=self.shape, dtype=self.dtype) for p in gathered.payloads],
            world_size=gathered.world_size,
        )


class _DeferredPacker:
    """``.pack`` that builds the schema from the first payload it sees (shared with the gather closure)."""

    def __init__(self, slot: dict[str, FusedPayloadPacker]) -> None:
        self._slot = slot

    def resolve(self, payload: CompressedPayload) -> FusedPayloadPacker:
        if "packer" not in self._slot:
            self._slot["packer"] = FusedPayloadPacker.from_payload(payload)
        return self._slot["packer"]

    def pack(self, payload: CompressedPayload) -> Any:
        return self.resolve(payload).pack(payload)


def make_fused_payload_all_gather(byte_all_gather: Callable[[Any], GatheredPayloads]):
    """All-gather adapter that moves buffer + tensor metadata as one byte tensor (one collective)."""
    deferred = _DeferredPacker({})

    def fused_payload_all_gather(payload: CompressedPayload) -> GatheredPayloads:
        adapter = FusedPayloadAllGather(byte_all_gather=byte_all_gather, packer=deferred.resolve(payload),
                                        shape=payload.shape, dtype=payload.dtype)
        return adapter(payload)

    fused_payload_all_gather.packer = deferred  # type: ignore[attr-defined]
    return fused_payload_all_gather


def make_payload_all_gather(buffer_all_gather: Callable[[Any], GatheredPayloads]):
    """All-gather adapter that gathers the buffer and every tensor metadata item separately."""

    def payload_all_gather(payload: CompressedPayload) -> GatheredPayloads:
        buffers = buffer_all_gather(payload.buffer)
        world = buffers.world_size
        per_key: dict[str, list[Any]] = {}
        for key, value in dict(payload.metadata).items():
            if hasattr(value, "shape") and hasattr(value, "dtype"):
                per_key[key] = list(buffer_all_gather(value).payloads)
            else:
                per_key[key] = [value] * world
        return GatheredPayloads(
            payloads=[
                CompressedPayload(buffer=buf, shape=payload.shape, dtype=payload.dtype,
                                  metadata={k: vals[i] for k, vals in per_key.items()})
                for i, buf in enumerate(buffers.payloads)
            ],
            world_size=world,
        )

    return payload_all_gather


def should_fuse_payload(tensor: Any, *, enabled: bool, min_numel: int = DEFAULT_FUSED_PAYLOAD_MIN_NUMEL) -> bool:
    """Fuse when enabled and the tensor has at least ``min_numel`` elements (always, if ``min_numel <= 0``)."""
    if not enabled:
        return False
    if min_numel <= 0:
        return True
    numel = getattr(tensor, "numel", None)
    if callable(numel):
        return int(numel()) >= min_numel
    shape = getattr(tensor, "shape", None)
    if shape is None:
        return False
    total = 1
    for dim in shape:
        total *= int(dim)
    return total >= min_numel
