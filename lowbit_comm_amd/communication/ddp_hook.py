"""PyTorch DDP communication hook over the compressed bucket path.

``create_ddp_comm_hook`` keeps the keyword surface of the reference's
``ccdl_comm/communication/ddp_hook.py:48-81`` so call sites port unchanged.  What runs here is the
compute of that hook - error-feedback compensate, quantize+pack, fused dequant-reduce, residual
update - on HIP kernels; the collectives themselves are *injected* (``all_gather=``, ``all_reduce=``,
``reduce_scatter_all_gather=``, ``async_all_gather=`` ...).  This build ships no collective transport of
its own: a strategy (or the asynchronous gather) whose transport is not injected raises
:class:`UnsupportedCollective`.
"""
from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass, field
from typing import Any

from lowbit_comm_amd.communication.async_pipeline import AsyncBucketPipeline, chain_after
from lowbit_comm_amd.communication.collectives import CompressedPayload
from lowbit_comm_amd.communication.ddp import DDPBucketProcessor
from lowbit_comm_amd.communication.gather_reduce import CompressedAllGatherReduce, GatheredPayloads
from lowbit_comm_amd.communication.payload_packing import (
    DEFAULT_FUSED_PAYLOAD_MIN_NUMEL,
    make_fused_payload_all_gather,
    should_fuse_payload,
)
from lowbit_comm_amd.communication.workspace import DequantizedWorkspaceCache
from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.exceptions import UnsupportedCollective
from lowbit_comm_amd.quantization.codec import (
    allocate_dequantized_buffer,
    allocate_quantized_buffer,
    dequantize_reduce_tensors,
    dequantize_reduce_update_error_feedback,
    dequantize_tensor,
    inplace_dequantize_reduce_mean_update_error_feedback,
    quantize_tensor,
    writes_prepared,
)
from lowbit_comm_amd.quantization.error_feedback import ErrorFeedbackState
from lowbit_comm_amd.quantization.error_feedback_policy import ErrorFeedbackPolicy

STRATEGIES = ("auto", "all_gather", "all_reduce", "reduce_scatter", "hierarchical", "topology")


@dataclass(frozen=True)
class StrategyPlan:
    """How the requested strategy was resolved (fields of ``ccdl_comm/communication/strategy.py:46-55``).
    The resolution here only looks at which transports were injected; there is no topology planner."""

    requested_strategy: str
    strategy: str
    fallback_strategy: str = "all_gather"
    reason: str = ""
    requires_fallback: bool = False
    capability_flags: dict[str, bool] = field(default_factory=dict)


def _torch_future() -> Any:
    import torch

    return torch.futures.Future()


_TORCH_DTYPE_NAMES = {"torch.bfloat16": "bf16", "torch.float16": "fp16", "torch.float32": "fp32"}


def resolve_dtype(dtype: str, tensor: Any) -> str:
    """``"auto"`` -> ``fp16`` / ``bf16`` / ``fp32`` from the bucket tensor's dtype."""
    if dtype != "auto":
        return dtype
    text = str(getattr(tensor, "dtype", ""))
    known = _TORCH_DTYPE_NAMES.get(text)
    if known is not None:
        return known
    if "bfloat16" in text:
        return "bf16"
    if "float16" in text or text.endswith("half"):
        return "fp16"
    if "float32" in text or text.endswith("float"):
        return "fp32"
    raise ValueError(f"cannot infer CCDL dtype from bucket tensor dtype: {text!r}")


def coerce_payload(value: Any, *, shape: tuple[int, ...], dtype: str) -> CompressedPayload:
    """Accept a :class:`CompressedPayload`, a ``{"buffer": ...}`` dict or a bare buffer from a quantizer."""
    if isinstance(value, CompressedPayload):
        return value
    if isinstance(value, dict) and "buffer" in value:
        return CompressedPayload(buffer=value["buffer"], shape=tuple(value.get("shape", shape)),
                                 dtype=str(value.get("dtype", dtype)), metadata=dict(value.get("metadata", {})))
    return CompressedPayload(buffer=value, shape=shape, dtype=dtype)


def _buffer_of(payload: Any) -> Any:
    return payload.buffer if hasattr(payload, "buffer") else payload


def _numel(tensor: Any) -> int:
    count = getattr(tensor, "numel", None)
    if callable(count):
        return int(count())
    total = 1
    for dim in getattr(tensor, "shape", ()):
        total *= int(dim)
    return total


def _shaped(workspace: Any, shape: tuple[int, ...]) -> Any:
    """First ``prod(shape)`` elements of a (possibly padded) workspace, viewed as ``shape``; objects that cannot
    be reshaped are passed through."""
    if not hasattr(workspace, "reshape"):
        return workspace
    count = 1
    for dim in shape:
        count *= int(dim)
    numel = getattr(workspace, "numel", None)
    if callable(numel) and numel() == count:            # nothing to trim (whole groups): at most one view
        return workspace if tuple(getattr(workspace, "shape", ())) == tuple(shape) else workspace.reshape(shape)
    flat = workspace.reshape((-1,))
    try:
        flat = flat[:count]
    except TypeError:
        pass
    return flat.reshape(shape)


def _single_process_all_reduce(tensor: Any, reduce: str) -> Any:
    """Bypass for uncompressed small buckets when no ``bypass_all_reduce`` is injected: the identity,
    which is the all-reduce of a one-rank world.  With an initialised process group the caller must
    inject the collective."""
    try:
        import torch.distributed as dist

        if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
            raise UnsupportedCollective("all_reduce", reason="inject bypass_all_reduce= for uncompressed buckets; "
                                                             "this build ships no collective transport")
    except ImportError:
        pass
    del reduce
    return tensor


def _annotate(hook: Callable[[Any, Any], Any], provider: Callable[[], dict[str, Any]] | None) -> None:
    def default() -> dict[str, Any]:
        import torch
        import torch.distributed as dist

        return {"state": object, "bucket": dist.GradBucket, "return": torch.futures.Future[torch.Tensor]}

    try:
        hook.__annotations__ = (provider or default)()
    except (ImportError, ModuleNotFoundError, AttributeError):
        pass


def create_ddp_comm_hook(
    config: CompressionConfig,
    *,
    dtype: str = "auto",
    strategy: str = "all_reduce",
    reduce: str = "mean",
    quantize: Callable[[Any, CompressionConfig], Any] | None = None,
    dequantize: Callable[[Any, tuple[int, ...], CompressionConfig, str], Any] | None = None,
    all_reduce: Callable[[CompressedPayload, str], CompressedPayload] | None = None,
    all_gather: Callable[[Any], GatheredPayloads] | None = None,
    async_gather: bool = False,
    async_error_feedback: bool = False,
    synchronize_async_feedback_completion: bool = True,
    async_all_gather: Callable[[Any], Any] | None = None,
    native_error_feedback_update: Callable[[Any, Any, Any], Any] | None = None,
    native_dequantize_reduce_update_feedback: Callable[..., Any] | None = None,
    native_inplace_dequantize_reduce_update_feedback: Callable[..., bool] | None = None,
    reduce_scatter_all_gather: Callable[..., Any] | None = None,
    hierarchical_all_reduce: Callable[..., Any] | None = None,
    topology_all_reduce: Callable[..., Any] | None = None,
    topology_method: str | None = None,
    allocate_dequantized_workspace: Callable[[Any, tuple[int, ...], CompressionConfig], Any] | None = None,
    workspace_cache_max_entries: int | None = 1,
    workspace_cache_max_bytes: int | None = None,
    completion_manager: Any | None = None,
    fuse_payload: bool = False,
    fuse_payload_min_numel: int = DEFAULT_FUSED_PAYLOAD_MIN_NUMEL,
    min_compress_numel: int = 0,
    bypass_all_reduce: Callable[[Any, str], Any] | None = None,
    error_feedback: ErrorFeedbackState | None = None,
    extension_status: Any | None = None,
    future_factory: Callable[[], Any] = _torch_future,
    annotation_provider: Callable[[], dict[str, Any]] | None = None,
) -> Callable[[Any, Any], Any]:
    """Build ``hook(state, bucket) -> Future`` for ``DistributedDataParallel.register_comm_hook``."""
    del topology_method
    requested = strategy.strip().lower()
    if requested not in STRATEGIES:
        raise UnsupportedCollective(strategy, reason="explicit strategy is unknown and no fallback was declared")
    if async_gather and async_all_gather is None:
        raise UnsupportedCollective("async_gather", reason="inject async_all_gather=; this build ships no collective transport")
    injected = {"reduce_scatter": reduce_scatter_all_gather, "hierarchical": hierarchical_all_reduce,
                "topology": topology_all_reduce}
    if requested in injected and injected[requested] is None:
        raise UnsupportedCollective(requested, reason=f"{requested} transport unavailable for explicit strategy")
    effective = requested
    reason = "explicit strategy"
    if requested == "auto":
        effective = "reduce_scatter" if reduce_scatter_all_gather is not None else "all_gather"
        reason = ("a reduce-scatter transport was injected" if effective == "reduce_scatter"
                  else "no reduce-scatter transport was injected")
    plan = StrategyPlan(requested_strategy=requested, strategy=effective, reason=reason,
                        capability_flags={name: fn is not None for name, fn in injected.items()})

    def active_quantize(tensor: Any, active: CompressionConfig) -> Any:
        if quantize is not None:
            return quantize(tensor, active)
        return quantize_tensor(tensor, active, extension_status=extension_status)

    def active_dequantize(payload: Any, shape: tuple[int, ...], active: CompressionConfig, active_dtype: str) -> Any:
        if dequantize is not None:
            return dequantize(payload, shape, active, active_dtype)
        return dequantize_tensor(_buffer_of(payload), shape, active, dtype=active_dtype,
                                 extension_status=extension_status)

    feedback = ErrorFeedbackState() if error_feedback is None else error_feedback
    policy = ErrorFeedbackPolicy(config)
    uncompressed = bypass_all_reduce or _single_process_all_reduce
    inplace_reduce_feedback = (native_inplace_dequantize_reduce_update_feedback
                               or inplace_dequantize_reduce_mean_update_error_feedback)
    combined_reduce_feedback = native_dequantize_reduce_update_feedback or dequantize_reduce_update_error_feedback
    workspaces = DequantizedWorkspaceCache(
        allocator=allocate_dequantized_workspace or allocate_dequantized_buffer,
        max_entries=workspace_cache_max_entries, max_cached_bytes=workspace_cache_max_bytes)
    # With a native module whose fused quantize also writes ``bucket + residual`` the compensate step needs no kernel
    # and no allocation of its own: the sum lands in a cached workspace and the payload in a cached buffer, both
    # under the budgets of the decode workspaces.
    fuse_compensate = quantize is None and writes_prepared(extension_status)
    # Same condition for keeping a bucket's payload buffer from one iteration to the next: a DDP iteration is over
    # (its futures waited for) before the bucket comes back, so the gather has long read the payload.
    reuse_payload_buffers = fuse_compensate
    prepared_workspaces = DequantizedWorkspaceCache(
        allocator=allocate_dequantized_buffer, max_entries=workspace_cache_max_entries,
        max_cached_bytes=workspace_cache_max_bytes)
    payload_buffers = DequantizedWorkspaceCache(
        allocator=lambda tensor, shape, active: allocate_quantized_buffer(tensor.reshape(shape), active,
                                                                         dtype=resolve_dtype("auto", tensor)),
        max_entries=workspace_cache_max_entries, max_cached_bytes=workspace_cache_max_bytes)

    def compensate_and_quantize(key: Any, original: Any) -> tuple[Any, Any] | None:
        """``(bucket + residual, its quantized payload)`` from one launch, or ``None`` when that launch is not to be
        had (no residual yet, another shape, types without a common fused kernel, a policy it declines)."""
        residual = feedback.get(key) if callable(getattr(feedback, "get", None)) else None
        if residual is None or tuple(getattr(residual, "shape", ())) != tuple(original.shape):
            return None
        if not (getattr(original, "is_cuda", False) and original.is_contiguous() and residual.is_contiguous()):
            return None
        like = original if residual.dtype == original.dtype else residual     # the sum has the promoted type
        if str(like.dtype) != "torch.float32" and like.dtype != original.dtype:
            return None
        shape = tuple(original.shape)
        prepared = _shaped(prepared_workspaces.get(key, like, shape, config), shape)
        buffer = payload_buffers.get(key, like, shape, config)
        try:
            quantize_tensor(original, config, extension_status=extension_status, output=buffer, residual=residual,
                            prepared_out=prepared)
        except (ValueError, RuntimeError):
            return None
        return prepared, buffer

    def small(tensor: Any) -> bool:
        return min_compress_numel > 0 and _numel(tensor) < min_compress_numel

    def clone(tensor: Any) -> Any:
        return tensor.clone() if callable(getattr(tensor, "clone", None)) else tensor

    if effective in injected:
        transport = injected[effective]

        # A transport that pipelines the stream of buckets (``transport.pipelined``) returns a future per bucket and
        # holds the last stages of the newest buckets back until the next one arrives; the iteration's last bucket
        # has no next one, so it is followed by a flush.
        flush = getattr(transport, "flush", None) if getattr(transport, "pipelined", False) else None

        def process_bucket(bucket: Any) -> Any:
            tensor = bucket.buffer()
            # a bucket object that cannot say whether it is the last one is treated as the last: correct, unpipelined
            last = callable(flush) and (not callable(getattr(bucket, "is_last", None)) or bucket.is_last())
            if small(tensor):
                if last:
                    flush()
                return uncompressed(clone(tensor), reduce)
            result = transport(tensor, config=config, op=reduce, async_op=False, dtype=resolve_dtype(dtype, tensor),
                               extension_status=extension_status)
            if last:
                flush()
            return result

    elif effective == "all_gather":
        if all_gather is None and not async_gather:
            raise UnsupportedCollective("all_gather", reason="inject all_gather=; this build ships no collective transport")

        def missing_gather(payload: Any) -> Any:
            raise UnsupportedCollective("all_gather", reason="this bucket needs the synchronous gather: inject all_gather=")

        plain_gather = packed_gather = all_gather or missing_gather

        def gather_asynchronously(key: Any, prepared: Any, local: CompressedPayload, shape: tuple[int, ...],
                                  active_dtype: str, decision: Any) -> Any:
            """Start the gather, return the bucket's future, finish when the gather's own future fires
            (ccdl_comm/communication/ddp_hook.py:211-311)."""
            work = async_all_gather(_buffer_of(local))
            outer = future_factory()
            read_residual = getattr(feedback, "get", None)
            residual = read_residual(key) if decision.update and callable(read_residual) else None
            fused_update_done = [False]

            def decode(gathered: Any) -> Any:
                buffers = [_buffer_of(p) for p in gathered.payloads]
                if decision.update and residual is not None:
                    try:
                        workspace = workspaces.get(key, prepared, shape, config)
                        if inplace_reduce_feedback(buffers, prepared, workspace, residual, config,
                                                   extension_status=extension_status, reduce=reduce):
                            fused_update_done[0] = True
                            return _shaped(workspace, shape)
                    except Exception:
                        pass
                    try:
                        restored = combined_reduce_feedback(buffers, prepared, residual, shape, config,
                                                            dtype=active_dtype, extension_status=extension_status,
                                                            reduce=reduce)
                        fused_update_done[0] = True
                        return restored
                    except Exception:
                        pass
                return dequantize_reduce_tensors(buffers, shape, config, dtype=active_dtype,
                                                 extension_status=extension_status, reduce=reduce)

            def update(restored: Any) -> None:
                if not decision.update or fused_update_done[0]:
                    return
                latest = read_residual(key) if callable(read_residual) else None
                if native_error_feedback_update is not None and latest is not None:
                    native_error_feedback_update(prepared, restored, latest)
                else:
                    feedback.update(key, original=prepared, transmitted=restored)

            if decision.apply or decision.update:
                return AsyncBucketPipeline(gather_work=work, future=outer, dequantize_reduce=decode, update_feedback=update,
                                           advance_policy=lambda: policy.advance(key), completion_manager=completion_manager,
                                           synchronize_completion=synchronize_async_feedback_completion).run()

            def complete(_unused: Any = None) -> Any:
                restored = decode(work.wait())
                policy.advance(key)
                outer.set_result(restored)
                return restored

            chain_after(work, complete)
            return outer

        def process_bucket(bucket: Any) -> Any:
            key = bucket.index() if callable(getattr(bucket, "index", None)) else id(bucket)
            original = bucket.buffer()
            if small(original):
                return uncompressed(clone(original), reduce)
            decision = policy.decide(key, numel=_numel(original))
            facade = dequantize is None and reduce in ("mean", "sum")
            fused = compensate_and_quantize(key, original) if decision.apply and facade and fuse_compensate else None
            if fused is not None:
                prepared = fused[0]
            else:
                prepared = feedback.compensate(key, original) if decision.apply else original
            active_dtype = resolve_dtype(dtype, prepared)
            shape = tuple(prepared.shape)
            gather = (packed_gather if should_fuse_payload(prepared, enabled=fuse_payload,
                                                           min_numel=fuse_payload_min_numel) else plain_gather)
            if facade:
                # facade path: flat uint8 buffers, fused decode+reduce (+ residual update) on the GPU
                if fused is not None:
                    packed = fused[1]
                elif reuse_payload_buffers and getattr(prepared, "is_cuda", False) and prepared.is_contiguous():
                    # the bucket's payload goes into the buffer its key had last iteration: nothing is allocated and
                    # the native module meets the addresses it has bound launches for
                    packed = quantize_tensor(prepared, config, extension_status=extension_status,
                                             output=payload_buffers.get(key, prepared, shape, config))
                else:
                    packed = active_quantize(prepared, config)
                local = coerce_payload(packed, shape=shape, dtype=active_dtype)
                needs_feedback = decision.apply or decision.update
                if async_gather and (async_error_feedback or not needs_feedback):
                    return gather_asynchronously(key, prepared, local, shape, active_dtype, decision)
                buffers = [_buffer_of(p) for p in gather(local).payloads]
                restored = None
                residual = feedback.get(key) if decision.update and callable(getattr(feedback, "get", None)) else None
                if residual is not None and getattr(residual, "dtype", None) == getattr(prepared, "dtype", None):
                    workspace = workspaces.get(key, prepared, shape, config)
                    try:
                        if inplace_reduce_feedback(buffers, prepared, workspace, residual, config,
                                                   extension_status=extension_status, reduce=reduce):
                            restored = _shaped(workspace, shape)
                    except RuntimeError:
                        restored = None
                if restored is None:
                    restored = dequantize_reduce_tensors(buffers, shape, config, dtype=active_dtype,
                                                         extension_status=extension_status, reduce=reduce)
                    if decision.update:
                        latest = feedback.get(key) if callable(getattr(feedback, "get", None)) else None
                        if native_error_feedback_update is not None and latest is not None:
                            native_error_feedback_update(prepared, restored, latest)
                        else:
                            feedback.update(key, original=prepared, transmitted=restored)
                policy.advance(key)
                return restored
            collective = CompressedAllGatherReduce(
                config=config,
                compress=lambda tensor, active: coerce_payload(active_quantize(tensor, active),
                                                               shape=tuple(tensor.shape), dtype=active_dtype),
                all_gather=gather,
                decompress=active_dequantize,
            )
            restored = collective.run(prepared, shape=shape, dtype=active_dtype, reduce=reduce)
            if decision.update:
                feedback.update(key, original=prepared, transmitted=restored)
            policy.advance(key)
            return restored

    else:  # all_reduce
        if all_reduce is None:
            raise UnsupportedCollective("all_reduce", reason="inject all_reduce=; this build ships no collective transport")
        processor = DDPBucketProcessor(config=config, quantize=active_quantize, dequantize=active_dequantize,
                                       all_reduce=all_reduce, error_feedback=feedback)

        def process_bucket(bucket: Any) -> Any:
            tensor = bucket.buffer()
            if small(tensor):
                return uncompressed(clone(tensor), reduce)
            return processor.process(bucket, dtype=resolve_dtype(dtype, tensor))

    def hook(state: Any, bucket: Any) -> Any:
        del state
        result = process_bucket(bucket)
        if hasattr(result, "set_result"):
            return result
        future = future_factory()
        future.set_result(result)
        return future

    hook._ccdl_strategy_plan = plan
    hook._ccdl_requested_strategy = requested
    hook._ccdl_effective_strategy = effective
    _annotate(hook, annotation_provider)
    return hook


def make_fused_all_gather(byte_all_gather: Callable[[Any], GatheredPayloads]):
    """Convenience re-export: wrap a byte all-gather so payloads travel packed (one collective per bucket)."""
    return make_fused_payload_all_gather(byte_all_gather)

