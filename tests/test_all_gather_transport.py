"""GPU tests of the all-gather form of the compressed all-reduce (``make_all_gather_transport``, ``AllGatherPlan``): a
stream of buckets must leave, bit for bit, what the CPU oracle computes for quantize -> gather -> reduce in rank order
(the data path of the reference hook's all_gather strategy, ccdl_comm/communication/ddp_hook.py:190-330), pipelined or
not, with one launch per bucket when pipelined (counted with torch.profiler), also through ``create_ddp_comm_hook``.

The gather is a stand-in on the one GPU: row 0 receives this rank's payload, the other rows hold the payloads of W - 1
peers whose buckets are this rank's bucket times a per-rank factor, quantized by the library beforehand."""
import pytest
import torch

from lowbit_comm_amd import CompressionConfig
from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
from oracle import codec_torch

pytestmark = pytest.mark.gpu
CFG = CompressionConfig()
G = 64
NAMES = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}


def grad(n, dtype, seed, dev, sigma=1e-3):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=gen) * sigma).to(dtype).to(dev)


def same_bits(a, b):
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    assert a.dtype == b.dtype and a.shape == b.shape, (a.dtype, b.dtype, a.shape, b.shape)
    view = torch.int32 if a.dtype == torch.float32 else torch.int16
    return torch.equal(a.view(view), b.view(view))


class Peers:
    """The other ranks of the gather: for a payload of a given size, W - 1 payloads made from seeded tensors."""

    def __init__(self, world, dtype, dev):
        self.world, self.dtype, self.dev = world, dtype, dev
        self.tensors = {}                 # element count -> the peers' buckets (CPU copies for the oracle)
        self.numel_of = {}                # payload bytes -> element count

    def expect(self, n):
        from lowbit_comm_amd.hip import ops

        if n not in self.tensors:
            self.tensors[n] = [grad(n, self.dtype, 4000 + 7 * r + n % 97, self.dev) for r in range(1, self.world)]
            self.numel_of[ops.payload_nbytes(n, G)] = n

    def all_gather(self, received, mine):
        from lowbit_comm_amd.hip import ops

        n = self.numel_of[mine.numel()]
        assert mine.data_ptr() == received.data_ptr()          # this rank's payload already lies in its row (rank 0)
        for r, tensor in enumerate(self.tensors[n], start=1):
            assert ops.quant_pack_payload_into(tensor, received[r, :mine.numel()], group_size=G)


def oracle(bucket_cpu, residual_cpu, peers_cpu, op):
    """(reduced bucket, new residual) of quantize -> gather -> reduce in rank order, this rank being rank 0."""
    n, name = bucket_cpu.numel(), NAMES[bucket_cpu.dtype]
    prepared = bucket_cpu if residual_cpu is None else bucket_cpu + residual_cpu
    codes, scales = codec_torch.quantize(prepared, G)
    dropped = prepared - codec_torch.dequantize(codes, scales, n, G, "fp32") if residual_cpu is not None else None
    payloads = [(codes, scales)] + [codec_torch.quantize(t, G) for t in peers_cpu]
    return codec_torch.reduce_payloads(payloads, n, G, name, op), dropped


def kernel_counts(run):
    from torch.profiler import ProfilerActivity, profile

    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        run()
        torch.cuda.synchronize()
    counts = {}
    for event in prof.events():
        if event.device_type == torch.autograd.DeviceType.CUDA:
            counts[event.name] = counts.get(event.name, 0) + 1
    return counts


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("error_feedback", [False, True])
@pytest.mark.parametrize("world,lanes,pipelined", [(8, 1, True), (8, 2, True), (4, 1, True), (3, 1, True), (1, 1, True),
                                                   (8, 1, False), (2, 1, False)])
@pytest.mark.parametrize("op", ["mean", "sum"])
def test_all_gather_transport_equals_the_oracle(hip_device, dtype, error_feedback, world, lanes, pipelined, op):
    from lowbit_comm_amd.hip.reduce_scatter import make_all_gather_transport

    sizes = [G * 320, G * 320, G * 191, 70_001, G * 320, 640, G * 8 * 64 * 3 + 24]
    peers = Peers(world, dtype, hip_device)
    for n in sizes:
        peers.expect(n)
    transport = make_all_gather_transport(world_size=world, rank=0, all_gather=peers.all_gather, pipelined=pipelined,
                                          lanes=lanes, error_feedback=error_feedback)
    assert transport.pipelined is pipelined
    buckets = [torch.empty(n, dtype=dtype, device=hip_device) for n in sizes]
    residuals = [torch.zeros(n) if error_feedback else None for n in sizes]
    for step in range(3):                         # residuals carry over, plans and bound launches are met again
        inputs = []
        for k, bucket in enumerate(buckets):
            bucket.copy_(grad(bucket.numel(), dtype, 5000 + 10 * step + k, hip_device))
            inputs.append(bucket.cpu())
        results = [transport(bucket, config=CFG, op=op) for bucket in buckets]
        if pipelined:
            transport.flush()
            results = [future.wait() for future in results]
        torch.cuda.synchronize()
        for k, (bucket, result) in enumerate(zip(buckets, results)):
            want, dropped = oracle(inputs[k], residuals[k], [t.cpu() for t in peers.tensors[bucket.numel()]], op)
            assert result.data_ptr() == bucket.data_ptr(), "reduced in place"
            assert same_bits(result, want), f"step {step} bucket {k} ({bucket.numel()} elements)"
            if error_feedback:
                residuals[k] = dropped
                assert same_bits(transport.residuals.for_tensor(bucket), dropped), f"step {step} residual {k}"


def test_pipelined_all_gather_transport_launches_once_per_bucket(hip_device):
    from lowbit_comm_amd.hip.reduce_scatter import make_all_gather_transport

    world, n, count = 8, G * 8 * 640, 12
    peers = Peers(world, torch.bfloat16, hip_device)
    peers.expect(n)
    transport = make_all_gather_transport(world_size=world, rank=0, all_gather=peers.all_gather, error_feedback=True,
                                          pipelined=True)
    buckets = [grad(n, torch.bfloat16, 6000 + k, hip_device) for k in range(count)]

    def iteration():
        for bucket in buckets:
            transport(bucket, config=CFG, op="mean")
        transport.flush()

    iteration()                                   # plans, residuals and bound launches exist from here on
    counts = kernel_counts(iteration)
    shared = sum(v for name, v in counts.items() if "bucket_step_kernel" in name)
    alone = sum(v for name, v in counts.items() if "quant_pack_kernel" in name and "bucket_step" not in name)
    reduces = sum(v for name, v in counts.items() if "dequant_reduce_kernel" in name)
    assert shared == count - 1 and alone == count * (world - 1) + 1 and reduces == 1, counts
    assert transport.pipeline.stats["merged_launches"] == 2 * (count - 1)


@pytest.mark.parametrize("error_feedback", [False, True])
@pytest.mark.parametrize("pipelined", [True, False])
def test_all_gather_transport_behind_the_comm_hook(hip_device, error_feedback, pipelined):
    """The transport under ``strategy="topology"``: the hook hands every bucket over, flushes after the last one, and
    every future holds what the oracle computes."""
    from lowbit_comm_amd.hip.reduce_scatter import make_all_gather_transport

    class Bucket:
        def __init__(self, tensor, index, last):
            self._tensor, self._index, self._last = tensor, index, last

        def buffer(self):
            return self._tensor

        def index(self):
            return self._index

        def is_last(self):
            return self._last

    world, sizes = 8, [G * 8 * 80, G * 8 * 80, 70_001, G * 8 * 80]
    peers = Peers(world, torch.bfloat16, hip_device)
    for n in sizes:
        peers.expect(n)
    transport = make_all_gather_transport(world_size=world, rank=0, all_gather=peers.all_gather, error_feedback=error_feedback,
                                          pipelined=pipelined)
    hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), strategy="topology", reduce="mean",
                                topology_all_reduce=transport)
    buckets = [grad(n, torch.bfloat16, 6100 + k, hip_device) for k, n in enumerate(sizes)]
    inputs = [b.cpu() for b in buckets]
    futures = [hook(None, Bucket(b, k, k == len(buckets) - 1)) for k, b in enumerate(buckets)]
    torch.cuda.synchronize()
    for k, future in enumerate(futures):
        assert future.done()
        want, _ = oracle(inputs[k], torch.zeros(sizes[k]) if error_feedback else None,
                         [t.cpu() for t in peers.tensors[sizes[k]]], "mean")
        assert same_bits(future.value().reshape(-1), want), f"bucket {k}"


def test_all_gather_plan_refuses_the_steps_of_the_other_form(hip_device):
    """The plan inherits the reduce-scatter plan's buffers and steps only as far as they apply: the reduce needs an
    output from the caller (the plan keeps none), and the second leg's steps say that they do not exist here."""
    from lowbit_comm_amd.hip.reduce_scatter import AllGatherPlan

    n, world, rank = 64 * 40 + 17, 3, 1
    plan = AllGatherPlan(n, torch.float32, world_size=world, rank=rank, config=CompressionConfig(), device=hip_device)
    with pytest.raises(ValueError, match="pass out="):
        plan.reduce_received(op="sum")
    with pytest.raises(ValueError, match="pass out="):
        plan.bound_reduce(op="sum")
    for step in (plan.requantize_shard, plan.reduce_and_requantize, plan.bound_reduce_requantize, plan.decode_gathered):
        with pytest.raises(TypeError, match="no requantize"):
            step()
    with pytest.raises(TypeError, match="no requantize"):
        plan.bound_decode(torch.empty(n, device=hip_device))

    # and the steps that do apply still give the oracle's result
    bucket = grad(n, torch.float32, 31, hip_device)
    peers = {r: grad(n, torch.float32, 40 + r, hip_device) for r in range(world) if r != rank}

    def all_gather(received, mine):
        for r, peer in peers.items():
            codes, scales = codec_torch.quantize(peer.cpu(), 64)
            received[r, :plan.payload_bytes].copy_(codec_torch.pack(codes, scales))

    out = torch.empty(n, device=hip_device)
    reduced = plan.run(bucket, all_gather, op="sum", out=out)
    payloads = [codec_torch.quantize((bucket if r == rank else peers[r]).cpu(), 64) for r in range(world)]
    want = codec_torch.reduce_payloads(payloads, n, 64, "fp32", "sum")
    assert same_bits(reduced.cpu().reshape(-1), want)
