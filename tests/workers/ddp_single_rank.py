"""Worker for tests/test_hip_host.py: the compressed hook registered on a real DistributedDataParallel model.

One process, one GPU, a one-rank RCCL process group.  Modes "portable" / "native": the all_gather strategy in that
wire format, the packed payload bytes moved by a real RCCL ``all_gather_into_tensor``.  Mode "reduce_scatter": the
pre-bound reduce-scatter plan with its two exchanges as real RCCL calls (all_to_all_single, all_gather_into_tensor)
and local error feedback; "reduce_scatter_pipelined": the same transport with the bucket pipeline behind it (futures
completed by later buckets, the hook's flush after ``GradBucket.is_last()``).  Prints one JSON line with the gradient
errors against an unwrapped copy of the model.
"""
from __future__ import annotations

import json
import os
import socket
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parents[2]))


def free_port() -> int:
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def main() -> int:
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(free_port())
    import torch
    import torch.distributed as dist
    from torch.nn.parallel import DistributedDataParallel

    from lowbit_comm_amd import CompressionConfig
    from lowbit_comm_amd.communication import GatheredPayloads
    from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
    from lowbit_comm_amd.hip.loader import load_hip_extension

    wire_format = sys.argv[1] if len(sys.argv) > 1 else "portable"
    dist.init_process_group("nccl", rank=0, world_size=1)
    try:
        device = torch.device("cuda:0")
        torch.manual_seed(0)

        def make():
            return torch.nn.Sequential(torch.nn.Linear(512, 1024), torch.nn.ReLU(), torch.nn.Linear(1024, 256)).to(device)

        model, plain = make(), make()
        plain.load_state_dict(model.state_dict())
        wrapped = DistributedDataParallel(model, device_ids=[0], bucket_cap_mb=1)
        status = load_hip_extension(wire_format="portable" if wire_format.startswith("reduce_scatter") else wire_format)
        assert status.available, status.reason
        seen = []

        def gather(payload):
            """The packed payload bytes through a real RCCL all-gather; row r is rank r's payload."""
            from dataclasses import replace

            mine = payload.buffer.reshape(-1)
            seen.append(int(mine.numel()))
            world = dist.get_world_size()
            rows = torch.empty((world, mine.numel()), dtype=mine.dtype, device=mine.device)
            dist.all_gather_into_tensor(rows, mine)
            return GatheredPayloads(payloads=[replace(payload, buffer=rows[r]) for r in range(world)], world_size=world)

        transport = None
        if wire_format.startswith("reduce_scatter"):
            from lowbit_comm_amd.hip.reduce_scatter import make_reduce_scatter_transport

            def all_to_all(received, send):
                seen.append(int(send.shape[1]))
                dist.all_to_all_single(received, send)

            def all_gather(gathered, mine):
                dist.all_gather_into_tensor(gathered, gathered[0])

            transport = make_reduce_scatter_transport(world_size=1, rank=0, all_to_all=all_to_all,
                                                      all_gather=all_gather, error_feedback=True,
                                                      pipelined=wire_format == "reduce_scatter_pipelined")
            hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), strategy="reduce_scatter",
                                        reduce="mean", reduce_scatter_all_gather=transport)
        else:
            hook = create_ddp_comm_hook(CompressionConfig(error_feedback=True), strategy="all_gather", reduce="mean",
                                        all_gather=gather, extension_status=status)
        wrapped.register_comm_hook(None, hook)
        x = torch.randn(64, 512, device=device)
        errors = []
        for _ in range(3):
            wrapped.zero_grad()
            plain.zero_grad()
            wrapped(x).square().mean().backward()
            plain(x).square().mean().backward()
            torch.cuda.synchronize()
            errors.append(max(float((a.grad - b.grad).norm() / (b.grad.norm() + 1e-12))
                              for a, b in zip(model.parameters(), plain.parameters())))
        pipeline = getattr(transport, "pipeline", None)
        print(json.dumps({"errors": errors, "buckets": len(seen), "payload_bytes": sorted(set(seen)),
                          "finite": all(bool(torch.isfinite(p.grad).all()) for p in model.parameters()),
                          "pipeline": None if pipeline is None else dict(pipeline.stats, pending=pipeline.pending)}))
    finally:
        dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
