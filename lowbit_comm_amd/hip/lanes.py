"""Dealing independent buckets to a few HIP streams in turn.

A launch on this part costs about 2.6 us of ramp-up and drain before and after its bytes move, and two launches on
one stream do not overlap.  Consecutive DDP buckets are independent of each other, so their launches may go to
different streams: the ramp-up of one bucket's kernel then overlaps the drain of the one before (measured on a stream
of 613 bucket steps of 25 MiB: 28.0 -> 26.1 us per bucket with two lanes; on 100 MiB steps 29.9, 27.3 and 26.7 us
with one, two and three).  What the caller
has to provide is what independence means: every lane needs its own output buffers (send matrix, shard output), so
that nothing written on one lane is touched on another before :meth:`StreamLanes.join`.

    lanes = StreamLanes(2)
    lanes.fork()                                   # the lanes wait for the work already on the current stream
    for k, launch in enumerate(bucket_launches):   # BoundLaunch objects
        launch(lanes.handle(k))
    lanes.join()                                   # the current stream waits for every lane

All streams have the default priority.  (The reference runs its compute on the single stream torch hands it; this is
an MI355X-side scheduling aid with no counterpart there.)
"""
from __future__ import annotations

from typing import Any


class StreamLanes:
    """``count`` streams of one device that are forked from, and joined back into, the caller's current stream."""

    def __init__(self, count: int = 2, device: Any | None = None) -> None:
        import torch

        if count < 1:
            raise ValueError("count must be at least 1")
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        self.streams = [torch.cuda.Stream(device=self.device) for _ in range(count)]      # default priority
        self._handles = [s.cuda_stream for s in self.streams]

    def __len__(self) -> int:
        return len(self.streams)

    def stream(self, index: int) -> Any:
        """The ``torch.cuda.Stream`` that item ``index`` of a sequence goes to."""
        return self.streams[index % len(self.streams)]

    def handle(self, index: int) -> int:
        """The raw ``hipStream_t`` of that stream, as a bound launch takes it."""
        return self._handles[index % len(self._handles)]

    def fork(self) -> None:
        """Order every lane after what the current stream has been given so far."""
        import torch

        current = torch.cuda.current_stream(self.device)
        for lane in self.streams:
            lane.wait_stream(current)

    def join(self) -> None:
        """Order the current stream after everything the lanes have been given so far."""
        import torch

        current = torch.cuda.current_stream(self.device)
        for lane in self.streams:
            current.wait_stream(lane)


__all__ = ["StreamLanes"]
