"""Recording calls of this package into a HIP graph.

No counterpart in the reference (MLX builds its graph lazily by itself).  On this part a call
through the Python surface costs the host 10-30 microseconds, as much as the device needs for a
layer kernel, so a serving loop replays the verify step instead of launching it call by call.
The kernels allow it: nothing in them depends on host state from the time of capture (split-K
arrival counters return to zero by themselves, accepted lengths can be device tensors,
workspaces belong to the stream).
"""
from __future__ import annotations

from typing import Any, Callable, Tuple

import torch


def record(fn: Callable[[], Any]) -> Tuple["torch.cuda.CUDAGraph", Any]:
    """Run ``fn`` once on a side stream - workspaces are created on first use, and an allocation
    cannot be recorded - then record a second run of it on that stream.

    Returns ``(graph, outputs)``: ``graph.replay()`` repeats the recorded launches on the
    tensors ``fn`` read and wrote, so new inputs are copied into the same tensors
    (``x.copy_(new)``) and results are read from ``outputs`` after the replay.  ``fn`` must not
    synchronise with the host or read device values (``.item()``, ``bool(tensor)``): pass
    accepted lengths as int32 device tensors."""
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outputs = fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    return graph, outputs
