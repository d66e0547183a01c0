"""Replay of a module's forward as one HIP graph (not in the reference).

A decode step through the drop-in modules costs about ten microseconds of host time per layer for three to
seven microseconds of kernel time, so a stack of quantized layers called eagerly leaves the GPU idle most of the
time.  ``GraphedForward`` records the forward of any module built from this package's layers once, for one input
shape, and replays the recording: one graph launch per step whatever the number of layers.  The kernels of this
library keep no state between calls, allocate nothing and never synchronise, so their launches can be recorded;
outputs are allocated by torch inside the recording and live in the graph's memory pool.
"""
from __future__ import annotations

import torch


class GraphedForward:
    """``g = GraphedForward(module, example)``; ``y = g(x)`` copies ``x`` into the recorded input, replays the graph
    and returns the recorded output tensor (the same tensor object every call: clone it to keep a result across
    calls).  ``x`` must have the shape, dtype and device of ``example``.  ``g.input`` / ``g.output`` are the static
    tensors, for callers that write the input in place and call ``g.replay()`` themselves.

    The module's buffers are read at replay time through the addresses recorded, so a change of their contents in
    place is seen, a buffer replaced by a new tensor (``.to()``, ``load_state_dict(assign=True)``) is not: record
    again after such a change."""

    def __init__(self, module: torch.nn.Module, example: torch.Tensor, warmup: int = 3):
        if not example.is_cuda:
            raise RuntimeError("GraphedForward: the example input must be on a GPU")
        self.module = module
        self.input = example.detach().clone()
        side = torch.cuda.Stream(device=example.device)
        side.wait_stream(torch.cuda.current_stream(example.device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(max(1, warmup)):   # builds the layers' prepared calls and lazily made buffers outside the recording
                module(self.input)
        torch.cuda.current_stream(example.device).wait_stream(side)
        torch.cuda.synchronize(example.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.output = module(self.input)

    def replay(self) -> None:
        self.graph.replay()

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape != self.input.shape or x.dtype != self.input.dtype or x.device != self.input.device:
            raise RuntimeError(f"GraphedForward: recorded for {self.input.dtype} {tuple(self.input.shape)} on "
                               f"{self.input.device}, got {x.dtype} {tuple(x.shape)} on {x.device}")
        self.input.copy_(x)
        self.graph.replay()
        return self.output
