"""Stream mixes: what the next layer reads as a function of the results of all layers so far.

Depth-weighted average: with X_0 the embedding's output and X_(i+1) the result of the i-th layer run (its input plus what
its branches add), the stream that goes on is sum_j w[j] X_j over j = 0 .. i+1, with a weight vector of the layer's own.
The results are kept for the step in one float32 tensor ``[runs + 1, T, dim]``; the sum runs in 32-bit, in the order of j.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildEnv, StepContext, StreamMix
from .registry import STREAM_MIXES
from .spec import PartSpec


@STREAM_MIXES.register("depth_weighted_average")
class DepthWeightedAverage(StreamMix):
    """params: ``index`` (how many layer runs come before this one), ``n_runs`` (layer runs of the model); tensor
    ``weights`` ``[index + 2]``."""

    graph_safe = True
    KEY = "depth_weighted_average.streams"

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.index = int(spec.params["index"])
        self.n_runs = int(spec.params["n_runs"])
        if not 0 <= self.index < self.n_runs:
            raise ValueError(f"depth_weighted_average: run {self.index} of {self.n_runs}")
        self.weights = tensors["weights"].to(env.device, torch.float32).contiguous()
        if self.weights.numel() != self.index + 2:
            raise ValueError(f"depth_weighted_average: run {self.index} needs {self.index + 2} weights, got {self.weights.numel()}")

    def enter(self, x: torch.Tensor, ctx: StepContext) -> None:
        if self.index == 0:  # the embedding's output is the first of the results
            ctx.settle()
            streams = torch.empty((self.n_runs + 1,) + tuple(x.shape), dtype=torch.float32, device=x.device)
            streams[0].copy_(x)
            ctx.shared[self.KEY] = streams

    def leave(self, x: torch.Tensor, ctx: StepContext) -> None:
        streams = ctx.shared.get(self.KEY)
        if streams is None or streams.shape[1:] != x.shape:
            raise RuntimeError("depth_weighted_average: the run with index 0 has not been through this step")
        ctx.settle()
        # where the block allows it the sum is left to the norm that reads x next (the next layer's, or the one before the head)
        ctx.pending = ctx.kernels.stream_average(streams, x, self.weights, self.index + 2, defer=bool(ctx.may_defer))
