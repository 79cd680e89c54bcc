"""Blocks: how the parts of a layer are arranged around the residual stream.
Pre-norm (src/levanter/models/gpt2.py:237-248): x += mixer(norm1(x)); x += feed_forward(norm2(x))."""
from __future__ import annotations

from typing import Dict

import torch

from .base import Block, CacheUnitView, Part, StepContext
from .registry import BLOCKS


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    roles = ("norm1", "mixer", "norm2", "feed_forward")
    defers_residual = True

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        self.norm1, self.mixer, self.norm2, self.feed_forward = (parts[r] for r in self.roles)

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        # a product that the part before has left unfinished is folded into the norm that follows it, or finished first
        if not self.norm1.folds_pending:
            ctx.settle()
        self.mixer.forward(self.norm1(x, ctx), x, ctx, unit, writes_cache)
        if not self.norm2.folds_pending:
            ctx.settle()
        self.feed_forward.forward(self.norm2(x, ctx), x, ctx)


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """One norm whose output every branch reads: with h = norm1(x), x += mixer(h) + feed_forward(h). ``feed_forward`` may be
    missing (a layer that only mixes). With a ``stream_mix`` part the sum is that layer's result, and what the next layer
    reads is the mix's function of it and of earlier layers' results."""

    roles = ("norm1", "mixer")

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        unknown = [r for r in parts if r not in ("norm1", "mixer", "feed_forward", "stream_mix")]
        if unknown:
            raise ValueError(f"block 'parallel' has no role {', '.join(unknown)}")
        self.norm1, self.mixer = parts["norm1"], parts["mixer"]
        self.feed_forward = parts.get("feed_forward")
        self.stream_mix = parts.get("stream_mix")

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        # both branches add to x and the mix reads it: the block does not say ``defers_residual``, so no product is ever
        # left unfinished here
        if self.stream_mix is not None:
            self.stream_mix.enter(x, ctx)
        h = self.norm1(x, ctx)
        self.mixer.forward(h, x, ctx, unit, writes_cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(h, x, ctx)
        if self.stream_mix is not None:
            self.stream_mix.leave(x, ctx)
