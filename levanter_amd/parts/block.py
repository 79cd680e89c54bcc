"""Blocks: how the parts of a layer are arranged around the residual stream.
Pre-norm (src/levanter/models/gpt2.py:237-248): x += mixer(norm1(x)); x += feed_forward(norm2(x))."""
from __future__ import annotations

from typing import Dict

import torch

from .base import Block, CacheUnitView, Part, StepContext
from .linear import Linear
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
    defers_residual = True  # x is read through norm1 and the parts only; the stream mix may leave its sum to the next norm

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        unknown = [r for r in parts if r not in ("norm1", "mixer", "feed_forward", "stream_mix")]
        if unknown:
            raise ValueError(f"block 'parallel' has no role {', '.join(unknown)}")
        self.norm1, self.mixer = parts["norm1"], parts["mixer"]
        self.feed_forward = parts.get("feed_forward")
        self.stream_mix = parts.get("stream_mix")
        self.fused_in = self.fused_out = None
        self._fuse_products()

    def _fuse_products(self) -> None:
        """Both branches read the same input and add to the same stream: where the mixer offers ``proj`` / ``attend`` / ``out``
        and the feed-forward ``up`` / ``activate`` / ``down``, their first products become one (the weights' rows side by
        side) and their second products one (the sum over both branches' columns), and the parts' own copies are dropped."""
        m, f = self.mixer, self.feed_forward
        if f is None or not all(hasattr(m, a) for a in ("proj", "attend", "out")) or not all(hasattr(f, a) for a in ("up", "activate", "down")):
            return
        if m.proj.n_out % 8 or m.out.n_in % 8 or m.proj.weight.dtype != f.up.weight.dtype:
            return  # the second branch's columns would start off a 16-byte boundary
        env = m.env

        def cat_bias(a, b, na, nb):
            if a is None and b is None:
                return None
            dev = (a if a is not None else b).device
            return torch.cat([a if a is not None else torch.zeros(na, device=dev), b if b is not None else torch.zeros(nb, device=dev)])

        self.n_mixer_cols, self.n_mixer_heads, self.n_inner = m.proj.n_out, m.out.n_in, f.up.n_out
        # rows of zeros at the end keep the product's rows a multiple of 8 wide, so that 16-byte loads of the heads stay aligned
        fill = (-(m.proj.n_out + f.up.n_out)) % 8
        w_in = torch.cat([m.proj.weight, f.up.weight, torch.zeros(fill, m.proj.n_in, dtype=m.proj.weight.dtype, device=m.proj.weight.device)], 0)
        b_in = cat_bias(m.proj.bias, f.up.bias, m.proj.n_out, f.up.n_out)
        if b_in is not None and fill:
            b_in = torch.cat([b_in, torch.zeros(fill, device=b_in.device)])
        self.fused_in = Linear(w_in, b_in, "out_in", env)
        out_bias = None if m.out.bias is None and f.down.bias is None else sum(b for b in (m.out.bias, f.down.bias) if b is not None)
        self.fused_out = Linear(torch.cat([m.out.weight, f.down.weight], 1), out_bias, "out_in", env)
        m.proj = m.out = f.up = f.down = None

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        may_defer = ctx.may_defer
        if self.stream_mix is not None:
            self.stream_mix.enter(x, ctx)
        if not self.norm1.folds_pending:
            ctx.settle()
        h = self.norm1(x, ctx)
        ctx.may_defer = False  # both branches add to x, one after the other: neither leaves its product unfinished
        if self.fused_in is not None:
            pz = self.fused_in(h, ctx)  # [T, the mixer's projections | the feed-forward's]
            am = ctx.empty(h.shape[0], self.fused_out.n_in)
            self.mixer.attend(pz[:, :self.n_mixer_cols], ctx, unit, writes_cache, am[:, :self.n_mixer_heads])
            self.feed_forward.activate(pz[:, self.n_mixer_cols:self.n_mixer_cols + self.n_inner], ctx, am[:, self.n_mixer_heads:])
            self.fused_out(am, ctx, residual=x)
        else:
            self.mixer.forward(h, x, ctx, unit, writes_cache)
            if self.feed_forward is not None:
                self.feed_forward.forward(h, x, ctx)
        ctx.may_defer = may_defer
        if self.stream_mix is not None:
            self.stream_mix.leave(x, ctx)
