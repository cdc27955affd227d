"""Arrangements of a layer's parts."""

from __future__ import annotations

from ..kernels import ops
from .base import BLOCKS, Block


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """``h = x + mixer(norm(x)); out = h + ffn(norm(h))``
    (reference: torchllms/models/networks.py:635-644).  Each residual sum is fused into the
    norm that reads it; the last one is handed on as ``delta``."""

    graph_safe = True
    SLOTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}

    def forward(self, h, delta, ctx, cache):
        h, y = self.mixer_norm.forward_add_for(self.mixer, h, delta)
        a = self.mixer.forward(y, ctx, cache["mixer"])
        h, y = self.ffn_norm.forward_add_for(self.ffn, h, a)
        f = self.ffn.forward(y, ctx)
        return h, f


class _Parallel(Block):
    """One norm whose output every branch of the layer reads: ``x <- x + mult * (sum of the branches)``.
    The sum is handed on unapplied (``ops.ScaledSum``), so that the next norm's kernel adds it."""

    graph_safe = True

    def __init__(self, parts, residual_mult: float = 1.0):
        super().__init__(parts)
        self.residual_mult = float(residual_mult)

    def branches(self, y, ctx, cache):
        raise NotImplementedError

    def forward(self, h, delta, ctx, cache):
        h, y = self.norm1.forward_add(h, self.norm1.delta(delta))
        return h, ops.ScaledSum(self.branches(y, ctx, cache), self.residual_mult)


@BLOCKS.register("parallel")
class ParallelBlock(_Parallel):
    """``h = norm1(x); x <- x + mult * (mix(h) + mlp(h))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer", "mlp": "feed_forward"}

    def branches(self, y, ctx, cache):
        return [self.mix.forward(y, ctx, cache["mix"]), self.mlp.forward(y, ctx)]


@BLOCKS.register("parallel_mixer")
class ParallelMixerBlock(_Parallel):
    """The same layer without a feed-forward: ``x <- x + mult * mix(norm1(x))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer"}

    def branches(self, y, ctx, cache):
        return [self.mix.forward(y, ctx, cache["mix"])]
