"""Arrangement of one mixer and one feed-forward with their norms.

``PreNormBlock`` is the reference's ``DecoderLayer.forward`` (``src/decoder_layer.py:41-54``):
``h = h + mixer(norm1(h)); h = h + ff(norm2(h))``.  The residual ``h`` lives in a float32
tensor; what a sub-layer produced is carried as ``pending`` and added inside the next
norm's kernel, so each block hands its feed-forward output on to whoever normalises next.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import Block, FeedForward, Mixer, Norm, Part, ResidualSink, register_arrangement


class PreNormBlock(Block):
    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Norm) -> None:
        super().__init__(prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ff_norm = ff_norm

    def children(self) -> Tuple[Part, ...]:
        return (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)

    def input_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional[Norm] = None):
        """``next_norm``: the norm that will read this block's output (the next block's first norm), if the caller
        allows the feed-forward to add its output to the residual itself (see ``ResidualSink``)."""
        normed = self.mixer_norm.forward(residual, pending, ctx)
        if not getattr(self.mixer, "accepts_deferred", False):
            normed = ctx.ops.materialize(normed)  # (a DeferredNorm becomes a tensor; a tensor stays)
        if getattr(self.mixer, "accepts_sink", False):
            mixed = self.mixer.forward(normed, ctx, cache, owns_cache, sink=ResidualSink(residual, self.ff_norm))
        else:
            mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        normed = self.ff_norm.forward(residual, mixed, ctx)
        if not getattr(self.feed_forward, "accepts_deferred", False):
            normed = ctx.ops.materialize(normed)
        if next_norm is not None and getattr(self.feed_forward, "accepts_sink", False):
            return self.feed_forward.forward(normed, ctx, sink=ResidualSink(residual, next_norm))
        return self.feed_forward.forward(normed, ctx)


register_arrangement("pre_norm", PreNormBlock)
