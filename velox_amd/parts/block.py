"""Arrangement of one mixer and one feed-forward with their norms.

``PreNormBlock`` is the reference's ``DecoderLayer.forward`` (``src/decoder_layer.py:41-54``):
``h = h + mixer(norm1(h)); h = h + ff(norm2(h))``.  The residual ``h`` lives in a float32
tensor; what a sub-layer produced is carried as ``pending`` and added inside the next
norm's kernel, so each block hands its feed-forward output on to whoever normalises next.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import FeedForward, Mixer, Norm, Part


class PreNormBlock(Part):
    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Norm) -> None:
        super().__init__(prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ff_norm = ff_norm

    def children(self) -> Tuple[Part, ...]:
        return (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache, owns_cache: bool) -> torch.Tensor:
        normed = self.mixer_norm.forward(residual, pending, ctx)
        mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        normed = self.ff_norm.forward(residual, mixed, ctx)
        return self.feed_forward.forward(normed, ctx)


BLOCK_ARRANGEMENTS = {"pre_norm": PreNormBlock}
