"""Pre-norm arrangement: ``r += mixer(norm(r)); r += feed_forward(norm(r))``.

The add of each sub-layer's output is carried forward as ``delta`` and happens inside the
next norm kernel, as the reference threads ``(hidden, residual)`` through its layers
(rapid_llm/models/base.py:231-266,:363-375).
"""

from __future__ import annotations

from .base import BLOCKS, Block


class PreNormBlock(Block):
    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, residual, delta, ctx, cache):
        x = self.mixer_norm.forward(residual, delta, ctx)
        a = self.mixer.forward(x, ctx, cache)
        x = self.feed_forward_norm.forward(residual, a, ctx)
        return self.feed_forward.forward(x, ctx)


BLOCKS.register("prenorm", PreNormBlock)
