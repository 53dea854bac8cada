"""Pre-norm arrangement: ``r += mixer(norm(r)); r += feed_forward(norm(r))``.

The add of each sub-layer's output is carried forward as ``delta`` and happens inside the
next norm kernel, as the reference threads ``(hidden, residual)`` through its layers
(rapid_llm/models/base.py:231-266,:363-375).
"""

from __future__ import annotations

from .base import BLOCKS, Block
from .lazy import run_norm


class PreNormBlock(Block):
    replayable = True
    accepts_deferred = True  # the incoming delta may be a DeferredProduct

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, residual, delta, ctx, cache):
        x = run_norm(self.mixer_norm, residual, delta, ctx, consumer=self.mixer)
        a = self.mixer.forward(x, ctx, cache)
        x = run_norm(self.feed_forward_norm, residual, a, ctx, consumer=self.feed_forward)
        return self.feed_forward.forward(x, ctx)


BLOCKS.register("prenorm", PreNormBlock)
