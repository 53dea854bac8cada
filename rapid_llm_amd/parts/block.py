"""Pre-norm arrangement: ``r += mixer(norm(r)); r += feed_forward(norm(r))``.

The add of each sub-layer's output is carried forward as ``delta`` and happens inside the
next norm kernel, as the reference threads ``(hidden, residual)`` through its layers
(rapid_llm/models/base.py:231-266,:363-375).
"""

from __future__ import annotations

from ..kernels import ops
from .base import BLOCKS, Block


def run_norm(norm, residual, delta, ctx, rows=None):
    """``norm(residual + delta)`` where ``delta`` may be a product's
    :class:`~rapid_llm_amd.kernels.ops.ResidualUpdate` (already added)."""
    if isinstance(delta, ops.ResidualUpdate) and not getattr(norm, "accepts_update", False):
        delta = None
    return norm.forward(residual, delta, ctx, rows) if rows is not None else norm.forward(residual, delta, ctx)


def run_part(part, x, residual, *args):
    """A mixer or feed-forward on the norm's output; fusing parts get the residual too."""
    if getattr(part, "fuses_residual", False):
        return part.forward(x, *args, residual=residual)
    if isinstance(x, ops.NormedRows):
        x = x.materialize()
    return part.forward(x, *args)


class PreNormBlock(Block):
    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, residual, delta, ctx, cache):
        x = run_norm(self.mixer_norm, residual, delta, ctx)
        a = run_part(self.mixer, x, residual, ctx, cache)
        x = run_norm(self.feed_forward_norm, residual, a, ctx)
        return run_part(self.feed_forward, x, residual, ctx)


BLOCKS.register("prenorm", PreNormBlock)
