"""Values that a neighbouring part may still fold its own work into.

A decode step is a chain of small kernels, and the residual norm between two products is
the smallest: it only has to know every row's sum of squares.  Two lazy values let the
products on either side absorb it, without any part knowing its neighbours:

* :class:`DeferredProduct`: what a mixer or a feed-forward returns in place of its last
  product ``x W^T`` when that product's own kernels could absorb a norm (``Linear.deferred``
  decides: bfloat16 and few rows).  Whoever receives it may run the product with an epilogue
  of its own, or simply ``materialize()`` it.
* :class:`ScaledRows`: what a norm returns in place of normalised rows when its consumer
  says it accepts them: the rows times the norm's weight, and the pieces of every row's sum
  of squares; the factor ``rsqrt(mean + eps)`` is a scalar per row and commutes with the
  consumer's own product, which applies it to its result.

Blocks and models route these only between parts that declare them (``fuses_products`` on
a norm, ``accepts_scaled_rows`` on a mixer or feed-forward, ``accepts_deferred`` on a
block); everything else sees plain tensors.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


class DeferredProduct:
    def __init__(self, linear: Any, x: torch.Tensor) -> None:
        self.linear = linear
        self.x = x

    @property
    def shape(self) -> tuple[int, int]:
        return (self.x.shape[0], self.linear.out_features)

    def materialize(self, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return self.linear(self.x, out_dtype)


@dataclass
class ScaledRows:
    rows: torch.Tensor  # [M, size], the residual rows times the norm's weight
    partial: torch.Tensor  # [parts, 16] float32: pieces of every row's sum of squares
    size: int
    eps: float

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype

    @property
    def device(self):
        return self.rows.device


def plain(value):
    """A tensor, whatever lazy value it still was."""
    return value.materialize() if isinstance(value, DeferredProduct) else value


def run_norm(norm, residual, delta, ctx, consumer=None, rows=None):
    """``norm.forward`` with the lazy values routed as the two sides declare them."""
    if getattr(norm, "fuses_products", False):
        return norm.forward(
            residual, delta, ctx, rows, scaled_ok=bool(getattr(consumer, "accepts_scaled_rows", False))
        )
    return norm.forward(residual, plain(delta), ctx, rows)
