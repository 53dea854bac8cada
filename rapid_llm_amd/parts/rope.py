"""Rotary position encoding: tables of cos and sin per position, and how they are applied.

``inv_freq[i] = 1 / theta^(2i/d)`` in float32 over the ``d`` channels that rotate
(rapid_llm/modules/rotary_embedding.py:25-37: ``d = head_dim * partial_rotary_factor``); the
angle of position ``p`` is the float32 product ``p * inv_freq[i]`` (:194-202).  The tables stay
float32 (the reference casts them to the activation type each step, :214-218).  The part owns
what defines the encoding, the tables, how many of a head's leading channels rotate
(``rotary_dim``) and which of them form a pair (``pairing``); the rotation itself runs inside
the mixer's kernels, which gather rows of these tables by position and are told both.
Another frequency rule (scaled, banded) is another ``inv_freq`` and therefore a subclass
overriding :meth:`inverse_frequencies`.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding


class NoPositionEncoding(PositionEncoding):
    replayable = True
    kind = "none"

    def __init__(self, **_ignored) -> None:
        self.cos = None
        self.sin = None


class Rotary(PositionEncoding):
    """``pairing="half_split"``: channel ``i`` rotates with ``i + rotary_dim / 2``
    (rapid_llm/kernels/ops/rope/rope_emb.py:47-82); ``"interleaved"``: ``2i`` with ``2i + 1``."""

    replayable = True
    kind = "rope"

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None,
                 pairing: str = "half_split") -> None:
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        self.pairing = pairing
        if pairing not in ops.ROTARY_PAIRINGS:
            raise ValueError(f"rotation pairing {pairing!r} is not one of {sorted(ops.ROTARY_PAIRINGS)}")
        if self.rotary_dim % 2 or not 2 <= self.rotary_dim <= head_dim:
            raise ValueError(
                f"a rotation takes an even number of a head's {head_dim} channels, at least two, got {self.rotary_dim}"
            )
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def inverse_frequencies(self) -> torch.Tensor:
        d = self.rotary_dim
        return 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))

    def bind(self, params, runtime) -> None:
        inv_freq = self.inverse_frequencies().to(runtime.device)
        self.cos, self.sin = ops.rope_table(inv_freq, runtime.max_seq_len)


class RotaryHalfSplit(Rotary):
    """The reference's rotation: pairs ``(i, i + rotary_dim / 2)``."""

    kind = "rope_half_split"

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None) -> None:
        super().__init__(head_dim, theta, rotary_dim, "half_split")


POSITION_ENCODINGS.register("none", NoPositionEncoding)
POSITION_ENCODINGS.register("rope", Rotary)
POSITION_ENCODINGS.register("rope_half_split", RotaryHalfSplit)
