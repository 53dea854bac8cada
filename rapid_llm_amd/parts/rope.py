"""Rotary position encoding, half-split pairing: tables of cos and sin per position.

``inv_freq[i] = 1 / theta^(2i/d)`` in float32 (rapid_llm/modules/rotary_embedding.py:30-37);
the angle of position ``p`` is the float32 product ``p * inv_freq[i]`` (:194-202).  The
tables stay float32 (the reference casts them to the activation type each step, :214-218);
the rotation itself runs inside the attention mixer's fused kernel, which gathers rows of
these tables by position.  Another frequency rule (scaled, banded) is another ``inv_freq``
and therefore another subclass overriding :meth:`inverse_frequencies`.
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


class RotaryHalfSplit(PositionEncoding):
    replayable = True
    kind = "rope_half_split"

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None) -> None:
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim != head_dim:
            raise ValueError(
                f"rotation over {self.rotary_dim} of {head_dim} channels is not implemented "
                "(the fused kernel pairs channel i with i + head_dim/2)"
            )
        if head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {head_dim}")
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def inverse_frequencies(self) -> torch.Tensor:
        d = self.rotary_dim
        return 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))

    def bind(self, params, runtime) -> None:
        inv_freq = self.inverse_frequencies().to(runtime.device)
        self.cos, self.sin = ops.rope_table(inv_freq, runtime.max_seq_len)


POSITION_ENCODINGS.register("none", NoPositionEncoding)
POSITION_ENCODINGS.register("rope_half_split", RotaryHalfSplit)
