"""Token embedding (row gather into the float32 residual stream) and the output projection.

rapid_llm/modules/vocab_parallel.py:102-103 (``F.embedding``) and :125-126 (``F.linear(h, W)``);
a tied output projection is the embedding table under a second name
(rapid_llm/models/weights.py:197-214).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import ParamSpec, Part, Source
from .linear import Linear


class TokenEmbedding(Part):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, checkpoint_name: str, name: str = "embed") -> None:
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.checkpoint_name = checkpoint_name
        self.name = name
        self.table: torch.Tensor | None = None

    def param_specs(self):
        return [
            ParamSpec(
                self.name + ".weight",
                (self.vocab_size, self.hidden_size),
                "matrix",
                (Source(self.checkpoint_name, self.vocab_size),),
            )
        ]

    def bind(self, params, runtime) -> None:
        self.table = params[self.name + ".weight"]

    def forward(self, token_ids: torch.Tensor, fed_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """Rows of the table for the ids; an id ``-(r + 1)`` takes ``fed_tokens[r]``."""
        out = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=token_ids.device)
        ops.embed(token_ids, self.table, out, fed_tokens)
        return out


class OutputProjection(Part):
    """``logits = h W^T`` in float32, over the rows that were asked for only."""

    replayable = True

    def __init__(
        self,
        vocab_size: int,
        hidden_size: int,
        checkpoint_name: str,
        tied_to: str | None,
        name: str = "output",
    ) -> None:
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.checkpoint_name = checkpoint_name
        self.tied_to = tied_to
        self.name = name
        self.proj = Linear(hidden_size, vocab_size)

    def param_specs(self):
        return [
            ParamSpec(
                self.name + ".weight",
                (self.vocab_size, self.hidden_size),
                "matrix",
                (Source(self.checkpoint_name, self.vocab_size),),
                fallback=self.tied_to,
            )
        ]

    def bind(self, params, runtime) -> None:
        self.proj.bind(params[self.name + ".weight"])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.proj(h, out_dtype=torch.float32)
