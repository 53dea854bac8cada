"""Token embedding (row gather into the float32 residual stream) and the output projection.

rapid_llm/modules/vocab_parallel.py:102-103 (``F.embedding``) and :125-126 (``F.linear(h, W)``);
a tied output projection is the embedding table under a second name
(rapid_llm/models/weights.py:197-214).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import EMBEDDINGS, OUTPUT_PROJECTIONS, Embedding, OutputProjection, ParamSpec, Source
from .linear import Linear


class TokenEmbedding(Embedding):
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

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        """Rows of the table for the ids; an id ``-(r + 1)`` takes ``ctx.fed_tokens[r]``."""
        out = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=token_ids.device)
        ops.embed(token_ids, self.table, out, getattr(ctx, "fed_tokens", None))
        return out


class LinearOutput(OutputProjection):
    """``logits = h W^T`` in float32, over the rows that were asked for only.  ``tied_to``
    names the parameter (the embedding's table) that stands in when the checkpoint ships no
    tensor of this part's own."""

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

    def forward(self, h: torch.Tensor, ctx=None) -> torch.Tensor:
        return self.proj(h, out_dtype=torch.float32)


EMBEDDINGS.register("token_embedding", TokenEmbedding)
OUTPUT_PROJECTIONS.register("linear_output", LinearOutput)
