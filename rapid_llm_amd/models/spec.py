"""Pure-data description of a model: what the generic ``CausalLM`` is built from.

An architecture's builder turns its typed configuration into a :class:`ModelSpec`:
which mixer, feed-forward, norms and block each layer has (chosen layer by layer, each
with its own parameters), which embedding and output projection stand at its two ends,
and the order in which layers run.  The order is data too: ``run_order`` may name a layer
twice, and a layer may read another layer's cache (``LayerSpec.share_cache_with``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class IgnoreRule:
    """Checkpoint names that are dropped unread: ``pattern`` matches the whole name and,
    when ``min_index`` is given, the integer in group 1 is at least ``min_index``."""

    pattern: str
    min_index: int | None = None


@dataclass(frozen=True)
class LayerSpec:
    """One layer: parts by kind and parameters, plus where its tensors sit in the checkpoint."""

    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    block: PartSpec = PartSpec("prenorm")
    position: PartSpec = PartSpec("none")
    checkpoint_prefix: str = ""
    share_cache_with: int | None = None  # index of the layer whose cache this one reads


def token_embedding(vocab_size: int, hidden_size: int, checkpoint_name: str) -> PartSpec:
    """The plain table lookup."""
    return PartSpec(
        "token_embedding", {"vocab_size": vocab_size, "hidden_size": hidden_size, "checkpoint_name": checkpoint_name}
    )


def linear_output(vocab_size: int, hidden_size: int, checkpoint_name: str, tied: bool) -> PartSpec:
    """The plain product with a ``[vocab, hidden]`` matrix; ``tied``: the embedding's table
    stands in when the checkpoint ships none (the embedding part's parameter is ``embed.weight``)."""
    return PartSpec(
        "linear_output",
        {"vocab_size": vocab_size, "hidden_size": hidden_size, "checkpoint_name": checkpoint_name,
         "tied_to": "embed.weight" if tied else None},
    )


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    layers: tuple[LayerSpec, ...]
    final_norm: PartSpec
    embedding: PartSpec  # built with name="embed"
    output: PartSpec  # built with name="output"
    run_order: tuple[int, ...] | None = None  # None: 0..len(layers)-1
    ignore_tensors: tuple[IgnoreRule, ...] = ()
    max_position: int = 0  # largest position the architecture is defined for (0: unbounded)

    def order(self) -> tuple[int, ...]:
        return self.run_order if self.run_order is not None else tuple(range(len(self.layers)))
