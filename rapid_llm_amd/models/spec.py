"""Pure-data description of a model: what the generic ``CausalLM`` is built from.

An architecture's builder turns its typed configuration into a :class:`ModelSpec`:
which mixer, feed-forward, norms and block each layer has (chosen layer by layer, each
with its own parameters), and the order in which layers run.  The order is data too:
``run_order`` may name a layer twice, and a layer may read another layer's cache
(``LayerSpec.share_cache_with``).
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


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    layers: tuple[LayerSpec, ...]
    final_norm: PartSpec
    embedding_source: str  # checkpoint name of the embedding table
    output_source: str  # checkpoint name of the output projection
    tie_output_to_embedding: bool
    run_order: tuple[int, ...] | None = None  # None: 0..len(layers)-1
    ignore_tensors: tuple[IgnoreRule, ...] = ()
    max_position: int = 0  # largest position the architecture is defined for (0: unbounded)

    def order(self) -> tuple[int, ...]:
        return self.run_order if self.run_order is not None else tuple(range(len(self.layers)))
