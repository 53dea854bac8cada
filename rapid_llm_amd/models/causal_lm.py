"""The generic decoder: embedding, blocks in their run order, final norm, output projection.

Built from a :class:`~rapid_llm_amd.models.spec.ModelSpec` alone; nothing here names an
architecture.  The reference's skeleton is ``CausalLM`` (rapid_llm/models/base.py:378-631):
embed (:589-591), layers (:608-612), final norm (:619-621), row selection before the vocabulary
product (:625-630), output projection (:631).
"""

from __future__ import annotations

from dataclasses import replace

import torch

from ..parts.base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    OUTPUT_PROJECTIONS,
    POSITION_ENCODINGS,
    CacheNeed,
    ParamSpec,
)
from ..parts.lazy import plain, run_norm
from .spec import ModelSpec


class CausalLM:
    def __init__(self, spec: ModelSpec) -> None:
        import rapid_llm_amd.parts  # noqa: F401  registers the built-in part kinds

        self.spec = spec
        self.embed = EMBEDDINGS.create(spec.embedding.kind, **spec.embedding.params, name="embed")
        self.output = OUTPUT_PROJECTIONS.create(spec.output.kind, **spec.output.params, name="output")
        self.final_norm = NORMS.create(spec.final_norm.kind, **spec.final_norm.params, name="final_norm")
        self.order = list(spec.order())
        for li in self.order:
            if not 0 <= li < len(spec.layers):
                raise ValueError(f"run order names layer {li}; the model has {len(spec.layers)}")
        self._positions: dict[str, object] = {}
        self.blocks = []
        for i, layer in enumerate(spec.layers):
            pos_key = repr((layer.position.kind, sorted(layer.position.params.items())))
            position = self._positions.get(pos_key)
            if position is None:
                position = POSITION_ENCODINGS.create(layer.position.kind, **layer.position.params)
                self._positions[pos_key] = position
            mixer = MIXERS.create(
                layer.mixer.kind, **layer.mixer.params, position=position, name=f"layers.{i}.mixer"
            )
            ff = FEED_FORWARDS.create(
                layer.feed_forward.kind, **layer.feed_forward.params, name=f"layers.{i}.ff"
            )
            n1 = NORMS.create(layer.mixer_norm.kind, **layer.mixer_norm.params, name=f"layers.{i}.mixer_norm")
            n2 = NORMS.create(
                layer.feed_forward_norm.kind, **layer.feed_forward_norm.params, name=f"layers.{i}.ff_norm"
            )
            self.blocks.append(
                BLOCKS.create(
                    layer.block.kind,
                    **layer.block.params,
                    mixer=mixer,
                    feed_forward=ff,
                    mixer_norm=n1,
                    feed_forward_norm=n2,
                )
            )

    # ---- tensors ---------------------------------------------------------------
    def all_parts(self):
        yield self.embed
        for block in self.blocks:
            yield from block.parts()
        yield self.final_norm
        yield self.output
        yield from self._positions.values()

    def param_specs(self) -> list[ParamSpec]:
        specs: list[ParamSpec] = []
        for part in self.all_parts():
            specs.extend(part.param_specs())
        names = [s.name for s in specs]
        if len(names) != len(set(names)):
            raise ValueError("two parts declare a parameter of the same name")
        return specs

    def bind(self, params: dict[str, torch.Tensor], runtime) -> None:
        for part in self.all_parts():
            part.bind(params, runtime)

    def replayable(self) -> bool:
        """Whether a step of this model may be recorded into a graph: every part and every
        block says so (``Part.replayable``)."""
        return all(getattr(p, "replayable", False) for p in (*self.all_parts(), *self.blocks))

    # ---- cache -----------------------------------------------------------------
    def cache_needs(self) -> list[CacheNeed]:
        """One need per place in the run order.  ``LayerSpec.share_cache_with`` names a layer;
        it resolves to that layer's latest earlier place in the order."""
        needs: list[CacheNeed] = []
        last_place: dict[int, int] = {}
        for place, li in enumerate(self.order):
            need = self.blocks[li].mixer.cache_need()
            share = self.spec.layers[li].share_cache_with
            if share is not None:
                if share not in last_place:
                    raise ValueError(
                        f"layer {li} reads the cache of layer {share}, which has not run before it"
                    )
                need = replace(need, share_with=last_place[share])
            needs.append(need)
            last_place[li] = place
        return needs

    # ---- step ------------------------------------------------------------------
    def forward(self, ctx, caches) -> torch.Tensor:
        """Run the tokens of ``ctx`` through every layer (which writes their keys and values)
        and return float32 logits ``[len(ctx.logit_rows), vocab]``."""
        residual = self.embed.forward(ctx.token_ids, ctx)
        delta = None
        for place, li in enumerate(self.order):
            block = self.blocks[li]
            if not getattr(block, "accepts_deferred", False):
                delta = plain(delta)
            delta = block.forward(residual, delta, ctx, caches[place])
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=residual.device)
        h = run_norm(self.final_norm, residual, delta, ctx, rows=ctx.logit_rows)
        return self.output.forward(h, ctx)


def model_param_specs(spec: ModelSpec) -> list[ParamSpec]:
    return CausalLM(spec).param_specs()
