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
from ..parts.inject import StreamMix
from ..parts.lazy import plain, run_norm, settle
from ..parts.offsets import StreamOffsetTable
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
        self.offsets = None
        if spec.stream_offsets is not None:
            so = spec.stream_offsets
            for place in so.places:
                if not 0 <= place < len(self.order):
                    raise ValueError(f"a stream offset names place {place} of a run order of {len(self.order)}")
            self.offsets = StreamOffsetTable(so.checkpoint_name, so.places, spec.hidden_size, name="stream_offsets")
        self.mixes = None
        if spec.stream_mixes is not None:
            sm = spec.stream_mixes
            for place in sm.places:
                if not 0 <= place < len(self.order):
                    raise ValueError(f"a stream mix names place {place} of a run order of {len(self.order)}")
            self.mixes = StreamMix(sm.checkpoint_name, sm.places, spec.hidden_size, name="stream_mix")
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
            if (layer.feed_forward is None) != (layer.feed_forward_norm is None):
                raise ValueError(f"layer {i}: a feed-forward and its norm come together or not at all")
            ff = n2 = None
            if layer.feed_forward is not None:
                ff = FEED_FORWARDS.create(
                    layer.feed_forward.kind, **layer.feed_forward.params, name=f"layers.{i}.ff"
                )
                n2 = NORMS.create(
                    layer.feed_forward_norm.kind, **layer.feed_forward_norm.params, name=f"layers.{i}.ff_norm"
                )
            n1 = NORMS.create(layer.mixer_norm.kind, **layer.mixer_norm.params, name=f"layers.{i}.mixer_norm")
            post = {}
            if layer.mixer_post_norm is not None:
                post["mixer_post_norm"] = NORMS.create(
                    layer.mixer_post_norm.kind, **layer.mixer_post_norm.params, name=f"layers.{i}.mixer_post_norm"
                )
            if layer.feed_forward_post_norm is not None:
                if ff is None:
                    raise ValueError(f"layer {i}: a norm behind a feed-forward that is not there")
                post["feed_forward_post_norm"] = NORMS.create(
                    layer.feed_forward_post_norm.kind, **layer.feed_forward_post_norm.params,
                    name=f"layers.{i}.ff_post_norm",
                )
            self.blocks.append(
                BLOCKS.create(
                    layer.block.kind,
                    **layer.block.params,
                    mixer=mixer,
                    feed_forward=ff,
                    mixer_norm=n1,
                    feed_forward_norm=n2,
                    **post,
                )
            )

    # ---- tensors ---------------------------------------------------------------
    def all_parts(self):
        yield self.embed
        for block in self.blocks:
            yield from block.parts()
        yield self.final_norm
        yield self.output
        if self.offsets is not None:
            yield self.offsets
        if self.mixes is not None:
            yield self.mixes
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
        # the embedding's output, which the stream mixes take in again (the stream itself is
        # updated in place)
        first = residual.clone() if self.mixes is not None else None
        delta = None
        for place, li in enumerate(self.order):
            block = self.blocks[li]
            if self.mixes is not None and self.mixes.at(place):
                delta = settle(residual, delta)
                if delta is not None:
                    residual.add_(delta)
                    delta = None
                residual = self.mixes.forward(residual, first)
            if self.offsets is not None:
                self.offsets.add(residual, place)
            if not getattr(block, "accepts_deferred", False):
                delta = settle(residual, delta)
            delta = block.forward(residual, delta, ctx, caches[place])
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=residual.device)
        h = run_norm(self.final_norm, residual, delta, ctx, rows=ctx.logit_rows)
        return self.output.forward(h, ctx)


def model_param_specs(spec: ModelSpec) -> list[ParamSpec]:
    return CausalLM(spec).param_specs()
