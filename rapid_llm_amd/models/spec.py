"""Pure-data description of a model: what the generic ``CausalLM`` is built from.

An architecture's builder turns its typed configuration into a :class:`ModelSpec`:
which mixer, feed-forward, norms and block each layer has (chosen layer by layer, each
with its own parameters), which embedding and output projection stand at its two ends,
and the order in which layers run.  The order is data too: ``run_order`` may name a layer
twice, and a layer may read another layer's cache (``LayerSpec.share_cache_with``).  A layer
may lack the feed-forward sub-layer, learned vectors may be added to the stream at given
places of the order (``ModelSpec.stream_offsets``), and the stream may be mixed with the
embedding's output there (``ModelSpec.stream_mixes``).
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
    feed_forward: PartSpec | None  # None: the layer has the mixer's sub-layer only
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec | None
    block: PartSpec = PartSpec("prenorm")
    position: PartSpec = PartSpec("none")
    checkpoint_prefix: str = ""
    share_cache_with: int | None = None  # index of the layer whose cache this one reads
    # norms behind the sub-layers, applied to their outputs before the add (a block kind that
    # has them, "sandwich", receives them; None: the block has none)
    mixer_post_norm: PartSpec | None = None
    feed_forward_post_norm: PartSpec | None = None


def token_embedding(vocab_size: int, hidden_size: int, checkpoint_name: str) -> PartSpec:
    """The plain table lookup."""
    return PartSpec(
        "token_embedding", {"vocab_size": vocab_size, "hidden_size": hidden_size, "checkpoint_name": checkpoint_name}
    )


def token_embedding_scaled(vocab_size: int, hidden_size: int, checkpoint_name: str, scale: float,
                           sinusoid_base: float | None = None) -> PartSpec:
    """The table lookup times a constant; with ``sinusoid_base`` the sinusoidal vector of the
    token's position is added (sines in the even channels, cosines in the odd ones)."""
    params = {"vocab_size": vocab_size, "hidden_size": hidden_size, "checkpoint_name": checkpoint_name, "scale": scale}
    if sinusoid_base is not None:
        params["sinusoid_base"] = sinusoid_base
    return PartSpec("token_embedding", params)


@dataclass(frozen=True)
class StreamOffsets:
    """Learned vectors added to the residual stream: row ``t`` of the checkpoint tensor
    ``checkpoint_name`` (``[len(places), hidden]``) is added to every token's stream right
    before the layer at place ``places[t]`` of the run order runs."""

    checkpoint_name: str
    places: tuple[int, ...]


@dataclass(frozen=True)
class StreamMixes:
    """Right before the layer at each of ``places`` of the run order runs, the stream becomes
    ``M [x ; x0]``: ``x0`` is the embedding's output, ``M`` the checkpoint tensor
    ``checkpoint_name`` (``[hidden, 2 hidden]``, the columns of ``x`` first)."""

    checkpoint_name: str
    places: tuple[int, ...]


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
    stream_offsets: StreamOffsets | None = None
    stream_mixes: StreamMixes | None = None

    def order(self) -> tuple[int, ...]:
        return self.run_order if self.run_order is not None else tuple(range(len(self.layers)))
