"""Learned vectors added to the residual stream at given places of the run order.

A model whose layers run in passes (a span of layers repeated with the same weights) may tell
the passes apart by a vector of its own per pass, added to every token's stream before the
pass's first layer.  The table is one checkpoint tensor ``[rows, hidden]``; row ``t`` belongs
to place ``places[t]``.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import ParamSpec, Part, Source


class StreamOffsetTable(Part):
    replayable = True

    def __init__(self, checkpoint_name: str, places: tuple[int, ...], hidden_size: int, name: str = "stream_offsets"):
        self.checkpoint_name = checkpoint_name
        self.places = tuple(int(p) for p in places)
        if len(set(self.places)) != len(self.places):
            raise ValueError(f"two stream offsets name the same place: {self.places}")
        self.hidden_size = hidden_size
        self.name = name
        self.rows: dict[int, torch.Tensor] = {}

    def param_specs(self) -> list[ParamSpec]:
        return [
            ParamSpec(
                self.name + ".table", (len(self.places), self.hidden_size), "vector",
                (Source(self.checkpoint_name, len(self.places)),), init="normal",
            )
        ]

    def bind(self, params, runtime) -> None:
        table = params[self.name + ".table"]
        self.rows = {place: table[t] for t, place in enumerate(self.places)}

    def add(self, residual: torch.Tensor, place: int) -> None:
        """``residual[r, :] += row`` (float32, in place) if ``place`` has a row."""
        row = self.rows.get(place)
        if row is not None:
            ops.add_bias(residual, row)
