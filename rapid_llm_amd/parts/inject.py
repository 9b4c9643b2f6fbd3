"""The stream mixed with the embedding's output at given places of the run order.

A model whose layers run in passes (a span of layers repeated with the same weights) may begin
every pass by taking the embedding's output in again: ``x <- M [x ; x0]``, where ``x0`` is the
stream as the embedding left it and ``M`` one matrix ``[hidden, 2 hidden]`` whose first half of
columns meets ``x``.  The two float32 streams are laid side by side in the compute type, the
product writes the new float32 stream.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import ParamSpec, Part, Source
from .linear import Linear


class StreamMix(Part):
    replayable = True

    def __init__(self, checkpoint_name: str, places: tuple[int, ...], hidden_size: int, name: str = "stream_mix"):
        self.checkpoint_name = checkpoint_name
        self.places = frozenset(int(p) for p in places)
        if len(self.places) != len(tuple(places)):
            raise ValueError(f"two stream mixes name the same place: {tuple(places)}")
        self.hidden_size = hidden_size
        self.name = name
        self.proj = Linear(2 * hidden_size, hidden_size)

    def param_specs(self) -> list[ParamSpec]:
        h = self.hidden_size
        return [ParamSpec(self.name + ".weight", (h, 2 * h), "matrix", (Source(self.checkpoint_name, h),))]

    def bind(self, params, runtime) -> None:
        self.proj.bind(params[self.name + ".weight"])
        self.dtype = runtime.dtype

    def at(self, place: int) -> bool:
        return place in self.places

    def forward(self, residual: torch.Tensor, first: torch.Tensor) -> torch.Tensor:
        """The new float32 stream ``M [residual ; first]`` (``residual`` holds every pending add)."""
        both = torch.empty((residual.shape[0], 2 * self.hidden_size), dtype=self.dtype, device=residual.device)
        ops.pair_rows(residual, first, both)
        return self.proj(both, out_dtype=torch.float32)
