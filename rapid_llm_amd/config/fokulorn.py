"""The Fokulorn decoder's typed configuration: the keys of its ``config.json``.

A Fokulorn model is a list of layers, each with one of two mixers (softmax attention over a
sliding window whose values are its keys, or a matrix-memory recurrence) and an optional
clamped gated feed-forward; a span of the layers may run several times in a row with the
same weights.  Every size and every constant that differs between models of the design is a
key here; nothing of them appears anywhere else in the package.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, normalise_dtype_name, require

MIXER_TYPES = ("attention", "mlstm")


def _positive(where: str, data: Mapping[str, Any], key: str) -> int:
    value = require(data, key, int)
    if value < 1:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {value!r}")
    return value


@dataclass(frozen=True)
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int  # size of a query or key head; the values are the keys, so also of a value head
    scale: float  # factor of the scores
    window: int  # positions a query sees, its own included; 0: all before it
    rotary_dims: int  # leading channels of a head that rotate; 0: none
    rotary_base: float

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "AttentionMixerConfig":
        heads = _positive(where, data, "heads")
        kv_heads = _positive(where, data, "kv_heads") if data.get("kv_heads") is not None else heads
        dim = _positive(where, data, "dim")
        vdim = data.get("vdim", dim)
        if vdim != dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim {vdim!r} must equal dim {dim}")
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not divisible by {kv_heads} kv_heads")
        if dim % 2 or dim > 256:
            raise ConfigError(f"{where}: the attention kernels take even head sizes up to 256, got {dim}")
        mask = data.get("mask")
        window = 0
        if mask is not None:
            window = _positive(where + ".mask", mask, "size")
        rot = data.get("rot")
        dims, base = 0, 10000.0
        if rot is not None:
            dims = _positive(where + ".rot", rot, "dims")
            base = require(rot, "base", float)
            if dims % 2 or dims > dim or not base > 0:
                raise ConfigError(f"{where}.rot: {dims} rotating channels of {dim} at base {base}")
        return cls(heads, kv_heads, dim, require(data, "scale", float), window, dims, float(base))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.dim, "scale": self.scale,
        }
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rotary_dims:
            out["rot"] = {"dims": self.rotary_dims, "base": self.rotary_base}
        return out


@dataclass(frozen=True)
class MatrixMemoryMixerConfig:
    heads: int
    dim: int  # size of a query or key head
    vdim: int  # size of a value head
    gate_cap: float  # soft cap of both gates' pre-activations

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "MatrixMemoryMixerConfig":
        cap = require(data, "gate_cap", float)
        if not cap > 0:
            raise ConfigError(f"{where}: gate_cap must be positive, got {cap!r}")
        return cls(_positive(where, data, "heads"), _positive(where, data, "dim"), _positive(where, data, "vdim"), cap)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "DenseFeedForwardConfig":
        kind = data.get("kind", "dense")
        if kind != "dense":
            raise ConfigError(f"{where}: feed-forward kind {kind!r} is not known (only 'dense')")
        limit = require(data, "limit", float)
        if not limit > 0:
            raise ConfigError(f"{where}: limit must be positive, got {limit!r}")
        return cls(_positive(where, data, "ff"), limit)

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class FokulornLayerConfig:
    type: str  # one of MIXER_TYPES
    mixer: AttentionMixerConfig | MatrixMemoryMixerConfig
    mlp: DenseFeedForwardConfig | None

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class FokulornConfig:
    architecture: str
    width: int
    vocab: int
    embedding_scale: float
    norm_eps: float
    layers: tuple[FokulornLayerConfig, ...]
    # layers loop_start .. loop_stop - 1 run loop_times times in a row; 0 times: no loop
    loop_start: int
    loop_stop: int
    loop_times: int
    torch_dtype: str
    eos_token_ids: tuple[int, ...] = ()

    # the names the rest of the engine asks any configuration for
    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None) -> "FokulornConfig":
        data = dict(data)
        if overrides:
            data.update(overrides)
        layers = []
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise ConfigError("config.json key 'layers' must list at least one layer")
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = require(entry, "type", str)
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"{where}: 'mixer' must give the mixer's sizes")
            if kind == "attention":
                parsed: Any = AttentionMixerConfig.from_dict(where + ".mixer", mixer)
            elif kind == "mlstm":
                parsed = MatrixMemoryMixerConfig.from_dict(where + ".mixer", mixer)
            else:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            mlp = entry.get("mlp")
            layers.append(FokulornLayerConfig(
                kind, parsed, DenseFeedForwardConfig.from_dict(where + ".mlp", mlp) if mlp is not None else None
            ))
        loop = data.get("loop")
        start = stop = times = 0
        if loop is not None:
            start, stop, times = (require(loop, k, int) for k in ("start", "stop", "times"))
            if times < 1 or not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop over layers {start}..{stop} x {times} does not fit {len(layers)} layers")
        embedding = data.get("embedding") or {}
        norm = data.get("norm") or {}
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        eps = require(norm, "eps", float)
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {eps!r}")
        return cls(
            architecture=require(data, "architecture", str),
            width=_positive("config.json", data, "width"),
            vocab=_positive("config.json", data, "vocab"),
            embedding_scale=float(embedding.get("scale", 1.0)),
            norm_eps=eps,
            layers=tuple(layers),
            loop_start=start, loop_stop=stop, loop_times=times,
            torch_dtype=normalise_dtype_name(data.get("torch_dtype") or data.get("dtype") or "bfloat16"),
            eos_token_ids=eos_ids,
        )

    def run_order(self) -> tuple[int, ...]:
        """Layer indices in the order they run: the looped span repeated in place."""
        n = len(self.layers)
        if not self.loop_times:
            return tuple(range(n))
        span = tuple(range(self.loop_start, self.loop_stop))
        return tuple(range(self.loop_start)) + span * self.loop_times + tuple(range(self.loop_stop, n))

    def pass_places(self) -> tuple[int, ...]:
        """Places in the run order at which a pass of the loop begins, one per pass."""
        span = self.loop_stop - self.loop_start
        return tuple(self.loop_start + t * span for t in range(self.loop_times))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.architecture,
            "width": self.width,
            "vocab": self.vocab,
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
            "torch_dtype": self.torch_dtype,
        }
        if self.loop_times:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
