"""The Sikevik decoder's typed configuration: the keys of its ``config.json``.

A Sikevik model is a list of layers with a norm before and after each sub-layer.  A layer's
mixer is softmax attention over a sliding window that also keeps a request's first positions
readable, with one more term in the softmax's denominator, a norm per head on queries and keys,
no rotation, and value heads of a size of their own.  Its feed-forward is dense, a mixture of
experts with an optional shared expert, or absent.  A span of the layers may run several times
in a row with the same weights; every pass begins by mixing the stream with the embedding's
output through a learned matrix.  The embedding is scaled and a sinusoidal position vector is
added to it; the output projection is the embedding table.  Every size and every constant
that differs between models of the design is a key here; nothing of them appears anywhere else
in the package.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, normalise_dtype_name, require

MIXER_TYPES = ("attention",)
FEED_FORWARD_KINDS = ("dense", "moe")


def _positive(where: str, data: Mapping[str, Any], key: str) -> int:
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object")
    value = require(data, key, int)
    if value < 1:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {value!r}")
    return value


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int  # size of a query or key head
    vdim: int  # size of a value head
    scale: float  # factor of the scores
    window: int  # positions a query sees, its own included; 0: all before it
    keep_first: int  # first positions of a request that stay visible behind the window

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "SinkAttentionConfig":
        heads = _positive(where, data, "heads")
        kv_heads = _positive(where, data, "kv_heads") if data.get("kv_heads") is not None else heads
        dim = _positive(where, data, "dim")
        vdim = _positive(where, data, "vdim") if data.get("vdim") is not None else dim
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not divisible by {kv_heads} kv_heads")
        if dim % 2 or dim > 256 or vdim > 256:
            raise ConfigError(
                f"{where}: the attention kernels take even key sizes and value sizes up to 256, got {dim} and {vdim}"
            )
        window = keep = 0
        mask = data.get("mask")
        if mask is not None:
            window = _positive(where + ".mask", mask, "size")
            keep = mask.get("keep_first") or 0
            if not isinstance(keep, int) or isinstance(keep, bool) or keep < 0:
                raise ConfigError(f"{where}.mask: keep_first must be a count of positions, got {keep!r}")
        return cls(heads, kv_heads, dim, vdim, require(data, "scale", float), window, int(keep))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
        }
        if self.window:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int
    kind: str = "dense"

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertsFeedForwardConfig:
    experts: int
    top: int
    router_scale: float
    expert_ff: int
    shared_ff: int  # 0: no shared expert
    kind: str = "moe"

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "kind": "moe",
            "expert": {"ff": self.expert_ff},
            "router": {"experts": self.experts, "top": self.top, "scale": self.router_scale},
        }
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _feed_forward(where: str, data: Mapping[str, Any]):
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object or null")
    kind = data.get("kind", "dense")
    if kind == "dense":
        return DenseFeedForwardConfig(_positive(where, data, "ff"))
    if kind == "moe":
        router = data.get("router")
        experts = _positive(where + ".router", router, "experts")
        top = _positive(where + ".router", router, "top")
        if top > experts:
            raise ConfigError(f"{where}.router: a token cannot use {top} of {experts} experts")
        scale = float(require(router, "scale", float)) if router.get("scale") is not None else 1.0
        shared = data.get("shared")
        return ExpertsFeedForwardConfig(
            experts, top, scale, _positive(where + ".expert", data.get("expert"), "ff"),
            _positive(where + ".shared", shared, "ff") if shared is not None else 0,
        )
    raise ConfigError(f"{where}: feed-forward kind {kind!r} is not one of {', '.join(FEED_FORWARD_KINDS)}")


@dataclass(frozen=True)
class SikevikLayerConfig:
    type: str  # one of MIXER_TYPES
    mixer: SinkAttentionConfig
    mlp: DenseFeedForwardConfig | ExpertsFeedForwardConfig | None

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class SikevikConfig:
    architecture: str
    width: int
    vocab: int
    embedding_scale: float
    norm_eps: float
    layers: tuple[SikevikLayerConfig, ...]
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
    def from_dict(cls, data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None) -> "SikevikConfig":
        data = dict(data)
        if overrides:
            data.update(overrides)
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise ConfigError("config.json key 'layers' must list at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = require(entry, "type", str)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"{where}: 'mixer' must give the mixer's sizes")
            mlp = entry.get("mlp")
            layers.append(SikevikLayerConfig(
                kind, SinkAttentionConfig.from_dict(where + ".mixer", mixer),
                _feed_forward(where + ".mlp", mlp) if mlp is not None else None,
            ))
        loop = data.get("loop")
        start = stop = times = 0
        if loop is not None:
            start, stop, times = (require(loop, k, int) for k in ("start", "stop", "times"))
            if times < 1 or not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop over layers {start}..{stop} x {times} does not fit {len(layers)} layers")
        embedding = data.get("embedding") or {}
        norm = data.get("norm") or {}
        eps = require(norm, "eps", float)
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {eps!r}")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
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
