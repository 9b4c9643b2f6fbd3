"""Fokulorn decoder: configuration -> model description, and its registry entry.

Layer ``i``'s tensors are ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*`` and ``l<i>.mlp.*``;
the two ends are ``embed``, ``final.norm`` and ``head``; ``loop.step`` holds one vector per pass
of the looped span.  A bias is its projection's name with ``.b`` added.
"""

from __future__ import annotations

from ..config.fokulorn import FokulornConfig
from ..config.registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, StreamOffsets, linear_output, token_embedding_scaled


def build_fokulorn_spec(cfg: FokulornConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "checkpoint_name": name})

    layers = []
    for i, layer in enumerate(cfg.layers):
        prefix = f"l{i}."
        m = layer.mixer
        position = PartSpec("none")
        if layer.type == "attention":
            if m.rotary_dims:
                position = PartSpec(
                    "rope",
                    {"head_dim": m.dim, "theta": m.rotary_base, "rotary_dim": m.rotary_dims, "pairing": "interleaved"},
                )
            mixer = PartSpec(
                "gqa_attention",
                {
                    "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                    "window": m.window, "softmax_scale": m.scale, "checkpoint_prefix": prefix + "mix.",
                    "q_name": "q", "k_name": "k", "o_name": "o", "values": "keys", "head_gate_name": "g",
                    "qkv_bias": True, "bias_names": {"q": "q.b", "k": "k.b"},
                },
            )
        else:
            mixer = PartSpec(
                "matrix_memory",
                {
                    "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                    "gate_cap": m.gate_cap, "norm_eps": cfg.norm_eps, "checkpoint_prefix": prefix + "mix.",
                },
            )
        ff = ff_norm = None
        if layer.mlp is not None:
            ff = PartSpec(
                "gated",
                {
                    "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "limit": layer.mlp.limit,
                    "checkpoint_prefix": prefix + "mlp.", "gate_name": "gate", "up_name": "up", "down_name": "down",
                },
            )
            ff_norm = norm(prefix + "norm2")
        layers.append(
            LayerSpec(
                mixer=mixer, feed_forward=ff, mixer_norm=norm(prefix + "norm1"), feed_forward_norm=ff_norm,
                position=position, checkpoint_prefix=prefix,
            )
        )
    offsets = StreamOffsets("loop.step", cfg.pass_places()) if cfg.loop_times else None
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        layers=tuple(layers),
        final_norm=norm("final.norm"),
        embedding=token_embedding_scaled(cfg.vocab, cfg.width, "embed", cfg.embedding_scale),
        output=linear_output(cfg.vocab, cfg.width, "head", tied=False),
        run_order=cfg.run_order(),
        stream_offsets=offsets,
    )


register_architecture("Fokulorn", FokulornConfig, build_fokulorn_spec, aliases=("fokulorn",), replace=True)
