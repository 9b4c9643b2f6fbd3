"""Sikevik decoder: configuration -> model description, and its registry entry.

Layer ``i``'s tensors are ``l<i>.norm1``, ``l<i>.norm1b`` (before and behind the mixer),
``l<i>.norm2``, ``l<i>.norm2b`` (before and behind the feed-forward), ``l<i>.mix.*`` and
``l<i>.mlp.*`` (experts ``e<n>.up`` / ``e<n>.down``, ``router``, ``shared.up`` / ``shared.down``);
the two ends are ``embed`` (also the output projection) and ``final.norm``; ``loop.in`` is the
matrix that mixes the stream with the embedding's output at the start of every pass.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.sikevik import ExpertsFeedForwardConfig, SikevikConfig
from .spec import LayerSpec, ModelSpec, PartSpec, StreamMixes, linear_output, token_embedding_scaled

SINUSOID_BASE = 10000.0  # the design fixes it
DENSE_ACTIVATION = "gelu_tanh"
EXPERT_ACTIVATION = "relu_squared"


def build_sikevik_spec(cfg: SikevikConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "checkpoint_name": name})

    layers = []
    for i, layer in enumerate(cfg.layers):
        prefix = f"l{i}."
        m = layer.mixer
        mixer = PartSpec(
            "gqa_attention",
            {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "value_dim": m.vdim, "window": m.window, "keep_first": m.keep_first, "sink": True,
                "softmax_scale": m.scale, "qk_norm_eps": cfg.norm_eps, "checkpoint_prefix": prefix + "mix.",
                "q_name": "q", "k_name": "k", "v_name": "v", "o_name": "o",
                "q_norm_name": "q.norm", "k_norm_name": "k.norm",
            },
        )
        ff = ff_norm = ff_post = None
        if layer.mlp is not None:
            if isinstance(layer.mlp, ExpertsFeedForwardConfig):
                ff = PartSpec(
                    "routed_experts",
                    {
                        "hidden_size": cfg.width, "num_experts": layer.mlp.experts, "top": layer.mlp.top,
                        "expert_size": layer.mlp.expert_ff, "shared_size": layer.mlp.shared_ff,
                        "route_scale": layer.mlp.router_scale, "activation": EXPERT_ACTIVATION,
                        "checkpoint_prefix": prefix + "mlp.",
                    },
                )
            else:
                ff = PartSpec(
                    "two_layer",
                    {
                        "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff,
                        "activation": DENSE_ACTIVATION, "checkpoint_prefix": prefix + "mlp.",
                    },
                )
            ff_norm = norm(prefix + "norm2")
            ff_post = norm(prefix + "norm2b")
        layers.append(
            LayerSpec(
                mixer=mixer, feed_forward=ff, mixer_norm=norm(prefix + "norm1"), feed_forward_norm=ff_norm,
                block=PartSpec("sandwich"), checkpoint_prefix=prefix,
                mixer_post_norm=norm(prefix + "norm1b"), feed_forward_post_norm=ff_post,
            )
        )
    mixes = StreamMixes("loop.in", cfg.pass_places()) if cfg.loop_times else None
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        layers=tuple(layers),
        final_norm=norm("final.norm"),
        embedding=token_embedding_scaled(cfg.vocab, cfg.width, "embed", cfg.embedding_scale, SINUSOID_BASE),
        # the output projection is the embedding's table: the checkpoint ships no tensor of its own
        output=linear_output(cfg.vocab, cfg.width, "head", tied=True),
        run_order=cfg.run_order(),
        stream_mixes=mixes,
    )


register_architecture("Sikevik", SikevikConfig, build_sikevik_spec, aliases=("sikevik",), replace=True)
