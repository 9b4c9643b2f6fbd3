"""Plain, slow implementation of the Sikevik decoder, used only as the test oracle.

Whole sequences, dense masks, every expert as a loop over tokens, no cache, no paging, one
function per mechanism.  It shares no code with ``rapid_llm_amd``: it takes a ``config.json``
body as a dict and the weights as a dict of tensors under their checkpoint names, and computes
every formula in one floating type (float32 by default, float64 for a tighter oracle).

Notation: ``T`` tokens, ``W`` model width, ``H`` query heads, ``G`` key/value heads, ``dk`` the
size of a query or key head, ``dv`` of a value head, ``E`` experts of which a token uses ``top``.
"""

from __future__ import annotations

import math

import torch


def _same(x):
    return x


# --------------------------------------------------------------------------- #
# mechanisms
# --------------------------------------------------------------------------- #


def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * weight`` over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def plain_sinusoid(positions: torch.Tensor, width: int, dtype=torch.float32) -> torch.Tensor:
    """``[T, width]``: column ``2i`` is ``sin(p * 10000^(-2i/width))``, column ``2i + 1`` the
    cosine of the same angle.  Angles are float32 products, as an engine computes them."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    freq = (10000.0 ** (-2.0 * i / width)).to(torch.float32)
    ang = (positions.to(torch.float32)[:, None] * freq[None, :]).to(torch.float64)
    out = torch.zeros((positions.numel(), 2 * freq.numel()), dtype=torch.float64)
    out[:, 0::2] = ang.sin()
    out[:, 1::2] = ang.cos()
    return out[:, :width].to(dtype)


def plain_embedding(tokens: torch.Tensor, table: torch.Tensor, scale: float, positions=None) -> torch.Tensor:
    positions = torch.arange(tokens.numel()) if positions is None else positions
    return table[tokens] * scale + plain_sinusoid(positions, table.shape[1], table.dtype)


def plain_kept_window_mask(t: int, window: int | None, keep_first: int) -> torch.Tensor:
    """``[t, t]`` bool: query i sees key j when ``j <= i`` and (``i - j < window`` or
    ``j < keep_first``); no window: every ``j <= i``."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    seen = j <= i
    if window:
        seen &= ((i - j) < window) | (j < keep_first)
    return seen


def plain_sink_softmax(score: torch.Tensor, seen: torch.Tensor) -> torch.Tensor:
    """``p_j = exp(s_j) / (1 + sum_j exp(s_j))`` over the seen keys of every row: a softmax
    with one more key whose score is 0 and which carries no value."""
    score = score.masked_fill(~seen, float("-inf"))
    top = torch.clamp(score.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(score - top)
    return e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))


def plain_sink_attention(q, k, v, scale: float, window: int | None, keep_first: int) -> torch.Tensor:
    """``q [T, H, dk]``, ``k [T, G, dk]``, ``v [T, G, dv]`` -> ``[T, H, dv]``; query head ``h``
    reads key/value head ``h // (H / G)``."""
    t, heads, _ = q.shape
    group = heads // k.shape[1]
    seen = plain_kept_window_mask(t, window, keep_first)
    out = torch.empty((t, heads, v.shape[-1]), dtype=q.dtype)
    for h in range(heads):
        g = h // group
        p = plain_sink_softmax((q[:, h] @ k[:, g].T) * scale, seen)
        out[:, h] = p @ v[:, g]
    return out


def plain_attention_mixer(h, w, cfg, eps: float, cast=_same) -> torch.Tensor:
    """The attention mixer: projections without bias, a norm per head over ``dk`` on queries and
    keys (one weight vector shared by the heads), no rotation, the kept-window mask, the sink
    softmax, the output projection.  ``w(name)`` returns the mixer's tensor ``name``."""
    t = h.shape[0]
    heads, kv, dk = cfg["heads"], cfg.get("kv_heads") or cfg["heads"], cfg["dim"]
    dv = cfg.get("vdim", dk)
    q = cast(h @ w("q").T).view(t, heads, dk)
    k = cast(h @ w("k").T).view(t, kv, dk)
    v = cast(h @ w("v").T).view(t, kv, dv)
    q = cast(plain_rmsnorm(q, w("q.norm"), eps))
    k = cast(plain_rmsnorm(k, w("k.norm"), eps))
    mask = cfg.get("mask") or {}
    o = cast(plain_sink_attention(q, k, v, cfg["scale"], mask.get("size"), mask.get("keep_first", 0)))
    return cast(o.reshape(t, heads * dv) @ w("o").T)


def plain_gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def plain_relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z) ** 2


def plain_two_layer(h, up, down, act, cast=_same) -> torch.Tensor:
    """``down act(up h)`` for rows ``h``."""
    return cast(cast(act(cast(h @ up.T))) @ down.T)


def plain_route(h, router, top: int, scale: float):
    """Chosen experts ``[T, top]`` and their weights: the softmax scores of the chosen ones,
    divided by their sum (+ 1e-20), times ``scale``."""
    s = torch.softmax(h.to(torch.float32) @ router.to(torch.float32).T, dim=-1)
    score, chosen = torch.topk(s, top, dim=-1)
    return chosen, score / (score.sum(dim=-1, keepdim=True) + 1e-20) * scale


def plain_experts(h, w, cfg, cast=_same) -> torch.Tensor:
    """Mixture of experts, token by token: the weighted sum of the chosen experts' outputs,
    plus the shared expert where the configuration has one."""
    r = cfg["router"]
    chosen, weight = plain_route(h, w("router"), r["top"], r["scale"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t].tolist()):
            out[t] += g * plain_two_layer(h[t : t + 1], w(f"e{e}.up"), w(f"e{e}.down"), plain_relu_squared, cast)[0]
    if cfg.get("shared"):
        out = out + plain_two_layer(h, w("shared.up"), w("shared.down"), plain_relu_squared, cast)
    return cast(out)


def plain_feed_forward(h, w, cfg, cast=_same) -> torch.Tensor:
    if cfg["kind"] == "dense":
        return plain_two_layer(h, w("up"), w("down"), plain_gelu_tanh, cast)
    if cfg["kind"] == "moe":
        return plain_experts(h, w, cfg, cast)
    raise ValueError(cfg["kind"])


# --------------------------------------------------------------------------- #
# the model
# --------------------------------------------------------------------------- #


def plain_run_order(config: dict) -> list[tuple[int, bool]]:
    """``(layer, whether a pass of the loop begins here)`` in the order the layers run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    span = list(range(loop["start"], loop["stop"]))
    order = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(i, i == span[0]) for i in span]
    return order + [(i, False) for i in range(loop["stop"], n)]


def plain_forward(config: dict, weights: dict, tokens, dtype=torch.float32, cast=_same, trace=None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.  ``trace``: a list that receives the stream
    after every layer run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = plain_embedding(tokens, W["embed"], (config.get("embedding") or {}).get("scale", 1.0))
    x = x0
    for li, pass_begins in plain_run_order(config):
        layer = config["layers"][li]
        p = f"l{li}."
        if pass_begins:
            x = cast(torch.cat([cast(x), cast(x0)], dim=-1)) @ W["loop.in"].T
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        a = plain_attention_mixer(
            cast(plain_rmsnorm(x, W[p + "norm1"], eps)), lambda n: W[p + "mix." + n], layer["mixer"], eps, cast
        )
        x = x + plain_rmsnorm(a, W[p + "norm1b"], eps)
        if layer.get("mlp"):
            f = plain_feed_forward(
                cast(plain_rmsnorm(x, W[p + "norm2"], eps)), lambda n: W[p + "mlp." + n], layer["mlp"], cast
            )
            x = x + plain_rmsnorm(f, W[p + "norm2b"], eps)
        if trace is not None:
            trace.append(x.clone())
    return cast(plain_rmsnorm(x, W["final.norm"], eps)) @ W["embed"].T


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """What a bfloat16 engine stores: the value rounded to bfloat16, in the oracle's type."""
    return x.to(torch.bfloat16).to(x.dtype)
