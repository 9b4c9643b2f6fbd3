"""Plain, slow implementation of the Fokulorn decoder, used only as the test oracle.

Whole sequences, dense masks, token-by-token recurrences, no cache, no paging, one function
per mechanism.  It shares no code with ``rapid_llm_amd``: it takes a ``config.json`` body as
a dict and the weights as a dict of tensors under their checkpoint names, and computes every
formula in one floating type (float32 by default, float64 when a tighter oracle is wanted).

Notation: ``T`` tokens, ``W`` model width, ``H`` heads, ``G`` key/value heads, ``dk`` the size
of a query or key head, ``dv`` of a value head.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- #
# mechanisms
# --------------------------------------------------------------------------- #


def plain_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return plain_rms(x, eps) * weight


def plain_rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """Rotate the first ``dims`` channels of every head of ``x [T, heads, d]``: channels
    ``(2i, 2i + 1)`` turn by the angle ``p * base^(-2i/dims)``; the other channels pass."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims)).to(torch.float32)
    ang = (positions.to(torch.float32)[:, None] * freq[None, :]).to(torch.float64)
    c = ang.cos().to(x.dtype)[:, None, :]
    s = ang.sin().to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def plain_window_mask(t: int, window: int | None) -> torch.Tensor:
    """``[t, t]`` bool: query i sees key j when ``0 <= i - j < window`` (no window: ``j <= i``)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    seen = j <= i
    if window:
        seen &= (i - j) < window
    return seen


def plain_softmax_attention(q, k, v, scale: float, window: int | None) -> torch.Tensor:
    """``q [T, H, dk]``, ``k [T, G, dk]``, ``v [T, G, dv]`` -> ``[T, H, dv]``; query head ``h``
    reads key/value head ``h // (H / G)``."""
    t, heads, _ = q.shape
    group = heads // k.shape[1]
    seen = plain_window_mask(t, window)
    out = torch.empty((t, heads, v.shape[-1]), dtype=q.dtype)
    for h in range(heads):
        g = h // group
        score = (q[:, h] @ k[:, g].T) * scale
        score = score.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(score, dim=-1) @ v[:, g]
    return out


def _same(x):
    return x


def plain_keyvalue_attention(h, w, p, cfg, positions=None, cast=_same) -> torch.Tensor:
    """The softmax mixer whose values are its keys: ``v`` is the key projection before the
    rotation.  ``w(name)`` returns the mixer's tensor ``name``; ``cfg`` is its ``mixer`` dict.
    ``cast`` rounds what an engine would store in its compute type (projections, rotated
    heads, the heads' outputs)."""
    t = h.shape[0]
    heads, kv, dk = cfg["heads"], cfg["kv_heads"], cfg["dim"]
    positions = torch.arange(t) if positions is None else positions
    q = cast(h @ w("q").T + w("q.b")).view(t, heads, dk)
    k = cast(h @ w("k").T + w("k.b")).view(t, kv, dk)
    v = k
    rot = cfg.get("rot")
    if rot:
        q = cast(plain_rotate_interleaved(q, positions, rot["dims"], rot["base"]))
        k = cast(plain_rotate_interleaved(k, positions, rot["dims"], rot["base"]))
    mask = cfg.get("mask")
    o = cast(plain_softmax_attention(q, k, v, cfg["scale"], mask["size"] if mask else None))
    gate = torch.sigmoid(cast(h @ w("g").T))  # [T, H]: one number a head
    o = cast(o * gate[:, :, None])
    return cast(o.reshape(t, heads * v.shape[-1]) @ w("o").T)


def plain_mlstm_gates(h, w, cap: float):
    """Log input gate and log forget gate, ``[T, H]`` each, both softly capped at ``cap``."""
    i = cap * torch.tanh((h @ w("i").T + w("i.b")) / cap)
    f = F.logsigmoid(cap * torch.tanh((h @ w("f").T + w("f.b")) / cap))
    return i, f


def plain_mlstm_scan(q, k, v, i, f, state=None):
    """The matrix-memory recurrence, token by token.  ``q, k [T, H, dk]`` (``q`` already scaled),
    ``v [T, H, dv]``, ``i, f [T, H]``.  ``state = (S [H, dk, dv], n [H, dk], m [H])`` starts at
    zero, the running maximum too.  Returns ``o [T, H, dv]`` and the state after the last token."""
    t, heads, dk = q.shape
    dv = v.shape[-1]
    if state is None:
        state = (
            torch.zeros((heads, dk, dv), dtype=q.dtype),
            torch.zeros((heads, dk), dtype=q.dtype),
            torch.zeros((heads,), dtype=q.dtype),
        )
    S, n, m = (x.clone() for x in state)
    out = torch.empty((t, heads, dv), dtype=q.dtype)
    for step in range(t):
        m_new = torch.maximum(f[step] + m, i[step])
        keep = torch.exp(f[step] + m - m_new)
        take = torch.exp(i[step] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * (k[step][:, :, None] * v[step][:, None, :])
        n = keep[:, None] * n + take[:, None] * k[step]
        m = m_new
        num = torch.einsum("hkv,hk->hv", S, q[step])
        den = torch.maximum((n * q[step]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[step] = num / den[:, None]
    return out, (S, n, m)


def plain_mlstm(h, w, cfg, eps: float, cast=_same) -> torch.Tensor:
    """The matrix-memory mixer: projections, gates, recurrence, per-head unit RMS, the
    weight over all heads, the sigmoid gate, the output projection.  ``cast`` rounds the
    projections and the finished heads; gates, state and recurrence are never rounded."""
    t = h.shape[0]
    heads, dk, dv = cfg["heads"], cfg["dim"], cfg["vdim"]
    q = cast(h @ w("q").T).view(t, heads, dk) * dk ** -0.5
    k = cast(h @ w("k").T).view(t, heads, dk)
    v = cast(h @ w("v").T).view(t, heads, dv)
    i, f = plain_mlstm_gates(h, w, cfg["gate_cap"])
    o, _ = plain_mlstm_scan(q, k, v, i, f)
    o = plain_rms(o, eps).reshape(t, heads * dv) * w("norm")
    o = cast(o * torch.sigmoid(cast(h @ w("g").T)))
    return cast(o @ w("o").T)


def plain_clamped_glu(h, w, cfg, cast=_same) -> torch.Tensor:
    """``down(g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(gate(h), limit)`` and
    ``u = clamp(up(h), -limit, limit)``."""
    limit = cfg["limit"]
    g = cast(h @ w("gate").T).clamp(max=limit)
    u = cast(h @ w("up").T).clamp(-limit, limit)
    return cast(cast(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w("down").T)


# --------------------------------------------------------------------------- #
# the model
# --------------------------------------------------------------------------- #


def plain_run_order(cfg) -> list[tuple[int, int | None]]:
    """``(layer, pass)`` in the order the layers run; ``pass`` is the number of the loop's pass
    at the pass's first layer and ``None`` elsewhere."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] < 1 or loop["stop"] <= loop["start"]:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            order.append((i, t if i == loop["start"] else None))
    order += [(i, None) for i in range(loop["stop"], n)]
    return order


def plain_forward(cfg, weights, tokens, dtype=torch.float32, streams: list | None = None, cast=_same) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``streams``, when given, receives the residual
    stream after every layer run.  ``cast`` rounds every activation that an engine stores in
    its compute type (never the residual stream, gates or recurrent state): with a bfloat16
    rounding it measures what rounding alone does to the logits."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for layer, new_pass in plain_run_order(cfg):
        if new_pass is not None:
            x = x + W["loop.step"][new_pass]
        spec = cfg["layers"][layer]
        pre = f"l{layer}."

        def mix(name, pre=pre):
            return W[pre + "mix." + name]

        def mlp(name, pre=pre):
            return W[pre + "mlp." + name]

        h = cast(plain_rmsnorm(x, W[pre + "norm1"], eps))
        if spec["type"] == "attention":
            x = x + plain_keyvalue_attention(h, mix, None, spec["mixer"], cast=cast)
        elif spec["type"] == "mlstm":
            x = x + plain_mlstm(h, mix, spec["mixer"], eps, cast=cast)
        else:
            raise ValueError(f"unknown mixer {spec['type']!r}")
        if spec.get("mlp") is not None:
            h = cast(plain_rmsnorm(x, W[pre + "norm2"], eps))
            x = x + plain_clamped_glu(h, mlp, spec["mlp"], cast=cast)
        if streams is not None:
            streams.append(x.clone())
    x = cast(plain_rmsnorm(x, W["final.norm"], eps))
    return x @ W["head"].T

