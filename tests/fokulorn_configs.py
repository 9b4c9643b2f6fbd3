"""Small Fokulorn configurations that differ in every size and option, and random weights for
them, made here tensor by tensor (names and shapes written out once more, independent of the
package's own list of parameters)."""

from __future__ import annotations

import json
import random
from pathlib import Path

import torch


def _attn(heads, kv, dim, scale, window=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return m


def _mem(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# P: attention first, two kv heads (groups of 2) and as many kv heads as query heads, the whole
# head rotating and a quarter of it, a window shorter than three pages; recurrences with and
# without a feed-forward; the middle two layers run three times; a scale that is no power of two
FOKU_P = {
    "architecture": "Fokulorn", "width": 96, "vocab": 211, "embedding": {"scale": 7.5}, "norm": {"eps": 3e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 32, 0.2, 19, (32, 10000.0)), "mlp": _mlp(136, 1.5)},
        {"type": "mlstm", "mixer": _mem(3, 16, 40, 10.0), "mlp": None},
        {"type": "mlstm", "mixer": _mem(2, 48, 24, 8.0), "mlp": _mlp(72, 3.0)},
        {"type": "attention", "mixer": _attn(6, 6, 16, 0.3, 40, (8, 500.0)), "mlp": None},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
PAGE_P = 8

# Q: one head everywhere, a head size that is no multiple of 8 (20), a window of five
# keys (one page and a bit), a loop of one pass over the first layer only, the smallest sizes
FOKU_Q = {
    "architecture": "Fokulorn", "width": 64, "vocab": 130, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mlstm", "mixer": _mem(1, 8, 8, 20.0), "mlp": _mlp(48, 0.75)},
        {"type": "attention", "mixer": _attn(2, 1, 20, 0.25, 5, (10, 77.0)), "mlp": None},
    ],
    "loop": {"start": 0, "stop": 1, "times": 1},
}
PAGE_Q = 4

# R: no loop at all, no rotation, a window longer than most requests, eight query heads on two
# kv heads, a recurrence whose state rows are split over four lanes (key size 80)
FOKU_R = {
    "architecture": "Fokulorn", "width": 128, "vocab": 300, "embedding": {"scale": 11.0}, "norm": {"eps": 2e-5},
    "layers": [
        {"type": "mlstm", "mixer": _mem(2, 80, 72, 12.0), "mlp": None},
        {"type": "attention", "mixer": _attn(8, 2, 64, 0.11, 130), "mlp": _mlp(200, 2.5)},
        {"type": "mlstm", "mixer": _mem(4, 32, 32, 15.0), "mlp": _mlp(96, 4.0)},
    ],
}
PAGE_R = 16

# S: sizes that no vector access divides (width 100 = 4 * 25, feed-forward 50 and 27, vocabulary 97,
# key sizes 12 and 6, value sizes 10 and 22, an attention head of 18 channels of which 6 rotate): every
# kernel takes its element-by-element path and the bfloat16 products go to the library; two windows
# (two pools of pages), one of them a single key; a loop over the last two layers
FOKU_S = {
    "architecture": "Fokulorn", "width": 100, "vocab": 97, "embedding": {"scale": 10.0}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": _attn(5, 5, 18, 0.3, 1, (6, 3000.0)), "mlp": _mlp(50, 2.0)},
        {"type": "mlstm", "mixer": _mem(5, 12, 10, 6.0), "mlp": _mlp(27, 1.0)},
        {"type": "attention", "mixer": _attn(3, 1, 18, 0.2, 33, (18, 100.0)), "mlp": None},
        {"type": "mlstm", "mixer": _mem(2, 6, 22, 30.0), "mlp": None},
    ],
    "loop": {"start": 2, "stop": 4, "times": 2},
}
PAGE_S = 8

# T: recurrent layers only (no pages, no block tables: the cache is state slots alone), looped twice
FOKU_T = {
    "architecture": "Fokulorn", "width": 72, "vocab": 150, "embedding": {"scale": 4.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mlstm", "mixer": _mem(3, 24, 16, 9.0), "mlp": _mlp(40, 5.0)},
        {"type": "mlstm", "mixer": _mem(2, 16, 56, 14.0), "mlp": None},
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}
PAGE_T = 16

FOKU = {"P": (FOKU_P, PAGE_P, 301), "Q": (FOKU_Q, PAGE_Q, 302), "R": (FOKU_R, PAGE_R, 303), "S": (FOKU_S, PAGE_S, 304),
        "T": (FOKU_T, PAGE_T, 305)}


def tensor_shapes(cfg) -> dict[str, tuple[int, ...]]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,), "head": (cfg["vocab"], w)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            out[p + "mix.q"] = (m["heads"] * m["dim"], w)
            out[p + "mix.q.b"] = (m["heads"] * m["dim"],)
            out[p + "mix.k"] = (m["kv_heads"] * m["dim"], w)
            out[p + "mix.k.b"] = (m["kv_heads"] * m["dim"],)
            out[p + "mix.g"] = (m["heads"], w)
            out[p + "mix.o"] = (w, m["heads"] * m["vdim"])
        else:
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out[p + "mix.q"] = (qk, w)
            out[p + "mix.k"] = (qk, w)
            out[p + "mix.v"] = (vv, w)
            out[p + "mix.g"] = (vv, w)
            out[p + "mix.o"] = (w, vv)
            out[p + "mix.norm"] = (vv,)
            for gate in ("i", "f"):
                out[p + f"mix.{gate}"] = (m["heads"], w)
                out[p + f"mix.{gate}.b"] = (m["heads"],)
        if layer["mlp"] is not None:
            out[p + "norm2"] = (w,)
            out[p + "mlp.gate"] = (layer["mlp"]["ff"], w)
            out[p + "mlp.up"] = (layer["mlp"]["ff"], w)
            out[p + "mlp.down"] = (w, layer["mlp"]["ff"])
    return out


def make_weights(cfg, seed: int, sharp: float = 1.0) -> dict[str, torch.Tensor]:
    """Weights as a bfloat16 checkpoint stores them.  Projections are drawn at the scale that
    keeps activations of order one, so that scores differ, gates move and the clamps of the
    feed-forward are reached; forget gates lean towards keeping (a memory of hundreds of
    tokens); its keys lean towards its queries.  ``sharp`` multiplies the attention's query projections: few keys then carry each
    query's weight, and a key lost at a window's edge moves the output."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name in ("embed",):
            t = torch.randn(shape, generator=gen) * 0.5
        elif "norm" in last:
            t = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        elif name == "loop.step":
            t = torch.randn(shape, generator=gen) * 0.5
        elif name.endswith("f.b"):
            t = 3.0 + torch.randn(shape, generator=gen)
        elif last == "b":
            t = torch.randn(shape, generator=gen) * 0.5
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / shape[-1] ** 0.5)
            if name.endswith("mix.q") and f"{name[:-1]}q.b" in tensor_shapes(cfg):
                t = t * sharp
        out[name] = t
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] == "mlstm":
            # a token's key points roughly where its query does, so that q . k of a token with
            # itself is safely positive: where it is near zero the output's sign hangs on the
            # last bit (the output is divided by |n . q|), and no two roundings agree there
            out[f"l{i}.mix.k"] = 0.8 * out[f"l{i}.mix.q"] + 0.6 * out[f"l{i}.mix.k"]
    return {name: t.to(torch.bfloat16) for name, t in out.items()}


def make_model_dir(tmp_path: Path, which: str, sharp: float = 1.0, cfg=None, seed: int | None = None) -> Path:
    from safetensors.torch import save_file

    base, _page, base_seed = FOKU[which]
    cfg = cfg or base
    out = Path(tmp_path) / f"foku_{which}_{sharp}_{seed}"
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(cfg))
    save_file(make_weights(cfg, base_seed if seed is None else seed, sharp), str(out / "model.safetensors"))
    return out


def load_plain(model_dir: Path):
    from safetensors.torch import load_file

    return json.loads((Path(model_dir) / "config.json").read_text()), load_file(str(Path(model_dir) / "model.safetensors"))


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]
