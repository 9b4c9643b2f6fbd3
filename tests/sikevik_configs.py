"""Small Sikevik configurations that differ in every size and option, and random weights for
them, made here tensor by tensor (names and shapes written out once more, independent of the
package's own list of parameters)."""

from __future__ import annotations

import json
import random
from pathlib import Path

import torch


def _attn(heads, kv, dim, vdim, scale, window=None, keep=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
        if keep is not None:
            m["mask"]["keep_first"] = keep
    return m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, scale, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


# A: value heads narrower than key heads (32 / 16) and wider (16 / 48); groups of 2 and 3 query
# heads a kv head; a window of 19 with 5 kept positions (less than a page) and one of 41 with 21
# kept (more than two pages); experts first, then a dense layer, then a layer without a
# feed-forward; the middle two layers run three times; pages of 8
SIKE_A = {
    "architecture": "Sikevik", "width": 96, "vocab": 211, "embedding": {"scale": 7.5}, "norm": {"eps": 3e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 32, 16, 0.2, 19, 5), "mlp": _moe(6, 2, 1.5, 40, 56)},
        {"type": "attention", "mixer": _attn(6, 2, 16, 48, 0.3, 41, 21), "mlp": _dense(136)},
        {"type": "attention", "mixer": _attn(4, 2, 32, 16, 0.2, 19, 5), "mlp": None},
        {"type": "attention", "mixer": _attn(3, 3, 16, 16, 0.25, 33, 8), "mlp": _moe(4, 4, 1.0, 24)},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
PAGE_A = 8

# B: one head everywhere, equal key and value sizes, a window of five keys with one kept (the
# smallest of each), an expert layer where a token uses one expert of three and no shared
# expert, a loop of one pass over the first layer only, pages of 4
SIKE_B = {
    "architecture": "Sikevik", "width": 64, "vocab": 130, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(1, 1, 16, 16, 0.25, 5, 1), "mlp": _moe(3, 1, 2.5, 32)},
        {"type": "attention", "mixer": _attn(2, 1, 32, 32, 0.15, 5, 1), "mlp": _dense(48)},
    ],
    "loop": {"start": 0, "stop": 1, "times": 1},
}
PAGE_B = 4

# C: no loop at all (and no matrix for it), one layer without any mask (every earlier key is seen),
# one with a window longer than most requests and no kept positions, eight query heads on two kv
# heads, key heads of 64 with value heads of 32 and of 128, pages of 16
SIKE_C = {
    "architecture": "Sikevik", "width": 128, "vocab": 300, "embedding": {"scale": 11.0}, "norm": {"eps": 2e-5},
    "layers": [
        {"type": "attention", "mixer": _attn(8, 2, 64, 32, 0.11), "mlp": _dense(200)},
        {"type": "attention", "mixer": _attn(4, 4, 64, 128, 0.09, 130, 0), "mlp": _moe(8, 3, 1.75, 48, 64)},
        {"type": "attention", "mixer": _attn(8, 2, 64, 32, 0.11, 64, 64), "mlp": None},
    ],
}
PAGE_C = 16

# D: sizes that no vector access divides and head sizes between the matrix cores' steps (key
# heads of 18 and 12, value heads of 10 and 22, width 100, vocabulary 97, feed-forward widths 50
# and 27): every kernel takes its element-by-element path and the bfloat16 products go to the
# library; a window of one key with three kept; a loop over the last two layers
SIKE_D = {
    "architecture": "Sikevik", "width": 100, "vocab": 97, "embedding": {"scale": 10.0}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": _attn(5, 5, 18, 10, 0.3, 1, 3), "mlp": _dense(50)},
        {"type": "attention", "mixer": _attn(3, 1, 12, 22, 0.2, 33, 9), "mlp": _moe(5, 2, 0.5, 27, 9)},
        {"type": "attention", "mixer": _attn(5, 5, 18, 10, 0.3, 7, 0), "mlp": None},
    ],
    "loop": {"start": 1, "stop": 3, "times": 2},
}
PAGE_D = 8

SIKE = {"A": (SIKE_A, PAGE_A, 401), "B": (SIKE_B, PAGE_B, 402), "C": (SIKE_C, PAGE_C, 403), "D": (SIKE_D, PAGE_D, 404)}


def tensor_shapes(cfg) -> dict[str, tuple[int, ...]]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    if cfg.get("loop"):
        out["loop.in"] = (w, 2 * w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        out[p + "norm1b"] = (w,)
        out[p + "mix.q"] = (m["heads"] * m["dim"], w)
        out[p + "mix.k"] = (m["kv_heads"] * m["dim"], w)
        out[p + "mix.v"] = (m["kv_heads"] * m["vdim"], w)
        out[p + "mix.q.norm"] = (m["dim"],)
        out[p + "mix.k.norm"] = (m["dim"],)
        out[p + "mix.o"] = (w, m["heads"] * m["vdim"])
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = (w,)
        out[p + "norm2b"] = (w,)
        if mlp["kind"] == "dense":
            out[p + "mlp.up"] = (mlp["ff"], w)
            out[p + "mlp.down"] = (w, mlp["ff"])
        else:
            out[p + "mlp.router"] = (mlp["router"]["experts"], w)
            for e in range(mlp["router"]["experts"]):
                out[p + f"mlp.e{e}.up"] = (mlp["expert"]["ff"], w)
                out[p + f"mlp.e{e}.down"] = (w, mlp["expert"]["ff"])
            if mlp.get("shared"):
                out[p + "mlp.shared.up"] = (mlp["shared"]["ff"], w)
                out[p + "mlp.shared.down"] = (w, mlp["shared"]["ff"])
    return out


def make_weights(cfg, seed: int, sharp: float = 1.0) -> dict[str, torch.Tensor]:
    """Weights as a bfloat16 checkpoint stores them.  Projections are drawn at the scale that
    keeps activations of order one, so that scores differ; the router's rows are large, so that
    the experts' scores lie far apart and no choice hangs on rounding; the head norms' weights
    are multiplied by ``sharp``: few keys then carry each query's weight, and a key lost at a
    window's edge or among the kept ones moves the output."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = torch.randn(shape, generator=gen) * 0.5
        elif name.endswith("q.norm"):
            t = (1.0 + 0.1 * torch.randn(shape, generator=gen)) * sharp
        elif "norm" in last:
            t = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        elif last == "router":
            t = torch.randn(shape, generator=gen) * (6.0 / shape[-1] ** 0.5)
        elif name == "loop.in":
            t = torch.randn(shape, generator=gen) * (1.0 / shape[0] ** 0.5)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / shape[-1] ** 0.5)
        out[name] = t
    return {name: t.to(torch.bfloat16) for name, t in out.items()}


def make_model_dir(tmp_path: Path, which: str, sharp: float = 1.0, cfg=None, seed: int | None = None) -> Path:
    from safetensors.torch import save_file

    base, _page, base_seed = SIKE[which]
    cfg = cfg or base
    out = Path(tmp_path) / f"sike_{which}_{sharp}_{seed}"
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
