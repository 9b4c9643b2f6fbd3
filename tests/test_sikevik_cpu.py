"""CPU tests of the Sikevik decoder: its configuration, its description as parts, its weights by
name, the cache manager's kept first pages, and the plain implementation that the GPU tests
compare the engine with."""

import copy

import pytest
import torch

from plain_sikevik import (
    bf16_round,
    plain_experts,
    plain_forward,
    plain_kept_window_mask,
    plain_relu_squared,
    plain_route,
    plain_run_order,
    plain_sink_softmax,
    plain_sinusoid,
)
from sikevik_configs import SIKE, make_weights, random_tokens, tensor_shapes

BF16_TIMES_ROUNDING = 3.0  # the GPU tests' bfloat16 bound: so many times what rounding alone does


def test_plain_tells_the_faults_the_comparison_is_there_for():
    """With the tests' weights a window one key too long or too short, a kept position too many
    or too few, a softmax without the extra term, a pass that does not take the embedding's
    output in again, a position vector that is missing or counts from 1, an expert too few or
    another factor on the experts' weights move the logits by far more than the bounds allow."""
    cfg, _page, seed = SIKE["A"]
    w = make_weights(cfg, seed, sharp=3.0)
    toks = random_tokens(70, cfg["vocab"], 9)
    want = plain_forward(cfg, w, toks)
    spread = float(want.std())
    rounded = plain_forward(cfg, w, toks, cast=bf16_round)
    bound = BF16_TIMES_ROUNDING * float(((rounded - want).square().mean(dim=1).sqrt() / spread).max())

    def off(other):
        return float(((other - want).square().mean(dim=1).sqrt() / spread).max())

    for key in ("size", "keep_first"):
        for delta in (-1, 1):
            c = copy.deepcopy(cfg)
            c["layers"][0]["mixer"]["mask"][key] += delta
            assert off(plain_forward(c, w, toks)) > 3 * bound, (key, delta)
    c = copy.deepcopy(cfg)
    c["layers"][0]["mlp"]["router"]["top"] -= 1
    assert off(plain_forward(c, w, toks)) > 3 * bound
    c = copy.deepcopy(cfg)
    # (the norm behind the feed-forward takes out most of what the experts' common factor does:
    # it only shifts them against the shared expert)
    c["layers"][0]["mlp"]["router"]["scale"] *= 4.0
    assert off(plain_forward(c, w, toks)) > 3 * bound
    w2 = dict(w)
    w2["loop.in"] = w["loop.in"].clone()
    w2["loop.in"][:, cfg["width"]:] = 0  # the embedding's output is not taken in again
    assert off(plain_forward(cfg, w2, toks)) > 3 * bound
    import plain_sikevik

    for broken in (
        dict(plain_sink_softmax=lambda s, seen: torch.softmax(s.masked_fill(~seen, float("-inf")), dim=-1)),
        dict(plain_sinusoid=lambda p, width, dtype=torch.float32: torch.zeros((p.numel(), width), dtype=dtype)),
        dict(plain_sinusoid=lambda p, width, dtype=torch.float32: plain_sinusoid(p + 1, width, dtype)),
    ):
        saved = {k: getattr(plain_sikevik, k) for k in broken}
        try:
            for k, v in broken.items():
                setattr(plain_sikevik, k, v)
            assert off(plain_forward(cfg, w, toks)) > 3 * bound, list(broken)
        finally:
            for k, v in saved.items():
                setattr(plain_sikevik, k, v)


def test_plain_mask_and_sink():
    seen = plain_kept_window_mask(12, 4, 2)
    for i in range(12):
        for j in range(12):
            assert bool(seen[i, j]) == (j <= i and (i - j < 4 or j < 2))
    assert plain_kept_window_mask(5, None, 3).equal(torch.ones(5, 5).tril().bool())
    # the sink is a softmax over one more key of score 0 whose weight is dropped
    s = torch.randn(6, 9, dtype=torch.float64) * 3
    mask = plain_kept_window_mask(9, 3, 1)[3:]
    with_key = torch.softmax(torch.cat([s.masked_fill(~mask, float("-inf")), torch.zeros(6, 1, dtype=torch.float64)], 1), 1)
    torch.testing.assert_close(plain_sink_softmax(s, mask), with_key[:, :-1])
    # large negative scores: the weights vanish instead of summing to one
    assert float(plain_sink_softmax(torch.full((1, 3), -50.0), torch.ones(1, 3, dtype=torch.bool)).sum()) < 1e-20


def test_plain_experts_equal_their_dense_form():
    """The weighted sum over a token's chosen experts equals two dense products over all experts'
    hidden units with the unchosen ones' weights at zero (the form the engine computes)."""
    torch.manual_seed(3)
    width, experts, ff, shared, top, scale = 24, 5, 7, 6, 2, 1.5
    h = torch.randn(11, width, dtype=torch.float64)
    w = {"router": torch.randn(experts, width, dtype=torch.float64), "shared.up": torch.randn(shared, width, dtype=torch.float64),
         "shared.down": torch.randn(width, shared, dtype=torch.float64)}
    for e in range(experts):
        w[f"e{e}.up"] = torch.randn(ff, width, dtype=torch.float64)
        w[f"e{e}.down"] = torch.randn(width, ff, dtype=torch.float64)
    cfg = {"router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff}, "shared": {"ff": shared}}
    want = plain_experts(h, w.__getitem__, cfg)
    chosen, weight = plain_route(h, w["router"], top, scale)
    dense = torch.zeros(11, experts, dtype=torch.float64).scatter_(1, chosen, weight.double())
    up = torch.cat([w[f"e{e}.up"] for e in range(experts)] + [w["shared.up"]])
    down = torch.cat([w[f"e{e}.down"] for e in range(experts)] + [w["shared.down"]], dim=1)
    hidden = plain_relu_squared(h @ up.T)
    hidden[:, : experts * ff] *= dense.repeat_interleave(ff, dim=1)
    torch.testing.assert_close(hidden @ down.T, want)
    torch.testing.assert_close(weight.sum(dim=1).double(), torch.full((11,), scale, dtype=torch.float64), rtol=1e-5, atol=1e-6)


def test_run_order_and_stream_mixes():
    from rapid_llm_amd.config.registry import config_from_dict

    for which, (cfg, _page, _seed) in SIKE.items():
        entry, parsed = config_from_dict(cfg)
        assert entry.name == "Sikevik"
        plain = plain_run_order(cfg)
        assert list(parsed.run_order()) == [layer for layer, _ in plain]
        assert list(parsed.pass_places()) == [place for place, (_, begins) in enumerate(plain) if begins]
        again = config_from_dict(parsed.to_dict())[1]
        assert again == parsed
        spec = entry.build_spec(parsed)
        assert spec.order() == parsed.run_order()
        assert (spec.stream_mixes is None) == ("loop" not in cfg)
        if spec.stream_mixes is not None:
            assert spec.stream_mixes.places == parsed.pass_places()
        for layer, listed in zip(parsed.layers, cfg["layers"]):
            mask = listed["mixer"].get("mask") or {}
            assert (layer.mixer.window, layer.mixer.keep_first) == (mask.get("size", 0), mask.get("keep_first", 0))


def test_every_checkpoint_tensor_is_claimed_once_and_shapes_agree():
    from rapid_llm_amd.config.registry import config_from_dict
    from rapid_llm_amd.models.causal_lm import model_param_specs
    from rapid_llm_amd.weights.loader import WeightsError, load_params

    for which, (cfg, _page, seed) in SIKE.items():
        entry, parsed = config_from_dict(cfg)
        specs = model_param_specs(entry.build_spec(parsed))
        named = {src.name: spec.source_shape(src.rows) for spec in specs for src in spec.sources if src.name}
        assert named.pop("head") == (cfg["vocab"], cfg["width"])  # stands for the embedding's table
        assert named == tensor_shapes(cfg)
        weights = make_weights(cfg, seed)
        params = load_params(specs, weights.items(), engine_dtype=torch.bfloat16, device="cpu")
        assert params["output.weight"] is params["embed.weight"]
        for spec in specs:
            assert tuple(params[spec.name].shape) == spec.shape
            offset = 0
            for src in spec.sources:
                part = params[spec.name].narrow(spec.axis, offset, src.rows)
                if src.name and src.name != "head":
                    assert torch.equal(part.float(), weights[src.name].float())
                elif not src.name:
                    assert not part.any()  # padding of a packed matrix is zeros
                offset += src.rows
        routers = [s for s in specs if s.role == "matrix_f32"]
        has_experts = any(layer["mlp"] and layer["mlp"]["kind"] == "moe" for layer in cfg["layers"])
        assert bool(routers) == has_experts and all(params[s.name].dtype == torch.float32 for s in routers)
        side_by_side = [s for s in specs if s.axis == 1]
        assert bool(side_by_side) == has_experts  # the experts' down projections share their output
        broken = dict(weights)
        del broken["final.norm"]
        broken["l0.mix.extra"] = torch.zeros(3)
        with pytest.raises(WeightsError) as err:
            load_params(specs, broken.items(), engine_dtype=torch.bfloat16, device="cpu")
        assert any("final.norm" in m for m in err.value.missing) and any("l0.mix.extra" in u for u in err.value.unexpected)


def test_random_weights_fill_side_by_side_sources(tmp_path):
    from rapid_llm_amd.weights.random_init import write_random_model

    cfg = SIKE["D"][0]
    out = write_random_model(cfg, 5, tmp_path / "m")
    from safetensors.torch import load_file

    tensors = load_file(str(out / "model.safetensors"))
    assert {k: tuple(v.shape) for k, v in tensors.items()} == tensor_shapes(cfg)


def test_configuration_refuses_what_the_design_does_not_have():
    from rapid_llm_amd.config.model_config import ConfigError
    from rapid_llm_amd.config.registry import config_from_dict

    base = SIKE["A"][0]
    for change in (
        lambda c: c["layers"][0].__setitem__("type", "convolution"),
        lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3),
        lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 300),
        lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("keep_first", -1),
        lambda c: c["layers"][0]["mlp"].__setitem__("kind", "gated"),
        lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 7),
        lambda c: c["layers"][1]["mlp"].pop("ff"),
        lambda c: c["loop"].__setitem__("stop", 9),
        lambda c: c["norm"].pop("eps"),
    ):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)


# --------------------------------------------------------------------------- #
# the cache manager: a window that keeps a request's first pages
# --------------------------------------------------------------------------- #


def _manager(window, keep, page=4, pages=40, seqs=3, longest=400):
    from rapid_llm_amd.cache.manager import CacheManager, GroupSpec

    return CacheManager([GroupSpec(0, window, (0,), keep)], pages, page, seqs, longest)


def test_kept_first_pages_survive_the_window():
    m = _manager(window=10, keep=6)  # kept: pages 0 and 1 (positions 0..7)
    m.admit("a")
    assert m.reserve("a", 50, 0)
    row = m.tables[0][m.slot_of("a")]
    first_two = [int(row[0]), int(row[1])]
    assert all(first_two) and m.trim("a", 50) > 0
    # a query at 50 reads 41..50: pages 10 on; pages 2..9 came back, 0 and 1 stay
    assert [int(p) for p in row[:2]] == first_two
    assert not row[2:10].any() and row[10:13].all()
    m.check_invariants()
    # decoding on: one page at a time, the oldest of the window comes back, the kept never
    for n in range(51, 120):
        assert m.reserve("a", n, n - 1)
        m.trim("a", n)
        assert [int(p) for p in row[:2]] == first_two
        held = int((row != 0).sum())
        assert held <= 2 + (-(-10 // 4) + 1)
    m.check_invariants()
    m.release("a")
    m.check_invariants()
    assert m.pools[0].num_free == m.pools[0].num_usable


def test_a_portion_behind_a_trimmed_prefix_needs_no_kept_page_again():
    m = _manager(window=10, keep=6)
    m.admit("a")
    assert m.reserve("a", 30, 0)
    m.trim("a", 30)
    before = m.pools[0].num_free
    need = m.pages_needed("a", 60, 30)
    assert need[0] == -(-60 // 4) - -(-30 // 4)  # only the new positions' pages
    assert m.reserve("a", 60, 30)
    assert before - m.pools[0].num_free == need[0]
    m.check_invariants()


def test_requests_shorter_than_the_kept_span_and_pages_used_again():
    m = _manager(window=5, keep=9, pages=8)  # 7 usable pages
    m.admit("a")
    assert m.reserve("a", 3, 0)  # shorter than the kept span: one page
    assert m.pools[0].num_free == 6
    m.admit("b")
    assert m.reserve("b", 24, 0)  # six pages: the pool is empty
    assert m.pools[0].num_free == 0
    m.admit("c")
    assert not m.reserve("c", 1, 0)  # all or nothing
    m.trim("b", 24)  # b keeps pages 0..2 (kept) and 5 (positions 20..23): pages 3, 4 come back
    assert m.pools[0].num_free == 2
    assert m.reserve("c", 8, 0)
    m.release("a")
    m.release("b")
    m.release("c")
    m.check_invariants()
    assert m.pools[0].num_free == 7


def test_groups_are_told_apart_by_their_kept_positions():
    from rapid_llm_amd.cache.storage import plan_groups
    from rapid_llm_amd.parts.base import CacheNeed

    needs = [
        CacheNeed.keys_and_values(2, 32, window=19, value_dim=16, keep_first=5),
        CacheNeed.keys_and_values(2, 16, window=19, value_dim=48, keep_first=5),
        CacheNeed.keys_and_values(2, 32, window=19, value_dim=16, keep_first=0),
        CacheNeed.keys_and_values(2, 32, window=0, value_dim=16, keep_first=7),
        CacheNeed.keys_and_values(2, 32, window=0),
    ]
    groups, group_of = plan_groups(needs)
    assert group_of == [0, 0, 1, 2, 2]  # without a window nothing is kept apart
    assert [(g.window, g.keep_first) for g in groups] == [(19, 5), (19, 0), (0, 0)]
    assert needs[0].paged[1].shape == (2, 16) and needs[0].paged[0].shape == (2, 32)
