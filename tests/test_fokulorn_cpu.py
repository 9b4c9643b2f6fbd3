"""CPU tests of the Fokulorn decoder: its configuration, its description as parts, its weights
by name, and the plain implementation that the GPU tests compare the engine with."""

import copy

import pytest
import torch

from fokulorn_configs import FOKU, make_weights, random_tokens, tensor_shapes
from plain_fokulorn import plain_forward, plain_mlstm_scan, plain_run_order, plain_window_mask

BF16_TIMES_ROUNDING = 3.0  # the GPU tests' bfloat16 bound: so many times what rounding alone does


def test_plain_tells_a_window_one_key_off_and_a_lost_state():
    """The GPU comparison would see the faults it is there for: with the tests' weights a window
    one key too long or too short, a state that starts again in the middle of a request or a
    missing pass vector move the logits by far more than the bounds allow."""
    cfg, _page, seed = FOKU["P"]
    w = make_weights(cfg, seed, sharp=4.0)
    toks = random_tokens(60, cfg["vocab"], 9)
    want = plain_forward(cfg, w, toks)
    spread = float(want.std())
    rounded = plain_forward(cfg, w, toks, cast=lambda x: x.bfloat16().to(x.dtype))
    BF16_ROW = BF16_TIMES_ROUNDING * float(((rounded - want).square().mean(dim=1).sqrt() / spread).max())

    def off(other):
        return float(((other - want).square().mean(dim=1).sqrt() / spread).max())

    for delta in (-1, 1):
        c = copy.deepcopy(cfg)
        c["layers"][0]["mixer"]["mask"]["size"] += delta
        assert off(plain_forward(c, w, toks)) > 3 * BF16_ROW
    cut = torch.cat([plain_forward(cfg, w, toks[:30]), plain_forward(cfg, w, toks[30:])])
    assert off(cut) > 3 * BF16_ROW
    w2 = dict(w)
    w2["loop.step"] = torch.zeros_like(w["loop.step"])
    assert off(plain_forward(cfg, w2, toks)) > 3 * BF16_ROW


def test_plain_recurrence_continues_from_its_state_and_equals_its_sum_form():
    """The token-by-token recurrence cut in two gives the whole; and it equals the closed sum
    over earlier tokens, o_t = sum_s w_ts (q_t . k_s) v_s / (max(|sum_s w_ts q_t . k_s|, e^-m_t) + 1e-6)
    with w_ts = exp(i_s + f_{s+1} + ... + f_t - m_t), written out here with dense matrices."""
    torch.manual_seed(1)
    t, heads, dk, dv = 23, 2, 5, 7
    q, k = torch.randn(t, heads, dk, dtype=torch.float64), torch.randn(t, heads, dk, dtype=torch.float64)
    v = torch.randn(t, heads, dv, dtype=torch.float64)
    i = torch.randn(t, heads, dtype=torch.float64) * 2
    f = torch.nn.functional.logsigmoid(torch.randn(t, heads, dtype=torch.float64) * 2 + 1)
    whole, state = plain_mlstm_scan(q, k, v, i, f)
    first, mid = plain_mlstm_scan(q[:9], k[:9], v[:9], i[:9], f[:9])
    second, end = plain_mlstm_scan(q[9:], k[9:], v[9:], i[9:], f[9:], mid)
    torch.testing.assert_close(torch.cat([first, second]), whole)
    for a, b in zip(state, end):
        torch.testing.assert_close(a, b)
    F = f.cumsum(0)
    for h in range(heads):
        logw = i[None, :, h] + F[:, None, h] - F[None, :, h]  # [t, s]
        logw = logw.masked_fill(~plain_window_mask(t, None), float("-inf"))
        m = torch.maximum(logw.max(dim=1).values, F[:, h])  # the maximum starts at 0: the term F_t + 0
        wts = torch.exp(logw - m[:, None]) * (q[:, h] @ k[:, h].T)
        den = torch.maximum(wts.sum(1).abs(), torch.exp(-m)) + 1e-6
        torch.testing.assert_close((wts @ v[:, h]) / den[:, None], whole[:, h])


def test_run_order_and_pass_vectors():
    from rapid_llm_amd.config.registry import config_from_dict

    for which, (cfg, _page, _seed) in FOKU.items():
        entry, parsed = config_from_dict(cfg)
        assert entry.name == "Fokulorn"
        plain = plain_run_order(cfg)
        assert list(parsed.run_order()) == [layer for layer, _ in plain]
        assert list(parsed.pass_places()) == [place for place, (_, p) in enumerate(plain) if p is not None]
        again = config_from_dict(parsed.to_dict())[1]
        assert again == parsed
        spec = entry.build_spec(parsed)
        assert spec.order() == parsed.run_order()
        assert (spec.stream_offsets is None) == ("loop" not in cfg)


def test_every_checkpoint_tensor_is_claimed_once_and_shapes_agree():
    from rapid_llm_amd.config.registry import config_from_dict
    from rapid_llm_amd.models.causal_lm import model_param_specs
    from rapid_llm_amd.weights.loader import WeightsError, load_params

    for which, (cfg, _page, seed) in FOKU.items():
        entry, parsed = config_from_dict(cfg)
        specs = model_param_specs(entry.build_spec(parsed))
        named = {src.name: (src.rows, *spec.shape[1:]) for spec in specs for src in spec.sources if src.name}
        assert named == tensor_shapes(cfg)
        weights = make_weights(cfg, seed)
        params = load_params(specs, weights.items(), engine_dtype=torch.bfloat16, device="cpu")
        for spec in specs:
            assert tuple(params[spec.name].shape) == spec.shape
            offset = 0
            for src in spec.sources:
                rows = params[spec.name][offset : offset + src.rows]
                if src.name:
                    assert torch.equal(rows.float(), weights[src.name].float())
                else:
                    assert not rows.any()  # padding of a packed matrix is zeros
                offset += src.rows
        gates = [s for s in specs if s.role == "matrix_f32"]
        assert gates and all(params[s.name].dtype == torch.float32 for s in gates)
        broken = dict(weights)
        del broken["final.norm"]
        broken["l0.mix.extra"] = torch.zeros(3)
        with pytest.raises(WeightsError) as err:
            load_params(specs, broken.items(), engine_dtype=torch.bfloat16, device="cpu")
        assert any("final.norm" in m for m in err.value.missing) and any("l0.mix.extra" in u for u in err.value.unexpected)


def test_configuration_refuses_what_the_design_does_not_have():
    from rapid_llm_amd.config.model_config import ConfigError
    from rapid_llm_amd.config.registry import config_from_dict

    base = FOKU["P"][0]
    for change in (
        lambda c: c["layers"][0].__setitem__("type", "convolution"),
        lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 48),
        lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3),
        lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"),
        lambda c: c["loop"].__setitem__("stop", 9),
        lambda c: c["layers"][1]["mixer"].__setitem__("gate_cap", 0.0),
        lambda c: c["norm"].pop("eps"),
    ):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)
