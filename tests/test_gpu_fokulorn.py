"""The Fokulorn decoder in the engine against the plain implementation of ``plain_fokulorn.py``:
every mechanism alone, every way of cutting requests into steps, pages and state slots that
are used again, the edges of windows and the first tokens, long decoding, and greedy
generation through the entry point."""

from types import SimpleNamespace

import pytest
import torch

import parity
import replay_util as ru
from fokulorn_configs import FOKU, load_plain, make_model_dir, make_weights, random_tokens
from plain_fokulorn import (
    plain_clamped_glu,
    plain_forward,
    plain_mlstm_gates,
    plain_mlstm_scan,
    plain_rms,
    plain_rotate_interleaved,
)

pytestmark = pytest.mark.gpu

DEV = "cuda"
# float32 rows against the plain implementation in float64, as a root mean square over the row
# relative to the logits' spread.  Where a head's output is tiny before it is brought to unit
# size (the first tokens of a request), rounding is amplified: the plain implementation in
# float32 is itself off by up to 3e-4 there, so element-wise bounds of a few ulp do not hold,
# while every fault these tests look for moves a row by a hundred times this bound
F32_ROW = 5e-4
# bfloat16 rows (root mean square error over a row, relative to the logits' spread) may be off
# by this many times what rounding alone does to the worst row of the same requests: the plain
# implementation with every stored activation rounded to bfloat16, against itself unrounded.
# The engine rounds in a few more places (scores' weights, a bias added after its product); its
# worst rows were 1.7 to 2 times that figure.  Faults move rows by ten times more
# (``test_fokulorn_cpu.py``).
BF16_TIMES_ROUNDING = 3.0


def _round_bf16(x):
    return x.bfloat16().to(x.dtype)


def _oracles(pcfg, pw, requests):
    """Per request the plain logits in float64, and the worst row that rounding alone moves."""
    want = {rid: plain_forward(pcfg, pw, toks, torch.float64) for rid, toks in requests.items()}
    rounded = {rid: plain_forward(pcfg, pw, toks, torch.float64, cast=_round_bf16) for rid, toks in requests.items()}
    order = sorted(want)
    row, _peak, _worst = parity.errors(torch.cat([rounded[r] for r in order]), torch.cat([want[r] for r in order]))
    return want, row


def _ctx(lens, slots):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return SimpleNamespace(
        num_seqs=len(lens), h_seq_lens=list(lens), h_seq_slots=list(slots),
        cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV),
        seq_slots=torch.tensor(slots, dtype=torch.int32, device=DEV),
    )


# --------------------------------------------------------------------------- #
# mechanisms alone
# --------------------------------------------------------------------------- #


def _mlstm_reference(q, k, v, g, pre_i, pre_f, cap, weight, eps, state=None):
    """Plain recurrence + unit RMS per head + weight + sigmoid gate for one request."""
    t, heads, dk = q.shape
    i = cap * torch.tanh(pre_i / cap)
    f = torch.nn.functional.logsigmoid(cap * torch.tanh(pre_f / cap))
    o, state = plain_mlstm_scan(q * dk ** -0.5, k, v, i, f, state)
    o = plain_rms(o, eps).reshape(t, -1) * weight * torch.sigmoid(g.reshape(t, -1))
    return o, state


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunked", [False, True, None])
@pytest.mark.parametrize("heads,dk,dv", [(3, 16, 40), (1, 8, 8), (2, 80, 72), (2, 256, 20), (5, 33, 7), (2, 128, 130)])
def test_recurrence_kernels_against_plain(dtype, heads, dk, dv, chunked):
    """Three requests of unequal length in one launch, in slots that are not in order, each cut
    into three steps, the last of one token; the state between the steps is the kernels' own.  Token
    by token, in chunks of 64 (a request of 200 tokens crosses three chunk edges, one ends at
    an edge), and as the step's shape decides."""
    from rapid_llm_amd.kernels import ops

    torch.manual_seed(heads * 1000 + dk + dv)
    lens, slots, cuts = [37, 1, 200, 128], [4, 0, 2, 5], [2, 1, 33, 64]
    cap, eps = 9.0, 1e-5
    qk, vv = heads * dk, heads * dv
    width = 2 * qk + 2 * vv
    width += -width % 8
    cols = (0, qk, 2 * qk, 2 * qk + vv)
    reqs = []
    for n in lens:
        packed = torch.randn(n, width).to(dtype)
        pre = torch.randn(n, 2 * heads) * 3.0
        pre[:, heads:] += 2.0
        reqs.append((packed, pre))
    bias = torch.randn(2 * heads)
    weight = 1.0 + 0.2 * torch.randn(vv)
    S = torch.full((6, heads, dk, dv), float("nan"), device=DEV)
    n_state = torch.full((6, heads, dk), float("nan"), device=DEV)
    m_state = torch.full((6, heads), float("nan"), device=DEV)
    for s in slots:  # a slot that is taken starts at zero; the others hold what must never be read
        S[s], n_state[s], m_state[s] = 0, 0, 0
    got = [[] for _ in lens]
    for part in range(3):  # the last step brings the last token of every longer request alone
        spans = [((0, c), (c, max(c, n - 1)), (max(c, n - 1), n))[part] for c, n in zip(cuts, lens)]
        live = [i for i, (a, b) in enumerate(spans) if b > a]
        packed = torch.cat([reqs[i][0][spans[i][0]:spans[i][1]] for i in live]).to(DEV)
        pre = torch.cat([reqs[i][1][spans[i][0]:spans[i][1]] for i in live]).to(DEV)
        out = torch.empty((packed.shape[0], vv), dtype=dtype, device=DEV)
        ctx = _ctx([spans[i][1] - spans[i][0] for i in live], [slots[i] for i in live])
        ops.mlstm(packed, cols, pre, bias.to(DEV), weight.to(DEV), out, ctx, S, n_state, m_state,
                  heads, dk, dv, cap, eps, chunked=chunked)
        at = 0
        for i in live:
            n = spans[i][1] - spans[i][0]
            got[i].append(out[at:at + n].float().cpu())
            at += n
    for i, (packed, pre) in enumerate(reqs):
        x = packed.float()
        n = lens[i]
        want, (S_w, n_w, m_w) = _mlstm_reference(
            x[:, cols[0]:cols[0] + qk].view(n, heads, dk), x[:, cols[1]:cols[1] + qk].view(n, heads, dk),
            x[:, cols[2]:cols[2] + vv].view(n, heads, dv), x[:, cols[3]:cols[3] + vv].view(n, heads, dv),
            pre[:, :heads] + bias[:heads], pre[:, heads:] + bias[heads:], cap, weight, eps,
        )
        have = torch.cat(got[i])
        if dtype == torch.float32:
            torch.testing.assert_close(have, want, rtol=2e-4, atol=2e-5)
            torch.testing.assert_close(S[slots[i]].cpu(), S_w, rtol=1e-4, atol=1e-5)
            torch.testing.assert_close(n_state[slots[i]].cpu(), n_w, rtol=1e-4, atol=1e-5)
            torch.testing.assert_close(m_state[slots[i]].cpu(), m_w, rtol=1e-5, atol=1e-6)
        else:
            torch.testing.assert_close(have, want, rtol=2e-2, atol=2e-2)
    untouched = [s for s in range(6) if s not in slots]
    assert torch.isnan(S[untouched]).all() and torch.isnan(m_state[untouched]).all()


def test_recurrence_remembers_one_early_token():
    """One token with an open input gate among 400 whose gates are nearly shut, forget gates
    that keep: every later output is that token's value, also across a step's edge and for
    tokens that come one by one.  A state that is lost or cleared in between shows at once."""
    from rapid_llm_amd.kernels import ops

    torch.manual_seed(5)
    heads, dk, dv, n, special = 2, 16, 24, 400, 3
    qk, vv = heads * dk, heads * dv
    width = 2 * qk + 2 * vv
    cols = (0, qk, 2 * qk, 2 * qk + vv)
    packed = torch.randn(n, width)
    packed[:, cols[3]:] = 4.0  # output gates open
    pre = torch.empty(n, 2 * heads)
    pre[:, :heads] = -12.0
    pre[special, :heads] = 8.0
    pre[:, heads:] = 14.0
    S = torch.zeros((2, heads, dk, dv), device=DEV)
    ns = torch.zeros((2, heads, dk), device=DEV)
    ms = torch.zeros((2, heads), device=DEV)
    weight = torch.ones(vv)
    outs = []
    steps = [(0, 2), (2, 150), (150, 151), (151, 152), (152, 390)] + [(i, i + 1) for i in range(390, n)]
    for a, b in steps:
        out = torch.empty((b - a, vv), device=DEV)
        ops.mlstm(packed[a:b].contiguous().to(DEV), cols, pre[a:b].contiguous().to(DEV), None, weight.to(DEV), out,
                  _ctx([b - a], [1]), S, ns, ms, heads, dk, dv, 15.0, 1e-6)
        outs.append(out.cpu())
    got = torch.cat(outs).view(n, heads, dv)
    v_special = packed[special, cols[2]:cols[2] + vv].view(heads, dv)
    unit = v_special / v_special.square().mean(-1, keepdim=True).sqrt()
    gate = torch.sigmoid(torch.tensor(4.0))
    k_special = packed[special, cols[1]:cols[1] + qk].view(heads, dk)
    for t in (special, special + 1, 149, 150, 151, 152, 389, 390, n - 1):
        sign = torch.sign((packed[t, :qk].view(heads, dk) * k_special).sum(-1, keepdim=True))
        torch.testing.assert_close(got[t], unit * gate * sign, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clamped_gated_activation(dtype):
    from rapid_llm_amd.kernels import ops

    for inter, limit in ((72, 1.5), (99, 0.75), (136, 3.0)):
        gu = (torch.randn(21, 2 * inter) * 3.0).to(dtype)
        out = torch.empty((21, inter), dtype=dtype, device=DEV)
        ops.swiglu(gu.to(DEV), out, limit)
        g, u = gu.float()[:, :inter].clamp(max=limit), gu.float()[:, inter:].clamp(-limit, limit)
        want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
        tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(out.float().cpu(), want, **tol)
    # the plain silu * up is the same kernel without a limit
    out = torch.empty((21, inter), dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    want = torch.nn.functional.silu(gu.float()[:, :inter]) * gu.float()[:, inter:]
    torch.testing.assert_close(out.float().cpu(), want, **tol)


@pytest.mark.parametrize("rows", [1, 8, 16, 17, 40, 64, 200])
@pytest.mark.parametrize("inter,k", [(256, 128), (1024, 256), (3072, 1024)])
def test_clamped_activation_inside_the_gate_up_product(rows, inter, k):
    """Every product kernel that applies the gated activation in its epilogue (few rows, 17 to
    64 rows, the tile product) against the product followed by the activation on the CPU."""
    from rapid_llm_amd.kernels import ops

    torch.manual_seed(rows + inter)
    x = torch.randn(rows, k).bfloat16()
    w = (torch.randn(2 * inter, k) * (3.0 / k ** 0.5)).bfloat16()
    for limit in (1.5, 0.0):
        got = ops.gemm_bf16_swiglu(x.to(DEV), w.to(DEV), limit=limit)
        if got is None:
            assert rows > 16  # beyond the few-row kernel not every shape has a fused product
            return
        gu = (x.float() @ w.float().T).bfloat16().float()
        g, u = gu[:, :inter], gu[:, inter:]
        if limit:
            g, u = g.clamp(max=limit), u.clamp(-limit, limit)
            want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
        else:
            want = torch.nn.functional.silu(g) * u
        torch.testing.assert_close(got.float().cpu(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,k,n", [(1, 96, 6), (37, 70, 2), (300, 1024, 16), (5, 256, 40)])
def test_gate_projection_in_float32(dtype, tokens, k, n):
    from rapid_llm_amd.kernels import ops

    x = torch.randn(tokens, k).to(dtype)
    w = torch.randn(n, k)
    got = ops.gate_product(x.to(DEV), w.to(DEV))
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), (x.double() @ w.double().T).float(), rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_gate_and_scaled_embedding(dtype):
    from rapid_llm_amd.kernels import ops

    heads, d, tokens = 5, 24, 9
    y = torch.randn(tokens, heads * d).to(dtype)
    packed = torch.randn(tokens, 200 + 8).to(dtype)
    got = y.clone().to(DEV)
    ops.head_gate(got, packed.to(DEV), 200, heads, d)
    want = y.float().view(tokens, heads, d) * torch.sigmoid(packed.float()[:, 200:205])[:, :, None]
    tol = dict(rtol=1e-6, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.float().cpu().view(tokens, heads, d), want, **tol)
    table = torch.randn(50, 70).to(dtype)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    out = torch.empty((4, 70), dtype=torch.float32, device=DEV)
    ops.embed(ids.to(DEV), table.to(DEV), out, None, 7.5)
    torch.testing.assert_close(out.cpu(), table.float()[ids.long()] * 7.5, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,rot", [(4, 2, 32, 32), (6, 6, 16, 8), (2, 1, 24, 12), (3, 1, 20, 10), (8, 2, 64, 0)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_values_are_the_unrotated_keys_in_the_cache(dtype, nq, nkv, d, rot, with_bias):
    """The cache write of a packed ``[q | k | gates]`` row: rotated keys (interleaved pairs, the
    first ``rot`` channels) in the key pages, the same keys unrotated in the value pages; the
    projection's bias, when the kernel is given it, is added before either."""
    from rapid_llm_amd.kernels import ops

    page, tokens = 8, 21
    width = (nq + nkv) * d + 8
    width += -width % 8
    packed = torch.randn(tokens, width).to(dtype)
    positions = torch.arange(5, 5 + tokens, dtype=torch.int32)
    table = torch.tensor([[0, 3, 1, 4, 2, 0]], dtype=torch.int32)
    k_cache = torch.zeros((5, nkv, page, d), dtype=dtype, device=DEV)
    v_cache = torch.zeros((5, nkv, d, page), dtype=dtype, device=DEV)
    q_out = torch.empty((tokens, nq * d), dtype=dtype, device=DEV)
    cos = sin = None
    if rot:
        inv = 1.0 / (500.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
        cos, sin = ops.rope_table(inv.to(DEV), 64)
    bias = torch.randn(width) if with_bias else None
    ops.qknorm_rope_kvwrite(
        packed.to(DEV), q_out, k_cache, v_cache, None, None, cos, sin, positions.to(DEV),
        torch.zeros(tokens, dtype=torch.int32, device=DEV), table.to(DEV), page, nq, nkv, d, 0.0,
        int(positions.max()), "interleaved", value_head0=nq, bias=bias.to(DEV) if with_bias else None,
    )
    x = packed.float() + (bias if with_bias else 0.0)
    q = x[:, : nq * d].view(tokens, nq, d)
    k = x[:, nq * d:(nq + nkv) * d].view(tokens, nkv, d)
    q_want, k_want = (plain_rotate_interleaved(a, positions, rot, 500.0) if rot else a for a in (q, k))
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(q_out.float().cpu().view(tokens, nq, d), q_want, **tol)
    for t in range(tokens):
        pos = int(positions[t])
        pg, slot = int(table[0, pos // page]), pos % page
        torch.testing.assert_close(k_cache[pg, :, slot].float().cpu(), k_want[t], **tol)
        torch.testing.assert_close(v_cache[pg, :, :, slot].float().cpu(), k[t].to(dtype).float(), rtol=0, atol=0)
    # fewer than eight tokens take the kernel that writes the values head by head
    few = 3
    v_few = torch.zeros_like(v_cache)
    ops.qknorm_rope_kvwrite(
        packed[:few].contiguous().to(DEV), q_out[:few].contiguous(), torch.zeros_like(k_cache), v_few, None, None, cos,
        sin, positions[:few].contiguous().to(DEV), torch.zeros(few, dtype=torch.int32, device=DEV), table.to(DEV), page,
        nq, nkv, d, 0.0, int(positions[:few].max()), "interleaved", value_head0=nq,
        bias=bias.to(DEV) if with_bias else None,
    )
    for t in range(few):
        pos = int(positions[t])
        torch.testing.assert_close(v_few[int(table[0, pos // page]), :, :, pos % page].float().cpu(),
                                   k[t].to(dtype).float(), rtol=0, atol=0)


# --------------------------------------------------------------------------- #
# whole models: every way of cutting the requests
# --------------------------------------------------------------------------- #

LENGTHS = {
    "P": [1, 2, 3, 18, 19, 20, 21, 57, 150],   # the first tokens; around the window of 19; many pages
    "Q": [1, 4, 5, 6, 9, 33, 80],              # around the window of 5 and the page of 4
    "R": [2, 15, 64, 129, 131, 260],           # around the window of 130
    "S": [1, 2, 17, 33, 34, 35, 90],           # a window of one key; around the window of 33
    "T": [1, 2, 15, 16, 63, 64, 65, 200],      # around the chunk of 64 and the length from which steps run in chunks
}


def _requests(which):
    cfg, _page, seed = FOKU[which]
    return {f"q{i}": random_tokens(n, cfg["vocab"], seed * 100 + i) for i, n in enumerate(LENGTHS[which])}


def _runner(model_dir, dtype, page, num_pages, max_seq_len, slots=4):
    from rapid_llm_amd import EngineConfig, ModelRunner

    runner = ModelRunner(
        model_dir,
        EngineConfig(dtype=dtype, max_seq_len=max_seq_len, page_size=page, num_pages=num_pages,
                     max_num_seqs=slots, use_graph=False),
    )
    for layer in runner.device_cache.layers:  # whatever is read before it is written shows
        for t in layer.pages.values() if layer.owns_pages else ():
            t.fill_(float("nan"))
    return runner


def _poison_states(runner):
    """What a slot held before it is taken must not matter: it is cleared when it is taken."""
    for layer in runner.device_cache.layers:
        for t in layer.states.values():
            t.fill_(float("nan"))


def _check(got, want, dtype, label, rounding=None):
    order = sorted(want)
    if dtype == "bfloat16":
        a, b = torch.cat([got[r] for r in order]), torch.cat([want[r] for r in order])
        assert a.shape == b.shape and torch.isfinite(a).all(), label
        row, peak, worst = parity.errors(a, b)
        parity.record(label, row, peak)
        assert row <= BF16_TIMES_ROUNDING * rounding, (
            f"{label}: worst row {worst} is off by {row:.4f} of the logits' spread, rounding alone by {rounding:.4f}"
        )
        return
    spread = float(torch.cat([want[r] for r in order]).double().std())
    for rid in order:
        assert got[rid].shape == want[rid].shape and torch.isfinite(got[rid]).all(), (label, rid)
        rows = (got[rid].double() - want[rid].double()).square().mean(dim=1).sqrt() / spread
        bad = rows > F32_ROW
        assert not bad.any(), (
            f"{label}: request {rid}, first wrong position {int(torch.nonzero(bad)[0])}, "
            f"worst row {float(rows.max()):.3e} of the spread"
        )


@pytest.mark.parametrize("which", ["P", "Q", "R", "S", "T"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_plain(tmp_path, which, dtype):
    cfg, page, seed = FOKU[which]
    model_dir = make_model_dir(tmp_path, which, sharp=4.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    longest = max(LENGTHS[which])
    schedules = {
        "whole": ru.whole(requests),
        "decode": ru.prefill_then_decode(requests, 40),
        "portions": ru.changing_portions(requests),
        "portions_of_two": ru.changing_portions(requests, sizes=(2, 2, 3, 2, 64, 2)),
        "mixed": ru.mixed(requests, seed, max_tokens=None),
        "mixed_tight": ru.mixed(requests, seed + 1, max_tokens=2 * 64 * ((longest + 63) // 64)),
    }
    for label, steps in schedules.items():
        pages = ru.pages_for(steps, requests, page) + 1
        runner = _runner(model_dir, dtype, page, pages + 1, longest + 8)
        _poison_states(runner)
        got = ru.run_in_process(runner, steps)
        _check(got, want, dtype, f"{which}/{dtype}/{label}", rounding)
        runner.cache.check_invariants()
        assert not runner.cache.live_requests()
        del runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_slots_used_again(tmp_path, dtype):
    """Five requests through two state slots, each a short prompt and then 300 tokens one by
    one, two at a time in a step: slots and pages are taken again by later requests."""
    which = "P"
    cfg, page, seed = FOKU[which]
    model_dir = make_model_dir(tmp_path, which, sharp=4.0)
    pcfg, pw = load_plain(model_dir)
    requests = {f"d{i}": random_tokens(300 + 7 * i, cfg["vocab"], 40 + i) for i in range(5)}
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, 3, max_live=2, tail=295)
    runner = _runner(model_dir, dtype, page, ru.pages_for(steps, requests, page) + 2, 340, slots=2)
    _poison_states(runner)
    got = ru.run_in_process(runner, steps)
    _check(got, want, dtype, f"long decoding/{dtype}", rounding)
    runner.cache.check_invariants()


def test_trace_program_on_a_recurrent_model(tmp_path):
    """``bin/trace_run`` as a child process on a mixed trace over a tight pool."""
    which = "Q"
    cfg, page, seed = FOKU[which]
    model_dir = make_model_dir(tmp_path, which, sharp=4.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, seed + 5, max_tokens=256)
    got = ru.run_trace_program(model_dir, "float32", steps, tmp_path / "out", 256, cfg["vocab"])
    _check(got, want, "float32", "trace_run")
    assert rounding > 0


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_through_the_entry_point(tmp_path, use_graph):
    """``LLM.generate``: scheduler, chunked prompts beside decoding requests, sampling kernels;
    decode steps eagerly and replayed from graphs.  The plain implementation re-runs the whole
    sequence for every token."""
    from rapid_llm_amd import LLM, SamplingParams

    which = "P"
    cfg, page, seed = FOKU[which]
    model_dir = make_model_dir(tmp_path, which)
    pcfg, pw = load_plain(model_dir)
    prompts = [random_tokens(n, cfg["vocab"], seed + n) for n in (1, 7, 30, 45)]
    llm = LLM(str(model_dir), dtype="float32", page_size=page, num_pages=60, max_num_seqs=3, max_seq_len=96,
              max_chunk_size=16, max_num_batched_tokens=32, use_cuda_graph=use_graph)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=24))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out.token_ids:
            logits = plain_forward(pcfg, pw, ids)[-1]
            assert float(logits.max() - logits[tok]) <= 1e-3, (len(prompt), len(ids))
            ids.append(tok)
        assert len(out.token_ids) == 24
    llm.scheduler.cache.check_invariants()
    assert not llm.scheduler.cache.live_requests()
