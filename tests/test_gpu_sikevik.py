"""The Sikevik decoder in the engine against the plain implementation of ``plain_sikevik.py``:
every mechanism alone, every way of cutting requests into steps, pages and slots that are used
again, the edges of windows and of the kept first positions, long decoding, and greedy
generation through the entry point."""

import math
import random
from types import SimpleNamespace

import pytest
import torch

import parity
import replay_util as ru
from plain_sikevik import (
    bf16_round,
    plain_forward,
    plain_gelu_tanh,
    plain_kept_window_mask,
    plain_relu_squared,
    plain_rmsnorm,
    plain_route,
    plain_sink_softmax,
    plain_sinusoid,
)
from sikevik_configs import SIKE, load_plain, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

DEV = "cuda"
# float32 rows against the plain implementation in float64: root mean square over a row,
# relative to the logits' spread
F32_ROW = 2e-4
# bfloat16 rows may be off by this many times what rounding alone does to the worst row of the
# same requests (the plain implementation with every stored activation rounded to bfloat16,
# against itself unrounded); faults move rows by ten times more (``test_sikevik_cpu.py``)
BF16_TIMES_ROUNDING = 3.0


def _ops():
    from rapid_llm_amd.kernels import ops

    return ops


# --------------------------------------------------------------------------- #
# the attention kernels alone, on a paged cache laid out by hand
# --------------------------------------------------------------------------- #


def _plain_rows(q, k, v, scale, window, keep, sink, first_row):
    """Attention of the last ``q.shape[0]`` positions of one request over all its keys."""
    t, n = k.shape[0], q.shape[0]
    group = q.shape[1] // k.shape[1]
    seen = plain_kept_window_mask(t, window or None, keep)[first_row:]
    out = torch.empty((n, q.shape[1], v.shape[-1]), dtype=torch.float64)
    for h in range(q.shape[1]):
        s = (q[:, h].double() @ k[:, h // group].double().T) * scale
        if sink:
            p = plain_sink_softmax(s, seen)
        else:
            p = torch.softmax(s.masked_fill(~seen, float("-inf")), dim=-1)
        out[:, h] = p @ v[:, h // group].double()
    return out.reshape(n, -1).float()


def _paged(seqs, nq, nkv, d, dv, page, dtype, seed, window, keep, sink, scale, spike=None):
    """``seqs`` = (tokens already cached, tokens in this step) per request.  Pages in shuffled
    order, everything unwritten NaN, and the pages between the kept positions and the window of
    the step's first token mapped to the null page, as after trimming."""
    rng = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + n) // page) for a, n in seqs) + 1
    order = list(range(1, total_pages))
    rng.shuffle(order)
    max_pages = max(-(-(a + n) // page) for a, n in seqs) + 2
    table = torch.zeros((len(seqs) + 3, max_pages), dtype=torch.int32)
    k_cache = torch.full((total_pages, nkv, page, d), float("nan"))
    v_cache = torch.full((total_pages, nkv, dv, page), float("nan"))
    slots = list(range(len(seqs) + 3))
    rng.shuffle(slots)
    q_rows, positions, token_slot, expect = [], [], [], []
    for i, (a, n) in enumerate(seqs):
        t = a + n
        k = torch.randn((t, nkv, d), generator=gen)
        v = torch.randn((t, nkv, dv), generator=gen)
        q = torch.randn((n, nq, d), generator=gen)
        if spike is not None and i == spike[0]:
            # one key carries nearly all of the softmax mass of the request's last query
            far, group = spike[1], nq // nkv
            for j in range(nkv):
                u = q[-1, j * group].clone()
                q[-1, j * group : (j + 1) * group] = u
                k[far, j] = u * (30.0 / scale / float(u @ u))
            v[far] = 7.0
        if dtype == torch.bfloat16:
            q, k, v = (x.bfloat16().float() for x in (q, k, v))
        slot = slots[i]
        first_needed = max(0, a - window + 1) // page if window else 0
        kept_pages = -(-keep // page) if window else 0
        for p in range(-(-t // page)):
            pid = order.pop()
            if kept_pages <= p < first_needed:
                continue  # given back: the table keeps the null page, whose content is NaN
            table[slot, p] = pid
            lo, hi = p * page, min(t, (p + 1) * page)
            k_cache[pid, :, : hi - lo, :] = k[lo:hi].transpose(0, 1)
            v_cache[pid, :, :, : hi - lo] = v[lo:hi].permute(1, 2, 0)
        expect.append(_plain_rows(q, k, v, scale, window, keep, sink, a))
        q_rows.append(q.reshape(n, nq * d))
        positions += list(range(a, t))
        token_slot += [slot] * n
    ctx = SimpleNamespace(
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        token_slot=torch.tensor(token_slot, dtype=torch.int32, device=DEV),
        token_ids=torch.zeros(len(positions), dtype=torch.int32, device=DEV),
        h_seq_starts=[a for a, _ in seqs], h_seq_lens=[n for _, n in seqs],
        max_position=max(positions), extra={},
    )
    return (torch.cat(q_rows).to(DEV, dtype), k_cache.to(DEV, dtype), v_cache.to(DEV, dtype), table.to(DEV), ctx,
            torch.cat(expect))


ATTENTION_CASES = [
    # nq, nkv, d, dv, page, window, keep, sink, seqs (cached, new)
    (4, 2, 32, 16, 8, 19, 5, True, [(0, 60), (45, 1), (200, 1), (30, 31), (0, 1)]),
    (6, 2, 16, 48, 4, 41, 21, True, [(0, 130), (100, 1), (41, 2), (20, 1), (21, 1), (22, 1)]),
    (8, 2, 64, 32, 16, 0, 0, True, [(300, 1), (5, 70), (0, 2)]),        # no window: the sink alone
    (3, 3, 16, 16, 8, 33, 8, True, [(0, 33), (33, 1), (34, 1), (40, 1), (41, 9)]),  # equal sizes
    (4, 4, 64, 128, 16, 130, 0, False, [(0, 140), (129, 1), (130, 1), (131, 1)]),  # wider values, no sink
    (2, 1, 128, 64, 8, 64, 64, True, [(0, 200), (64, 1), (127, 1), (128, 1), (500, 1)]),  # keep = window
    (5, 5, 18, 10, 8, 7, 3, True, [(0, 40), (9, 1), (10, 1), (30, 2)]),   # sizes off the grid of 16
    (3, 1, 12, 22, 4, 33, 9, True, [(0, 50), (41, 1), (42, 1), (100, 1)]),
    (6, 3, 24, 24, 4, 1, 2, True, [(0, 9), (5, 1)]),                      # a window of the own key alone
    (4, 1, 64, 32, 16, 1000, 30, True, [(3000, 1), (990, 40), (0, 1100)]),  # long contexts
    (2, 1, 32, 16, 4, 0, 0, True, [(8300, 1), (8250, 60)]),  # more pages than a workgroup stages: the table is read
]


@pytest.mark.parametrize("case", ATTENTION_CASES, ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}v{c[3]}p{c[4]}w{c[5]}k{c[6]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attention_with_kept_positions_sink_and_value_size(case, dtype):
    ops = _ops()
    nq, nkv, d, dv, page, window, keep, sink, seqs = case
    scale = 0.8 / math.sqrt(d)
    q, kc, vc, table, ctx, want = _paged(seqs, nq, nkv, d, dv, page, dtype, d + dv + page, window, keep, sink, scale)
    out = torch.full((q.shape[0], nq * dv), float("nan"), dtype=dtype, device=DEV)
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, scale,
                        value_dim=dv, keep_first=keep, sink=sink)
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=3e-6)
    else:
        assert float((got - want).abs().max()) <= 0.03 * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,dv,page", [(64, 32, 16), (16, 48, 4), (18, 10, 8)])
def test_one_key_holds_the_mass_at_every_edge(dtype, d, dv, page):
    """One key among hundreds carries the last query's weight.  Where the key is kept (among
    the first ones) or inside the window the output is that key's value; one position further
    out the key is not seen and the output is far from it.  For a single decoded token and for
    the last token of a portion."""
    ops = _ops()
    nq, nkv, window, keep, scale = 4, 2, 50, 11, 0.125
    length = 400
    for far, visible in ((0, True), (10, True), (11, False), (200, False), (length - 51, False), (length - 50, True),
                         (length - 1, True)):
        for seqs, who in (([(length - 1, 1), (10, 1)], 0), ([(5, 1), (length - 120, 120)], 1)):
            q, kc, vc, table, ctx, want = _paged(seqs, nq, nkv, d, dv, page, dtype, far, window, keep, True, scale,
                                                 spike=(who, far))
            out = torch.empty((q.shape[0], nq * dv), dtype=dtype, device=DEV)
            ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, scale,
                                value_dim=dv, keep_first=keep, sink=True)
            got = out.float().cpu()
            row = 0 if who == 0 else got.shape[0] - 1
            assert bool((want[row] > 6.5).all()) == visible  # the construction works in the plain attention
            torch.testing.assert_close(got[row], want[row], rtol=2e-2, atol=3e-2)
            torch.testing.assert_close(got, want, rtol=2e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_the_sink_shows_when_scores_are_small(dtype):
    """Keys with score 0: n seen keys share n / (n + 1) of the weight, the sink takes the rest.
    A kernel that leaves it out returns the plain mean."""
    ops = _ops()
    nq, nkv, d, dv, page = 2, 1, 32, 16, 8
    seqs = [(0, 1), (0, 3), (6, 1)]
    q, kc, vc, table, ctx, want = _paged(seqs, nq, nkv, d, dv, page, dtype, 7, 0, 0, True, 0.0)
    out = torch.empty((q.shape[0], nq * dv), dtype=dtype, device=DEV)
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 0.0, value_dim=dv, sink=True)
    got = out.float().cpu()
    torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2)
    # the first token of a request sees itself alone: half its value
    v0 = vc[int(table[ctx.token_slot[0], 0]), 0, :, 0].float().cpu()
    torch.testing.assert_close(got[0, :dv], 0.5 * v0, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nq,nkv,d,dv", [(4, 2, 32, 16), (6, 2, 16, 48), (5, 5, 18, 10), (3, 1, 12, 22), (2, 2, 64, 64)])
@pytest.mark.parametrize("tokens", [3, 21])
def test_cache_write_of_value_heads_of_their_own_size(dtype, nq, nkv, d, dv, tokens):
    """Packed ``[q | k | v]`` rows with value heads of ``dv`` channels: normed queries, normed keys
    in the key pages, the values as projected in the transposed value pages, in both the kernel
    that writes head by head (few tokens) and the one that writes tiles of 16 tokens."""
    ops = _ops()
    page = 8
    width = (nq + nkv) * d + nkv * dv
    width += -width % 8
    packed = torch.randn(tokens, width).to(dtype)
    positions = torch.arange(5, 5 + tokens, dtype=torch.int32)
    table = torch.tensor([[0, 3, 1, 4, 2, 0]], dtype=torch.int32)
    k_cache = torch.zeros((5, nkv, page, d), dtype=dtype, device=DEV)
    v_cache = torch.zeros((5, nkv, dv, page), dtype=dtype, device=DEV)
    q_out = torch.empty((tokens, nq * d), dtype=dtype, device=DEV)
    qw, kw = 1.0 + 0.2 * torch.randn(d), 1.0 + 0.2 * torch.randn(d)
    eps = 1e-5
    ops.qknorm_rope_kvwrite(
        packed.to(DEV), q_out, k_cache, v_cache, qw.to(DEV), kw.to(DEV), None, None, positions.to(DEV),
        torch.zeros(tokens, dtype=torch.int32, device=DEV), table.to(DEV), page, nq, nkv, d, eps,
        int(positions.max()), value_dim=dv,
    )
    x = packed.float()
    q = plain_rmsnorm(x[:, : nq * d].view(tokens, nq, d), qw, eps)
    k = plain_rmsnorm(x[:, nq * d:(nq + nkv) * d].view(tokens, nkv, d), kw, eps)
    v = x[:, (nq + nkv) * d:(nq + nkv) * d + nkv * dv].view(tokens, nkv, dv)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(q_out.float().cpu().view(tokens, nq, d), q, **tol)
    for t in range(tokens):
        pos = int(positions[t])
        pg, slot = int(table[0, pos // page]), pos % page
        torch.testing.assert_close(k_cache[pg, :, slot].float().cpu(), k[t], **tol)
        torch.testing.assert_close(v_cache[pg, :, :, slot].float().cpu(), v[t], rtol=0, atol=0)


# --------------------------------------------------------------------------- #
# the row-wise mechanisms alone
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hidden", [96, 100, 256, 4100, 97, 18, 2050, 20000])
def test_norm_behind_a_sublayer_add_and_next_norm_in_one_kernel(dtype, hidden):
    ops = _ops()
    tokens = 9
    residual = torch.randn(tokens, hidden)
    y = (torch.randn(tokens, hidden) * 3.0).to(dtype)
    wy, w = 1.0 + 0.2 * torch.randn(hidden), 1.0 + 0.2 * torch.randn(hidden)
    eps_y, eps = 3e-6, 1e-5
    new = residual.double() + plain_rmsnorm(y.double(), wy.double(), eps_y)
    want = plain_rmsnorm(new, w.double(), eps).float()
    res = residual.clone().to(DEV)
    out = torch.empty((tokens, hidden), dtype=dtype, device=DEV)
    ops.normed_add_rmsnorm(res, y.to(DEV), wy.to(DEV), eps_y, w.to(DEV), out, eps)
    torch.testing.assert_close(res.cpu(), new.float(), rtol=1e-6, atol=1e-6)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    # chosen rows only (the last norm of a step), and the add alone
    rows = torch.tensor([7, 2], dtype=torch.int32, device=DEV)
    res = residual.clone().to(DEV)
    out = torch.empty((2, hidden), dtype=dtype, device=DEV)
    ops.normed_add_rmsnorm(res, y.to(DEV), wy.to(DEV), eps_y, w.to(DEV), out, eps, rows)
    torch.testing.assert_close(out.float().cpu(), want[[7, 2]], **tol)
    torch.testing.assert_close(res.cpu()[[0, 1, 3]], residual[[0, 1, 3]], rtol=0, atol=0)
    res = residual.clone().to(DEV)
    ops.normed_add_rmsnorm(res, y.to(DEV), wy.to(DEV), eps_y, None, None, 0.0)
    torch.testing.assert_close(res.cpu(), new.float(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_one_operand_activations_and_expert_weights(dtype):
    ops = _ops()
    tokens, experts, ff, shared = 13, 5, 27, 9
    cols = experts * ff + shared
    x = (torch.randn(tokens, cols) * 2.0).to(dtype)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    for kind, fn in (("gelu_tanh", plain_gelu_tanh), ("relu_squared", plain_relu_squared)):
        out = torch.empty((tokens, cols), dtype=dtype, device=DEV)
        ops.unary_act(x.to(DEV), out, kind)
        torch.testing.assert_close(out.float().cpu(), fn(x.float()), **tol)
    route = torch.rand(tokens, experts) * (torch.rand(tokens, experts) > 0.5)
    out = torch.empty((tokens, cols), dtype=dtype, device=DEV)
    ops.unary_act(x.to(DEV), out, "relu_squared", route.to(DEV), ff)
    want = plain_relu_squared(x.float())
    want[:, : experts * ff] *= route.repeat_interleave(ff, dim=1)
    torch.testing.assert_close(out.float().cpu(), want, **tol)


@pytest.mark.parametrize("experts,top,scale", [(8, 3, 1.75), (3, 1, 2.5), (4, 4, 1.0), (70, 5, 0.5), (1, 1, 3.0)])
def test_router_weights(experts, top, scale):
    ops = _ops()
    tokens = 37
    h = torch.randn(tokens, 48)
    router = torch.randn(experts, 48) * 0.8
    z = (h @ router.T).contiguous()
    chosen, weight = plain_route(h, router, top, scale)
    want = torch.zeros(tokens, experts).scatter_(1, chosen, weight)
    got = z.clone().to(DEV)
    ops.route(got, top, scale)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    assert ((got.cpu() > 0).sum(dim=1) == top).all()
    # product and weights in one kernel, from rows of either type; a token alone gives the same bits
    for dtype in (torch.float32, torch.bfloat16):
        hx = h.to(dtype)
        chosen, weight = plain_route(hx.float(), router, top, scale)
        want = torch.zeros(tokens, experts).scatter_(1, chosen, weight)
        fused = ops.router(hx.to(DEV), router.to(DEV), top, scale)
        torch.testing.assert_close(fused.cpu(), want, rtol=1e-4, atol=1e-5)
        alone = ops.router(hx[5:6].contiguous().to(DEV), router.to(DEV), top, scale)
        assert torch.equal(alone[0], fused[5])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hidden", [96, 100, 64, 99])
def test_scaled_embedding_with_sinusoidal_positions(dtype, hidden):
    ops = _ops()
    table = torch.randn(50, hidden).to(dtype)
    ids = torch.tensor([3, 49, 0, 3, 7], dtype=torch.int32)
    positions = torch.tensor([0, 1, 977, 5000, 31], dtype=torch.int32)
    i = torch.arange((hidden + 1) // 2, dtype=torch.float64)
    inv = (10000.0 ** (-2.0 * i / hidden)).to(torch.float32)
    out = torch.empty((5, hidden), dtype=torch.float32, device=DEV)
    ops.embed(ids.to(DEV), table.to(DEV), out, None, 7.5, positions.to(DEV), inv.to(DEV))
    want = table.float()[ids.long()] * 7.5 + plain_sinusoid(positions, hidden)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-6, atol=1e-6)
    # position 0: sines 0, cosines 1
    torch.testing.assert_close(out.cpu()[0] - table.float()[3] * 7.5,
                               torch.tensor([0.0, 1.0]).repeat((hidden + 1) // 2)[:hidden], rtol=0, atol=1e-6)


def test_two_streams_side_by_side():
    ops = _ops()
    for hidden in (100, 99):  # four channels a thread, and one
        a, b = torch.randn(7, hidden), torch.randn(7, hidden)
        for dtype in (torch.float32, torch.bfloat16):
            out = torch.empty((7, 2 * hidden), dtype=dtype, device=DEV)
            ops.pair_rows(a.to(DEV), b.to(DEV), out)
            torch.testing.assert_close(out.cpu(), torch.cat([a, b], dim=1).to(dtype), rtol=0, atol=0)


# --------------------------------------------------------------------------- #
# whole models: every way of cutting the requests
# --------------------------------------------------------------------------- #

LENGTHS = {
    "A": [1, 2, 3, 5, 6, 19, 20, 21, 22, 41, 42, 57, 150],  # the first tokens; around the kept 5 and 21; the windows of 19 and 41
    "B": [1, 2, 4, 5, 6, 7, 9, 33, 80],                     # around the window of 5, the kept one and the page of 4
    "C": [2, 15, 64, 65, 129, 130, 131, 260],               # around the windows of 64 and 130
    "D": [1, 2, 3, 4, 9, 10, 33, 34, 42, 43, 90],           # a window of one key; around the kept 3 and 9 and the window of 33
}


def _requests(which):
    cfg, _page, seed = SIKE[which]
    return {f"q{i}": random_tokens(n, cfg["vocab"], seed * 100 + i) for i, n in enumerate(LENGTHS[which])}


def _oracles(pcfg, pw, requests):
    """Per request the plain logits in float64, and the worst row that rounding alone moves."""
    want = {rid: plain_forward(pcfg, pw, toks, torch.float64) for rid, toks in requests.items()}
    rounded = {rid: plain_forward(pcfg, pw, toks, torch.float64, cast=bf16_round) for rid, toks in requests.items()}
    order = sorted(want)
    row, _peak, _worst = parity.errors(torch.cat([rounded[r] for r in order]), torch.cat([want[r] for r in order]))
    return want, row


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


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_plain(tmp_path, which, dtype):
    cfg, page, seed = SIKE[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    longest = max(LENGTHS[which])
    schedules = {
        "whole": ru.whole(requests),
        "decode": ru.prefill_then_decode(requests, 50),
        "portions": ru.changing_portions(requests),
        "portions_of_two": ru.changing_portions(requests, sizes=(2, 2, 3, 2, 64, 2)),
        "mixed": ru.mixed(requests, seed, max_tokens=None),
        "mixed_tight": ru.mixed(requests, seed + 1, max_tokens=2 * 64 * ((longest + 63) // 64)),
    }
    first = None
    for label, steps in schedules.items():
        pages = ru.pages_for(steps, requests, page) + 1
        runner = _runner(model_dir, dtype, page, pages + 1, longest + 8)
        got = ru.run_in_process(runner, steps)
        _check(got, want, dtype, f"{which}/{dtype}/{label}", rounding)
        if dtype == "float32":
            # one order of summation however the requests are cut: the same bits
            if first is None:
                first = got
            else:
                for rid in got:
                    assert torch.equal(got[rid], first[rid]), (label, rid)
        runner.cache.check_invariants()
        assert not runner.cache.live_requests()
        del runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_slots_used_again(tmp_path, dtype):
    """Five requests through two slots, each a short prompt and then 300 tokens one by one, two
    at a time in a step: the windows pass over decoded tokens, their pages come back and are
    taken again by later requests, the kept first pages stay."""
    which = "A"
    cfg, page, seed = SIKE[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = {f"d{i}": random_tokens(300 + 7 * i, cfg["vocab"], 40 + i) for i in range(5)}
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, 3, max_live=2, tail=295)
    # windows of at most 41 keys and 21 kept ones: far fewer pages than the requests are long
    runner = _runner(model_dir, dtype, page, 2 * (-(-(41 + 21) // page) + 4) + 2, 340, slots=2)
    got = ru.run_in_process(runner, steps)
    _check(got, want, dtype, f"long decoding/{dtype}", rounding)
    runner.cache.check_invariants()


def test_trace_program(tmp_path):
    """``bin/trace_run`` as a child process on a mixed trace over a tight pool."""
    which = "B"
    cfg, page, seed = SIKE[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, seed + 5, max_tokens=256)
    got = ru.run_trace_program(model_dir, "float32", steps, tmp_path / "out", 256, cfg["vocab"])
    _check(got, want, "float32", "trace_run")
    assert rounding > 0


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "float32"), ("C", "bfloat16")])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype, use_graph):
    """``LLM.generate``: scheduler, chunked prompts beside decoding requests, sampling kernels;
    decode steps eagerly and replayed from graphs (in bfloat16 a recorded step holds the shares
    of a tile's keys and their merge).  The plain implementation re-runs the whole sequence for
    every token; a bfloat16 engine may pick another of several nearly equal maxima."""
    from rapid_llm_amd import LLM, SamplingParams

    cfg, page, seed = SIKE[which]
    model_dir = make_model_dir(tmp_path, which)
    pcfg, pw = load_plain(model_dir)
    prompts = [random_tokens(n, cfg["vocab"], seed + n) for n in (1, 7, 30, 45)]
    llm = LLM(str(model_dir), dtype=dtype, page_size=page, num_pages=60, max_num_seqs=3, max_seq_len=96,
              max_chunk_size=16, max_num_batched_tokens=32, use_cuda_graph=use_graph)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=24))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out.token_ids:
            logits = plain_forward(pcfg, pw, ids)[-1]
            if dtype == "float32":
                assert float(logits.max() - logits[tok]) <= 1e-3, (len(prompt), len(ids))
            else:
                parity.assert_near_choice(logits, tok, f"generation/{which}/graph={use_graph}")
            ids.append(tok)
        assert len(out.token_ids) == 24
    llm.scheduler.cache.check_invariants()
    assert not llm.scheduler.cache.live_requests()
