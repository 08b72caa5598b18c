"""Bokorax through the step function, the cache manager, the scheduler and the entry point, against the plain
implementation, under every way of cutting the work; and each of its mechanisms' kernels alone.

The model-level runs in float32 use folders whose routers choose freely; those in bfloat16 use the same folders with
steady routers (``cases.steady`` says why). The routers' free choice in bfloat16 is covered where it can be pinned: the
choice kernel on given logits, and the experts' kernels on given choices."""

import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import bokorax_cases as cases
from tests import helpers
from tests.helpers import Request
from tests.plain import bokorax_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
DTYPE_IDS = ["fp32", "bf16"]
NAMES = ["P", "Q", "R", "S"]
DEV = "cuda:0"
F64 = torch.float64


def _runner(folder, dtype, n_pages=64, max_requests=4, graphs=False):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(folder, dtype, torch.device(DEV))
    runner = make_runner(net, 16, n_pages, max_requests, enable_graphs=graphs)
    helpers.poison_cache(runner)
    return runner


def _ids(folder, seed, count):
    return helpers.random_ids(seed, count, cases.config_of(folder)["vocab"])


_EXPECTED = {}


def _expected(folder, ids):
    key = (folder, tuple(ids))
    if key not in _EXPECTED:
        _EXPECTED[key] = plain.forward(cases.config_of(folder), cases.stored_weights(folder), ids)
    return _EXPECTED[key]


_NOISY = {}


def _what_rounding_does(folder, ids):
    """Per row of logits, how far the plain implementation itself moves (root mean square over the vocabulary, mean taken
    off, as a share of the row's spread) when every weight is off by a relative 2 ** -8, about what rounding to bfloat16
    does to every intermediate value. The design has places where that is amplified without any fault: a router's choice
    is a step function of its scores (a near tie between two experts falls either way), and every sublayer's output is
    divided by its own root mean square."""
    if folder not in _NOISY:
        gen = torch.Generator().manual_seed(99)
        _NOISY[folder] = [{k: (v.double() * (1 + 2.0 ** -8 * torch.randn(v.shape, generator=gen, dtype=torch.float64)))
                           for k, v in cases.stored_weights(folder).items()} for _ in range(3)]
    want = _expected(folder, ids)
    worst = torch.zeros(want.shape[0], dtype=torch.float64)
    for noisy in _NOISY[folder]:
        moved = plain.forward(cases.config_of(folder), noisy, ids) - want
        moved = moved - moved.mean(dim=-1, keepdim=True)
        worst = torch.maximum(worst, moved.pow(2).mean(dim=-1).sqrt() / want.std(dim=-1, unbiased=False))
    return worst


def _close(got, want, dtype, what, folder=None, ids=None, rows=None):
    """Row by row: the root mean square of the difference over the vocabulary (mean taken off) as a share of the row's
    spread. float32: 1e-4; bfloat16: 4 %; and on rows where rounding alone is amplified by the design (measured on the
    plain implementation, ``_what_rounding_does``), 0.2 % (float32) and eight times (bfloat16) what that moves the row
    by. No single value may be off by more than four times its row's bound."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    diff = got - want
    diff = diff - diff.mean(dim=-1, keepdim=True)
    spread = want.std(dim=-1, unbiased=False)
    rms, top = diff.pow(2).mean(dim=-1).sqrt() / spread, diff.abs().max(dim=-1).values / spread
    floor, share = (1e-4, 2e-3) if dtype == torch.float32 else (0.04, 8.0)
    bound = torch.full_like(rms, floor)
    if folder is not None and not bool((rms <= bound).all() and (top <= 4 * bound).all()):
        moved = _what_rounding_does(folder, ids)
        bound = torch.maximum(bound, share * (moved[:len(rms)] if rows is None else moved[list(rows)]))
    worst = int(torch.argmax(rms / bound))
    assert bool((rms <= bound).all()) and bool((top <= 4 * bound).all()), \
        f"{what}: row {worst}: rms error {float(rms[worst]):.3g} of the spread (bound {float(bound[worst]):.3g}), largest {float(top[worst]):.3g}"


def _check(folder, dtype, requests, got, what):
    for tag, req in requests.items():
        _close(got[tag], _expected(folder, req.ids), dtype, f"{what} request {tag}", folder, req.ids)


def _near(got, want, dtype, what, atol=None, rtol=None):
    a, r = (2e-5, 2e-5) if dtype == torch.float32 else (3e-2, 2e-2)
    a, r = (atol if atol is not None else a), (rtol if rtol is not None else r)
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    bound = a + r * want.abs()
    assert bool((err <= bound).all()), f"{what}: max error {float(err.max()):.3g}, over its bound by {float((err - bound).max()):.3g}"


# ================================================================================================ kernels alone
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_token_shift_kernel(dtype):
    """A row that starts, one that goes on from its slot's kept row, a single token, a row without a request."""
    from kestrel_amd.ops import core

    gen = torch.Generator().manual_seed(3)
    dim, mixes = 70, 5
    counts, slots = [4, 3, 1, 2], [2, 0, 1, -1]
    n = sum(counts)
    x = torch.randn(n, dim, generator=gen)
    kept = torch.randn(4, dim + 9, generator=gen)                  # wider rows: the kept row lies behind other state
    mu = torch.rand(mixes, dim, generator=gen)
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    token_row = [r for r, c in enumerate(counts) for _ in range(c)]
    as_int = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    out = torch.full((mixes, n, dim), float("nan"), dtype=dtype, device=DEV)
    kept_dev = kept.to(DEV)
    core.token_shift(x.to(DEV), kept_dev[:, 9:], mu.to(DEV), as_int(token_row), as_int(cu), as_int(slots), out)
    for r, (c, slot) in enumerate(zip(counts, slots)):
        rows = x[cu[r]:cu[r + 1]].double()
        before = kept[slot, 9:].double() if slot >= 0 else None
        for s in range(mixes):
            _near(out[s, cu[r]:cu[r + 1]], plain.token_shift(rows, mu[s].double(), before), dtype, f"row {r} mix {s}", atol=1e-6 if dtype == torch.float32 else 2e-2)


def _run_decayed(dtype, d, heads, pieces_per_row, slots, seed, slow_decay=False):
    """Rows fed in the given pieces (a list of token counts per row, step by step); returns what the kernel wrote, what the
    plain recurrence gives, and the state after."""
    from kestrel_amd.ops import core

    gen = torch.Generator().manual_seed(seed)
    width = heads * d
    dim = 24
    n_slots = 5
    state = torch.zeros(n_slots + 1, width * d + dim, device=DEV)
    totals = [sum(p) for p in pieces_per_row]
    data = []
    for total in totals:
        r, k, v, g = (torch.randn(total, width, generator=gen).to(dtype).float() for _ in range(4))
        pre = torch.randn(total, width, generator=gen) - (4.0 if slow_decay else 0.5)
        data.append((r, k, v, g, pre))
    u = torch.randn(width, generator=gen)
    gain = 1 + 0.3 * torch.randn(width, generator=gen)
    got = [[] for _ in totals]
    at = [0] * len(totals)
    steps = max(len(p) for p in pieces_per_row)
    as_int = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for step in range(steps):
        rows = [i for i, p in enumerate(pieces_per_row) if step < len(p) and p[step] > 0]
        counts = [pieces_per_row[i][step] for i in rows]
        cat = lambda j: torch.cat([data[i][j][at[i]:at[i] + c] for i, c in zip(rows, counts)])
        rkvg = torch.cat([cat(0), cat(1), cat(2), cat(3)], dim=1).to(DEV, dtype)
        pre = cat(4).to(DEV).contiguous()
        n = rkvg.shape[0]
        cu = [0]
        for c in counts:
            cu.append(cu[-1] + c)
        out = torch.full((n, width), float("nan"), dtype=dtype, device=DEV)
        x = torch.randn(n, dim, generator=gen).to(DEV)
        core.decayed_memory(rkvg[:, :width], rkvg[:, width:2 * width], rkvg[:, 2 * width:3 * width], rkvg[:, 3 * width:], pre, u.to(DEV),
                            gain.to(DEV), state, x, as_int(cu), as_int([slots[i] for i in rows]), out, heads, d, 1e-5)
        torch.cuda.synchronize()
        for j, (i, c) in enumerate(zip(rows, counts)):
            got[i].append(out[cu[j]:cu[j + 1]].double().cpu())
            if slots[i] >= 0:
                assert torch.equal(state[slots[i], width * d:].cpu(), x[cu[j + 1] - 1].cpu()), "the stream's last row is kept"
            at[i] += c
    want = []
    for (r, k, v, g, pre) in data:
        decay = torch.exp(-torch.exp(pre.double()))
        heads_out = []
        for a in range(heads):
            sl = slice(a * d, (a + 1) * d)
            o, _ = plain.wkv_recurrence(r[:, sl].double(), k[:, sl].double(), v[:, sl].double(), decay[:, sl], u[sl].double())
            heads_out.append(plain.rms(o, 1e-5))
        want.append(torch.cat(heads_out, dim=-1) * gain.double() * g.double())
    return [torch.cat(p) for p in got], want


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("d, heads", [(16, 3), (20, 2), (48, 2), (64, 4), (128, 2), (256, 1), (1, 2)])
def test_decayed_memory_kernel(dtype, d, heads):
    """Rows of 1 to 150 tokens cut into a prompt, portions and single tokens, beside a row without a request, at head sizes
    that fill a thread's registers exactly, partly, and that are no power of two; fast and slow decays."""
    pieces = [[150], [1, 1, 1, 1, 1, 1, 1], [17, 2, 0, 33, 1, 1, 40], [0, 0, 3, 0, 1], [5, 5]]
    slots = [0, 1, 2, 3, -1]
    for slow in (False, True):
        got, want = _run_decayed(dtype, d, heads, pieces, slots, seed=d + heads, slow_decay=slow)
        for row, (a, b) in enumerate(zip(got, want)):
            if slots[row] < 0:
                assert float(a.abs().max()) == 0.0, "a row without a request writes zeros"
            else:
                _near(a, b, dtype, f"d {d} row {row} slow {slow}", atol=2e-4 if dtype == torch.float32 else 4e-2, rtol=2e-4 if dtype == torch.float32 else 3e-2)


def test_a_slot_used_again_starts_from_nothing():
    """The cache manager clears a slot's state at admission: the second request in a slot must not see the first's."""
    folder = cases.model_dir("P")
    runner = _runner(folder, torch.float32, max_requests=1)
    for seed in (1, 2):
        reqs = {"r": Request("r", _ids(folder, 40 + seed, 30))}
        _check(folder, torch.float32, reqs, helpers.replay(runner, reqs, [[("r", 20)], [("r", 10)]]), f"use {seed}")


@pytest.mark.parametrize("outputs, top, groups, keep", [(10, 2, 2, 1), (8, 3, 4, 2), (5, 1, 0, 0), (64, 8, 8, 3), (200, 6, 10, 4),
                                                         (3, 3, 1, 1), (2, 2, 0, 0), (512, 4, 64, 2)])
def test_route_kernel(outputs, top, groups, keep):
    """The choice and the weights against the plain router on the same fp32 logits: groups, corrections that make choice
    scores negative (a group that is not kept counts as minus infinity, not as zero), more choices than a group holds."""
    from kestrel_amd.ops import core

    gen = torch.Generator().manual_seed(outputs + top)
    n, dim = 37, 16
    h = torch.randn(n, dim, generator=gen)
    router = torch.randn(outputs, dim, generator=gen) * 0.6
    correction = torch.randn(outputs, generator=gen) * 0.3 - 0.5            # mostly negative choice scores
    logits = torch.zeros(n, outputs + 1)
    logits[:, :outputs] = (h.double() @ router.double().T).float()
    r = {"top": top, "scale": 1.7}
    if groups:
        r["groups"] = {"count": groups, "keep": keep}
    # the plain router on exactly these logits: an identity "projection" of them
    want_i, want_w = plain.route(logits[:, :outputs].double(), torch.eye(outputs, dtype=F64), correction.double(), r)
    chosen = torch.zeros(n, top, dtype=torch.int32, device=DEV)
    weights = torch.zeros(n, top, device=DEV)
    core.route(logits.to(DEV), outputs, correction.to(DEV), top, groups, keep, 1.7, chosen, weights)
    got_i, got_w = chosen.cpu().long(), weights.cpu().double()
    for t in range(n):
        a = dict(zip(got_i[t].tolist(), got_w[t].tolist()))
        b = dict(zip(want_i[t].tolist(), want_w[t].tolist()))
        assert set(a) == set(b), f"token {t}: chose {sorted(a)}, plain {sorted(b)}"
        for e in a:
            assert abs(a[e] - b[e]) <= 1e-5 * max(1.0, abs(b[e])), f"token {t} expert {e}: {a[e]} vs {b[e]}"


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("n, dim, ff, n_experts, top", [(5, 40, 24, 3, 2), (70, 64, 48, 6, 3), (300, 128, 80, 9, 2), (1, 16, 16, 1, 1)])
def test_experts_linears_and_sum(dtype, n, dim, ff, n_experts, top):
    """The experts' two linears pair by pair and the weighted sum with identity experts and a gated shared expert; in
    bfloat16 also the pairs listed by expert through the matrix-core kernel, which must give what pair by pair gives."""
    from kestrel_amd.ops import core, fast
    from kestrel_amd.ops.linear import ACT_GATED, activation_code, pair_rows

    gen = torch.Generator().manual_seed(n + dim)
    rnd = lambda *shape: (torch.randn(*shape, generator=gen) * 0.3).to(dtype)
    h = rnd(n, dim)
    gate, up, down = rnd(n_experts, ff, dim), rnd(n_experts, ff, dim), rnd(n_experts, dim, ff)
    identity = 2
    chosen = torch.stack([torch.randperm(n_experts + identity, generator=gen)[:top] for _ in range(n)]).to(torch.int32)
    weights = torch.rand(n, top, generator=gen)
    shared, sg = torch.randn(n, dim, generator=gen), torch.randn(n, generator=gen)
    w = {}
    for e in range(n_experts):
        w.update({f"e{e}.gate": gate[e].double(), f"e{e}.up": up[e].double(), f"e{e}.down": down[e].double()})
    want = torch.zeros(n, dim, dtype=F64)
    for t in range(n):
        for k in range(top):
            e = int(chosen[t, k])
            want[t] += float(weights[t, k]) * (plain.expert(h[t:t + 1].double(), w, f"e{e}.")[0] if e < n_experts else h[t].double())
    want = want + torch.sigmoid(sg.double())[:, None] * shared.double()
    pairs = torch.stack([pair_rows(gate[e], up[e]) for e in range(n_experts)]).to(DEV)
    act = activation_code("silu")
    hidden = torch.zeros(n * top, ff, dtype=dtype, device=DEV)
    y = torch.full((n * top, dim), float("nan"), device=DEV)
    flat = chosen.to(DEV).view(-1)
    core.experts_linear(h.to(DEV), top, pairs, flat, hidden, act | ACT_GATED)
    core.experts_linear(hidden, 1, down.to(DEV), flat, y)
    out = torch.ones(n, dim, device=DEV)
    gate_column = torch.stack([torch.zeros(n), sg], dim=1).to(DEV)[:, 1]          # a column with a stride
    core.experts_combine(y, h.to(DEV), chosen.to(DEV), weights.to(DEV), n_experts, shared.to(DEV), gate_column, out, True)
    _near(out - 1, want, dtype, "pair by pair", atol=1e-5 if dtype == torch.float32 else 2e-2)
    if dtype == torch.bfloat16 and dim % 16 == 0 and ff % 16 == 0:
        from kestrel_amd.engine.batch import Workspace
        y2 = torch.full((n * top, dim), float("nan"), device=DEV)
        assert fast.experts_feed_forward_bf16(h.to(DEV), pairs, down.to(DEV), chosen.to(DEV), None, y2, act, Workspace(torch.device(DEV)))
        live = (chosen < n_experts).view(-1)
        _near(y2[live.to(DEV)], y[live.to(DEV)], dtype, "by expert against pair by pair", atol=1e-2, rtol=2e-2)


@pytest.mark.parametrize("kernel, dtype", [("generic", torch.float32), ("generic", torch.bfloat16), ("mfma", torch.bfloat16)],
                         ids=["generic-fp32", "generic-bf16", "mfma-bf16"])
@pytest.mark.parametrize("heads, kv_heads, d, dv", [(4, 2, 32, 64), (2, 2, 64, 64), (4, 1, 128, 128), (6, 3, 48, 32)])
def test_capped_scores_sinks_per_head_and_a_gate_per_head(kernel, dtype, heads, kv_heads, d, dv):
    """Attention whose scores pass through a cap (the scale is large, so the cap decides), with a sink score per head that
    dominates for some heads and is negligible for others, and a gate of one number per head; prompts, portions and single
    tokens in one launch, and a decode step."""
    from kestrel_amd.ops import core, fast
    from tests.test_biased_attention_gpu import Case

    for lengths, starts in (([70, 133, 9, 2, 64], [0, 100, 7, 0, 63]), ([1, 17, 250, 33], [0, 16, 249, 32])):
        case = Case(dtype, heads, kv_heads, d, dv, lengths=lengths, starts=starts, window=None, seed=heads + d)
        scale, cap = 0.9, 4.0
        sinks = torch.tensor([(-1) ** a * 3.0 * (a + 1) / heads for a in range(heads)])
        gate = torch.randn(case.n, heads, generator=torch.Generator().manual_seed(5)).to(dtype)
        out = torch.full((case.n, heads * dv), float("nan"), dtype=dtype, device=DEV)
        args = (case.q, case.k_cache, case.v_cache, case.table, case.token_row, None, case.kv_hi, out, scale, heads, kv_heads, d, dv,
                case.positions, None, None)
        more = dict(gate=gate.to(DEV), sinks=sinks.to(DEV), softcap=cap, gate_per_head=True)
        if kernel == "generic":
            core.attention_generic(*args, **more)
        else:
            assert fast.attention_biased_bf16(*args, case.batch(), **more), "the matrix-core kernel declined sizes it is meant to take"
        torch.cuda.synchronize()
        want, at = [], 0
        for q, k, v, n, s in zip(case.q_rows, case.k_rows, case.v_rows, lengths, starts):
            seen = plain.window_mask(n, None)[s:]
            o = plain.grouped_attention(q, k, v, scale, seen, cap, sinks.double())
            o = o * torch.sigmoid(gate[at:at + n - s].double())[:, :, None]
            want.append(o.reshape(n - s, heads * dv))
            at += n - s
        _near(out, torch.cat(want), dtype, f"{kernel} {lengths}")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("d, rot", [(24, 12), (64, 32), (128, 128), (32, 16)])
def test_prepare_kernel_values_from_keys_and_queries_alone(dtype, d, rot):
    """The prepare kernel with values that are the keys as projected (the value pages get the unnormalised, unrotated keys)
    and with rows of queries alone (a layer that reads another layer's cache): norm over the projection, rotation by halves;
    at a head size only the general form takes and at those of the form that gives a lane eight channels (bfloat16)."""
    from kestrel_amd.ops import core

    gen = torch.Generator().manual_seed(8)
    n, H, G, page = 21, 4, 2, 16
    eps = 1e-5
    places = list(range(3, 3 + n))
    freqs = plain.frequencies({"dims": rot, "base": 40.0})
    rows = torch.randn(n, (H + G) * d, generator=gen).to(dtype)
    q_gain, k_gain = 1 + 0.2 * torch.randn(H * d, generator=gen), 1 + 0.2 * torch.randn(G * d, generator=gen)
    k_cache = torch.full((3, G, page, d), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((3, G, d, page), float("nan"), dtype=dtype, device=DEV)
    slots = torch.arange(5, 5 + n, dtype=torch.int32, device=DEV)
    qk = rows.to(DEV).clone()
    as_f = lambda t: t.to(DEV, torch.float32).contiguous()
    core.qkv_prepare(qk, torch.tensor(places, dtype=torch.int32, device=DEV), slots, k_cache, v_cache, H, G, d, d, page, "projection",
                     as_f(q_gain), as_f(k_gain), eps, as_f(torch.tensor(freqs)), "halves", values_from_keys=True)
    q64, k64 = rows[:, :H * d].double(), rows[:, H * d:].double()
    want_q = plain.rotate_halves((plain.rms(q64, eps) * q_gain.double()).reshape(n, H, d), places, freqs).reshape(n, H * d)
    want_k = plain.rotate_halves((plain.rms(k64, eps) * k_gain.double()).reshape(n, G, d), places, freqs)
    tol = dict(atol=5e-6, rtol=5e-6) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    _near(qk[:, :H * d], want_q, dtype, "queries", **tol)
    for t in range(n):
        slot = 5 + t
        _near(k_cache[slot // page, :, slot % page], want_k[t], dtype, f"key {t}", **tol)
        assert torch.equal(v_cache[slot // page, :, :, slot % page].cpu().double(), k64[t].reshape(G, d)), "the values are the keys as projected"
    alone = rows[:, :H * d].to(DEV).clone()
    core.qkv_prepare(alone, torch.tensor(places, dtype=torch.int32, device=DEV), None, None, None, H, 0, d, d, page, "projection",
                     as_f(q_gain), None, eps, as_f(torch.tensor(freqs)), "halves")
    _near(alone, want_q, dtype, "queries alone", **tol)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rows", [1, 9, 70, 300])
def test_tanh_in_every_linear_kernel(rows, dtype):
    from kestrel_amd.ops.linear import activation_code, linear

    gen = torch.Generator().manual_seed(rows)
    a, w = torch.randn(rows, 64, generator=gen).to(dtype), (torch.randn(48, 64, generator=gen) * 0.2).to(dtype)
    out = torch.zeros(rows, 48, dtype=dtype, device=DEV)
    linear(a.to(DEV), w.to(DEV), None, out, act=activation_code("tanh"))
    _near(out, torch.tanh(a.double() @ w.double().T), dtype, "tanh", atol=1e-5 if dtype == torch.float32 else 2e-2)


# ================================================================================================ the model, cut every way
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_every_layer(name, dtype):
    """The residual stream after every layer, then the logits."""
    from kestrel_amd.parts.block import Block

    folder = cases.folder_for(name, dtype)
    runner = _runner(folder, dtype)
    ids = _ids(folder, 1, 45)
    seen = []
    original = Block.forward

    def spy(self, x, *args, **kwargs):
        result = original(self, x, *args, **kwargs)
        seen.append(x.detach().double().cpu())
        return result

    Block.forward = spy
    try:
        got = helpers.replay(runner, {"r": Request("r", ids)}, [[("r", len(ids))]])
    finally:
        Block.forward = original
    streams = []
    want = plain.forward(cases.config_of(folder), cases.stored_weights(folder), ids, streams)
    assert len(seen) == len(streams)
    # what a relative 2 ** -8 on every weight does to the plain streams (the norms behind the sublayers turn a small
    # output's rounding into a large step of the stream)
    _what_rounding_does(folder, ids)
    noisy = []
    for weights in _NOISY[folder]:
        moved = []
        plain.forward(cases.config_of(folder), weights, ids, moved)
        noisy.append(moved)
    for layer, (a, b) in enumerate(zip(seen, streams)):
        per_row = (a - b).abs().max(dim=1).values
        by_rounding = max(float((other[layer] - b).abs().max(dim=1).values.quantile(0.9)) for other in noisy)
        bound = max(1e-4 * float(b.abs().max()), 2e-3 * by_rounding) if dtype == torch.float32 else max(6e-2 * float(b.abs().max()), 4 * by_rounding)
        assert float(per_row.quantile(0.9)) <= bound, f"{name} layer {layer}: {float(per_row.quantile(0.9)):.3g} > {bound:.3g}"
    _close(got["r"], want, dtype, f"{name} logits", folder, ids)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(name, dtype):
    """Each request alone and whole: the first tokens of a sequence (1, 2, 3), lengths around a page's and a window's edges,
    and well beyond every window."""
    folder = cases.folder_for(name, dtype)
    runner = _runner(folder, dtype)
    for seed, length in enumerate([1, 2, 3, 7, 8, 16, 17, 33, 40, 41, 65, 120, 260]):
        reqs = {"r": Request("r", _ids(folder, 100 + seed, length))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", length)]]), f"{name} whole {length}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(name, dtype, graphs):
    """Most of the request in one step, then one token a step across the window's edge; and a request decoded from its very
    first token (the memory's state starts at zero and is carried through every step, the token before comes from it)."""
    folder = cases.folder_for(name, dtype)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, (length, head) in enumerate([(150, 60), (70, 1), (48, 47)]):
        reqs = {"r": Request("r", _ids(folder, 200 + seed, length))}
        got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (length - head))
        _check(folder, dtype, reqs, got, f"{name} decode {length}/{head}")
    assert (runner.graph_replays > 0) == graphs


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(name, dtype, graphs):
    """Portions cut anywhere: in the middle of a page and of a window, down to two tokens."""
    folder = cases.folder_for(name, dtype)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, cuts in enumerate([[2, 2, 3, 9, 16, 1, 31, 2, 40, 5, 64, 2], [17, 2, 2, 2, 50], [33, 32, 31, 7]]):
        reqs = {"r": Request("r", _ids(folder, 300 + seed, sum(cuts)))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", c)] for c in cuts]), f"{name} portions {seed}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_in_reused_pages_and_slots(name, dtype, graphs):
    """Up to four live requests of unequal lengths, portions of some beside single tokens of others, in a pool so small
    that pages and state slots are used again (what is given back is filled with NaN first); every request must come
    out as it does alone."""
    folder = cases.folder_for(name, dtype)
    lengths = {"a": 90, "b": 37, "c": 61, "d": 5, "e": 130, "f": 44, "g": 2}
    runner = _runner(folder, dtype, n_pages=24, max_requests=4, graphs=graphs)
    reqs = {tag: Request(tag, _ids(folder, 400 + i, n)) for i, (tag, n) in enumerate(lengths.items())}
    steps = [[("a", 50), ("b", 20)], [("a", 1), ("b", 17), ("c", 30)], [("a", 1), ("c", 2), ("d", 5)],
             [("a", 38), ("c", 29)],                                  # a, c and d end; b ended before
             [("e", 64), ("f", 3)], [("e", 1), ("f", 41), ("g", 2)], [("e", 1)], [("e", 62)], [("e", 1)], [("e", 1)]]
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, f"{name} mixed")
    assert runner.cache.free_slots == 4


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_long_decoding_under_graphs(dtype):
    """Three hundred tokens one by one beside a second request that comes and goes: the window passes, its pages go back."""
    folder = cases.folder_for("P", dtype)
    runner = _runner(folder, dtype, n_pages=24, max_requests=2, graphs=True)
    reqs = {"long": Request("long", _ids(folder, 500, 300)), "short": Request("short", _ids(folder, 501, 25))}
    steps = [[("long", 3)]] + [[("long", 1)]] * 100 + [[("long", 1), ("short", 20)]] + [[("long", 1), ("short", 1)]] * 5 \
        + [[("long", 1)]] * 191
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, "long decoding")
    assert not runner.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_a_far_key_the_windows_edge_and_the_memory_in_the_model(dtype):
    """On a folder crafted so that it shows (``cases.crafted``; ``test_bokorax_cpu.py`` measures by how much): a token that
    calls and, at a chosen distance before it, its echo, among tokens that are all different: just inside and just outside
    the window, at a page's border, far back (seen by the layers without a window and kept by the memory), and at the
    sequence's first place; inside a prompt, decoded alone, and with all but two tokens decoded."""
    base = cases.folder_for("P", dtype)
    folder = cases.crafted(base)
    window = cases.config_of(base)["layers"][2]["mixer"]["mask"]["size"]
    length = 3 * window + 20
    at = length - 7
    for distance in (window - 1, window, 1, 16, 17, 2 * window + 5, at):
        ids = list(range(10, 10 + length))
        ids[at], ids[at - distance] = cases.CALL, cases.ECHO
        want = _expected(folder, ids)
        for head in (len(ids), at - 3, 2):
            if head == 2 and distance not in (window, at):
                continue
            runner = _runner(folder, dtype)
            reqs = {"r": Request("r", ids)}
            got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (len(ids) - head))
            _close(got["r"], want, dtype, f"distance {distance}, prompt of {head}", folder, ids)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(name, dtype):
    """Requests of different lengths submitted together through ``InferenceEngine``: the scheduler cuts prompts into
    portions beside the decoding of the others; with and without graphs, one and two steps in flight."""
    from kestrel_amd import InferenceEngine, RuntimeConfig

    folder = cases.folder_for(name, dtype)
    config, weights = cases.config_of(folder), cases.stored_weights(folder)
    prompts = [_ids(folder, 600 + i, n) for i, n in enumerate([5, 17, 33, 70])]
    n_new = 24
    slack = 1e-4 if dtype == "float32" else 8e-2
    for graphs, depth in ((False, 1), (True, 2)):
        engine = InferenceEngine.create_sync(RuntimeConfig(model_path=folder, dtype=dtype, max_batch_size=4, kv_cache_pages=40,
                                                           max_num_batched_tokens=48, enable_graphs=graphs, pipeline_depth=depth,
                                                           max_seq_len=128))
        try:
            results = engine.generate_batch_sync(prompts, max_new_tokens=n_new, temperature=0.0, stop_ids=())
        finally:
            engine.shutdown_sync()
        for prompt, result in zip(prompts, results):
            assert result.finish_reason == "length" and len(result.tokens) == n_new
            logits = plain.forward(config, weights, list(prompt) + list(result.tokens[:-1]))
            for i, token in enumerate(result.tokens):
                row = logits[len(prompt) - 1 + i]
                gap = float(row.max() - row[token])
                assert gap <= slack * max(1.0, float(row.std())), \
                    f"{name} {dtype} graphs={graphs}: token {i} is {token}, plain gives {int(row.argmax())} ({gap:.3g} better)"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(dtype, tmp_path):
    """``bin/trace_run`` on a folder of this architecture whose ``config.json`` leaves the decay's rank to the weights file:
    steps from standard input, logits into files, a request left out of a step, slots and pages used again."""
    def drop_rank(config):
        for layer in config["layers"]:
            layer["mixer"].pop("decay_rank", None)

    folder = cases.rewrite(cases.folder_for("Q", dtype), lambda w: None, drop_rank)
    ids = {tag: _ids(folder, 700 + i, n) for i, (tag, n) in enumerate({"a": 40, "b": 9, "c": 70, "d": 3, "e": 21}.items())}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids["a"][:30], "want": [0, 29]}, {"id": "b", "tokens": ids["b"], "want": [8]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "c", "tokens": ids["c"][:64], "want": []}, {"id": "d", "tokens": ids["d"], "want": [0, 1, 2]},
                                {"id": "e", "tokens": ids["e"][:2], "want": [1]}], "end": ["d"]},
        {"step": 2, "entries": [{"id": "c", "tokens": ids["c"][64:], "want": [5]}, {"id": "a", "tokens": ids["a"][30:], "want": [0, 9]},
                                {"id": "e", "tokens": ids["e"][2:], "want": [18]}], "end": ["a", "c", "e"]},
    ]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                          capture_output=True, timeout=600, cwd=ROOT)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    full = {tag: _expected(folder, seq) for tag, seq in ids.items()}
    wanted = {0: [("a", 0), ("a", 29), ("b", 8)], 1: [("d", 0), ("d", 1), ("d", 2), ("e", 1)], 2: [("c", 69), ("a", 30), ("a", 39), ("e", 20)]}
    vocab = cases.config_of(folder)["vocab"]
    run_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    for step, places in wanted.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(places), vocab))
        want = torch.stack([full[tag][p] for tag, p in places])
        for row, (tag, p) in enumerate(places):
            _close(got[row:row + 1], want[row:row + 1], run_dtype, f"trace step {step} {tag}[{p}]", folder, ids[tag], rows=[p])


def test_command_line(tmp_path):
    """``python -m kestrel_amd random-weights`` from a configuration of this design, then ``generate`` on the folder."""
    import sys

    env = dict(os.environ, PYTHONPATH=ROOT)
    config = tmp_path / "cfg.json"
    config.write_text(json.dumps(cases.CONFIGS["S"]))
    made = subprocess.run([sys.executable, "-m", "kestrel_amd", "random-weights", "--out", str(tmp_path / "m"), "--config", str(config),
                           "--seed", "5", "--std", "0.08", "--bias-std", "0.5", "--gain-std", "0.2"], capture_output=True, text=True,
                          env=env, cwd=ROOT)
    assert made.returncode == 0, made.stderr
    folder = str(tmp_path / "m")
    prompt = _ids(folder, 990, 9)
    done = subprocess.run([sys.executable, "-m", "kestrel_amd", "generate", "--model-path", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0",
                           "--kv-cache-pages", "8", "--max-seq-len", "64"], capture_output=True, text=True, env=env, cwd=ROOT,
                          timeout=300)
    assert done.returncode == 0, done.stderr
    tokens = json.loads(done.stdout.strip().splitlines()[-1])["tokens"]
    assert len(tokens) == 6
