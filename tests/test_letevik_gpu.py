"""Letevik through the step function, the cache manager, the scheduler and the entry point, against the plain
implementation, under every way of cutting the work; and each of its mechanisms' kernels alone."""

import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import helpers
from tests import letevik_cases as cases
from tests.helpers import Request
from tests.plain import letevik_plain as plain

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
        _EXPECTED[key] = plain.forward(ids, cases.stored_weights(folder), cases.config_of(folder))
    return _EXPECTED[key]


_NOISY = {}


def _what_rounding_does(folder, ids):
    """Per row of logits, how far the plain implementation itself moves (root mean square over the vocabulary, mean taken
    off, as a share of the row's spread) when every weight is off by a relative 2 ** -8, about what rounding to bfloat16
    does to every intermediate value. The design amplifies that without any fault where the two maps of a head nearly
    cancel: the difference is divided by its own root mean square."""
    if folder not in _NOISY:
        gen = torch.Generator().manual_seed(99)
        _NOISY[folder] = [{k: (v.double() * (1 + 2.0 ** -8 * torch.randn(v.shape, generator=gen, dtype=F64)))
                           for k, v in cases.stored_weights(folder).items()} for _ in range(3)]
    want = _expected(folder, ids)
    worst = torch.zeros(want.shape[0], dtype=F64)
    for noisy in _NOISY[folder]:
        moved = plain.forward(ids, noisy, cases.config_of(folder)) - want
        moved = moved - moved.mean(dim=-1, keepdim=True)
        worst = torch.maximum(worst, moved.pow(2).mean(dim=-1).sqrt() / want.std(dim=-1, unbiased=False))
    return worst


def _close(got, want, dtype, what, folder=None, ids=None, rows=None):
    """Row by row: the root mean square of the difference over the vocabulary (mean taken off) as a share of the row's
    spread. float32: 1e-4; bfloat16: 4 %; and on rows where rounding alone is amplified by the design (measured on the
    plain implementation, ``_what_rounding_does``), 0.2 % (float32) and six times (bfloat16) what that moves the row by.
    No single value may be off by more than four times its row's bound. A fault of a mechanism moves rows by far more
    (the constructions below ask for several times the bound)."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    diff = got - want
    diff = diff - diff.mean(dim=-1, keepdim=True)
    spread = want.std(dim=-1, unbiased=False)
    rms, top = diff.pow(2).mean(dim=-1).sqrt() / spread, diff.abs().max(dim=-1).values / spread
    floor, share = (1e-4, 2e-3) if dtype == torch.float32 else (0.04, 6.0)
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


def _apart(a, b):
    """How far two rows of logits are apart, in the measure of ``_close``."""
    d = (a - b) - (a - b).mean()
    return float(d.pow(2).mean().sqrt() / a.std(unbiased=False))


# ------------------------------------------------------------------------------------------------ the model, cut every way
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_every_layer(name, dtype):
    """The residual stream after every run of a layer (a looped layer counts each time), then the logits."""
    from kestrel_amd.parts.block import Block

    folder = cases.model_dir(name)
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
    want = plain.forward(ids, cases.stored_weights(folder), cases.config_of(folder), streams)
    assert len(seen) == len(streams) == len(plain.layer_order(cases.config_of(folder)))
    for layer, (a, b) in enumerate(zip(seen, streams)):
        per_row = (a - b).abs().max(dim=1).values
        bound = (1e-4 if dtype == torch.float32 else 6e-2) * float(b.abs().max())
        assert float(per_row.quantile(0.9)) <= bound, f"{name} layer run {layer}: {float(per_row.quantile(0.9)):.3g} > {bound:.3g}"
    _close(got["r"], want, dtype, f"{name} logits", folder, ids)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(name, dtype):
    """Each request alone and whole: the first tokens of a sequence (1, 2, 3: shorter than the convolutions' taps), lengths
    around a page's and every window's edge, and well beyond every window."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    for seed, length in enumerate([1, 2, 3, 4, 7, 8, 16, 17, 24, 25, 33, 34, 41, 48, 49, 65, 120, 260]):
        reqs = {"r": Request("r", _ids(folder, 100 + seed, length))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", length)]]), f"{name} whole {length}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(name, dtype, graphs):
    """Most of the request in one step, then one token a step while windows pass over decoded tokens and the kept first
    keys stay; and a request decoded from its very first token (the convolutions' state and the token before start empty)."""
    folder = cases.model_dir(name)
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
    """Portions cut anywhere: in the middle of a page and of a window, shorter than the convolutions' taps, down to two tokens."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, cuts in enumerate([[2, 2, 3, 9, 16, 1, 31, 2, 40, 5, 64, 2], [17, 2, 2, 2, 50], [33, 32, 31, 7], [1, 1, 2, 1, 3, 30]]):
        reqs = {"r": Request("r", _ids(folder, 300 + seed, sum(cuts)))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", c)] for c in cuts]), f"{name} portions {seed}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_in_reused_pages_and_slots(name, dtype, graphs):
    """Up to four live requests of unequal lengths, portions of some beside single tokens of others, in a pool so small
    that pages and state slots are used again (what is given back is filled with NaN first); every request must come
    out as it does alone."""
    folder = cases.model_dir(name)
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
    """Three hundred tokens one by one beside a second request that comes and goes: windows pass, their pages go back, the
    pages of the kept first keys stay."""
    folder = cases.model_dir("P")
    runner = _runner(folder, dtype, n_pages=24, max_requests=2, graphs=True)
    reqs = {"long": Request("long", _ids(folder, 500, 300)), "short": Request("short", _ids(folder, 501, 25))}
    steps = [[("long", 3)]] + [[("long", 1)]] * 100 + [[("long", 1), ("short", 20)]] + [[("long", 1), ("short", 1)]] * 5 \
        + [[("long", 1)]] * 191
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, "long decoding")
    assert not runner.cache.live_slots


# ------------------------------------------------------------------------------------------------ faults that random weights hide
def _standing_out():
    base = cases.model_dir("T")
    config = cases.config_of(base)
    return cases.rewrite(base, lambda w: cases.stand_out(w, config)), config


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_a_far_key_the_windows_edge_and_the_kept_first_keys_in_the_model(dtype):
    """A token repeated at chosen places among tokens that are all different. With the keys' weights on the queries the
    repeated token's score stands out: in the latent layers at any distance, in the differential layers inside the window
    and among the kept first keys only. A window or a count of kept keys that is one off, a far key that is lost, or a page
    of kept keys that was given back changes the logits far beyond rounding: in a prompt and decoded."""
    folder, config = _standing_out()
    mask = config["layers"][0]["mixer"]["mask"]
    window, kept = mask["size"], mask["keep_first"]
    length, at = 150, 140
    places = [at - window + 1, at - window, at - 1, kept - 1, kept, 0, at - 100, at - 2 * window]
    for place in places:
        ids = list(range(10, 10 + length))                          # all different
        ids[at] = ids[place]
        want = _expected(folder, ids)
        for head in (length, at - 5, 2):                            # the repeat inside the prompt; decoded alone; all decoded
            runner = _runner(folder, dtype)
            reqs = {"r": Request("r", ids)}
            got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (length - head))
            _close(got["r"], want, dtype, f"repeat of place {place}, prompt of {head}", folder, ids)

    # the construction shows each edge: moving the repeat across it changes that token's logits by several bounds
    def moved(p1, p2):
        one, two = list(range(10, 10 + length)), list(range(10, 10 + length))
        one[at], two[at] = one[p1], two[p2]
        return _apart(_expected(folder, one)[at], _expected(folder, two)[at])
    assert moved(at - window + 1, at - window) > 0.16 and moved(kept - 1, kept) > 0.16, \
        (moved(at - window + 1, at - window), moved(kept - 1, kept))
    # and the far key: a model whose latent layers saw only the last 64 keys would differ as much
    unrepeated = list(range(10, 10 + length))
    one = list(unrepeated)
    one[at] = one[at - 100]
    assert _apart(_expected(folder, one)[at], _expected(folder, unrepeated)[at]) > 0.16


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_sinks_of_every_head_show(dtype):
    """Sinks of a few units, different per head: leaving them out, scaling them or giving every head the same one would move
    the logits by far more than the bound (shown on the plain implementation), and the kernels follow the plain one."""
    base = cases.model_dir("P")
    config = cases.config_of(base)

    def edit(weights):
        for i, layer in enumerate(config["layers"]):
            if layer["type"] == "latent_attention":
                heads = layer["mixer"]["heads"]
                weights[f"l{i}.mix.sink"] = torch.tensor([3.0 - 2.5 * h for h in range(heads)]).to(torch.bfloat16)

    def none(weights):
        edit(weights)
        for name in weights:
            if name.endswith(".sink"):
                weights[name] = torch.full_like(weights[name], -60.0)

    def same(weights):
        edit(weights)
        for name in weights:
            if name.endswith(".sink"):
                weights[name] = torch.full_like(weights[name], float(weights[name][0]))

    folder = cases.rewrite(base, edit)
    ids = _ids(folder, 800, 70)
    want = _expected(folder, ids)
    for other in (none, same):
        far = _expected(cases.rewrite(base, other), ids)
        assert min(_apart(want[t], far[t]) for t in (0, 1, 30, 69)) > 0.16
    runner = _runner(folder, dtype)
    reqs = {"r": Request("r", ids)}
    _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", 40)]] + [[("r", 1)]] * 30), "sinks")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_the_token_before_and_the_pass_vectors_show(dtype):
    """The pair embedding and the vector of every pass made large: a lost previous token (at the start of a portion, in a
    slot that another request used before) or a pass that takes another pass's vector moves the logits far."""
    base = cases.model_dir("Q")

    def edit(weights):
        weights["bigram"] = (weights["bigram"].float() * 6).to(torch.bfloat16)
        weights["loop.step"] = (weights["loop.step"].float() * 6).to(torch.bfloat16)

    def swapped(weights):
        edit(weights)
        weights["loop.step"] = weights["loop.step"].flip(0).contiguous()

    folder = cases.rewrite(base, edit)
    ids = _ids(folder, 810, 40)
    want = _expected(folder, ids)
    assert _apart(want[20], _expected(cases.rewrite(base, swapped), ids)[20]) > 0.16
    assert _apart(want[20], _expected(folder, ids[:19] + [ids[19] + 1] + ids[20:])[20]) > 0.16
    runner = _runner(folder, dtype, max_requests=1)
    for cuts in ([40], [20, 1, 1, 18], [2] * 20):
        reqs = {"r": Request("r", ids)}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", c)] for c in cuts], poison=True), f"cuts {cuts[:3]}")


# ------------------------------------------------------------------------------------------------ entry point, programs
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(name, dtype):
    """Requests of different lengths submitted together through ``InferenceEngine``: the scheduler cuts prompts into
    portions beside the decoding of the others; with and without graphs, one and two steps in flight."""
    from kestrel_amd import InferenceEngine, RuntimeConfig

    folder = cases.model_dir(name)
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
            logits = plain.forward(list(prompt) + list(result.tokens[:-1]), weights, config)
            for i, token in enumerate(result.tokens):
                row = logits[len(prompt) - 1 + i]
                gap = float(row.max() - row[token])
                assert gap <= slack * max(1.0, float(row.std())), \
                    f"{name} {dtype} graphs={graphs}: token {i} is {token}, plain gives {int(row.argmax())} ({gap:.3g} better)"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(dtype, tmp_path):
    """``bin/trace_run`` on a folder of this architecture: steps from standard input, logits into files, slots and pages for
    four requests used again, a request left out of a step."""
    folder = cases.model_dir("Q")
    ids = {tag: _ids(folder, 700 + i, n) for i, (tag, n) in enumerate({"a": 40, "b": 9, "c": 70, "d": 3, "e": 21}.items())}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids["a"][:30], "want": [0, 29]}, {"id": "b", "tokens": ids["b"], "want": [8]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": ids["a"][30:31], "want": [0]}, {"id": "c", "tokens": ids["c"][:64], "want": []},
                                {"id": "d", "tokens": ids["d"], "want": [0, 1, 2]}, {"id": "e", "tokens": ids["e"][:2], "want": [1]}], "end": ["d"]},
        {"step": 2, "entries": [{"id": "c", "tokens": ids["c"][64:], "want": []}], "end": ["c"]},
        {"step": 3, "entries": [{"id": "a", "tokens": ids["a"][31:], "want": [8]}, {"id": "e", "tokens": ids["e"][2:], "want": [18]}],
         "end": ["a", "e"]},
    ]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                          capture_output=True, timeout=600, cwd=ROOT)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    assert not (out / "2.f32").exists()
    full = {tag: _expected(folder, seq) for tag, seq in ids.items()}
    wanted = {0: [("a", 0), ("a", 29), ("b", 8)], 1: [("a", 30), ("d", 0), ("d", 1), ("d", 2), ("e", 1)], 3: [("a", 39), ("e", 20)]}
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
    logits = plain.forward(prompt + tokens[:-1], cases.stored_weights(folder), cases.config_of(folder))
    for i, token in enumerate(tokens):
        row = logits[len(prompt) - 1 + i]
        assert float(row.max() - row[token]) <= 1e-4 * max(1.0, float(row.std())), f"token {i}"


# ------------------------------------------------------------------------------------------------ each mechanism's kernel alone
def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_clamped_gate_kernel(dtype):
    """``min(g, limit) sigmoid(1.702 .) (clamp(u) + 1)`` over interleaved pairs, with values beyond both limits."""
    from kestrel_amd.ops import core

    g = _gen(1)
    for n, m, limit in ((5, 50, 0.8), (1, 136, 2.0), (3, 7, 5.0)):
        x = (torch.randn(n, 2 * m, generator=g) * 4).to(dtype)
        out = torch.empty(n, m, dtype=dtype, device=DEV)
        core.clamped_pairs(x.to(DEV), out, limit, 1.702, 1.0)
        gate, up = x.double()[:, 0::2].clamp(max=limit), x.double()[:, 1::2].clamp(-limit, limit)
        assert torch.allclose(out.double().cpu(), gate * torch.sigmoid(1.702 * gate) * (up + 1.0), **_tol(dtype))


def test_pass_vector_kernel():
    from kestrel_amd.ops import core

    g = _gen(2)
    x = torch.randn(6, 100, generator=g)
    for dtype in DTYPES:
        vector = torch.randn(100, generator=g).to(dtype)
        got = x.clone().to(DEV)
        core.add_vector(got, vector.to(DEV))
        assert torch.allclose(got.cpu(), x + vector.float(), atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_pair_embedding_kernel(dtype):
    """Three rows of a step: one that starts its sequence, one that goes on after token 8 in slot 2, one single token; the
    state then holds every row's last token."""
    from kestrel_amd.ops import core

    g = _gen(3)
    buckets, mp, mc, dim, vocab = 13, 31, 17, 24, 50
    table = torch.randn(buckets + 1, dim, generator=g).to(dtype)
    ids = [4, 9, 9, 2, 7, 7, 30, 11]
    state = _i32([-5, 41, 8, 22, 0])
    x = torch.zeros(8, dim, device=DEV)
    core.pair_embed(table.to(DEV), _i32(ids), _i32([0, 1, 2, 3, 10, 11, 12, 5]), _i32([0, 0, 0, 0, 1, 1, 1, 2]), _i32([0, 4, 7, 8]),
                    _i32([1, 2, 3]), state, buckets, mp, mc, x, vocab)
    rows = plain.bigram_rows(ids[:4], buckets, mp, mc) + plain.bigram_rows([8] + ids[4:7], buckets, mp, mc)[1:] + \
        plain.bigram_rows([22, 11], buckets, mp, mc)[1:]
    assert torch.allclose(x.cpu(), table.float()[rows], atol=1e-6)
    assert state.tolist() == [-5, 2, 30, 11, 0]


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("taps, rot, pairing", [(3, 20, "interleaved"), (2, 8, "halves"), (5, 0, "interleaved"), (1, 12, "interleaved"),
                                                  (0, 20, "halves")])
def test_convolution_rotation_and_cache_write_kernel(taps, rot, pairing, dtype):
    """A sequence of 11 tokens in portions of 1, 4, 2 (shorter than the taps) and 4 beside another row; the state carries
    the last ``taps - 1`` inputs, places before the start count as zeros, queries and keys are rotated after the convolution,
    values are not."""
    from kestrel_amd.ops import core

    g = _gen(4)
    Hq, Hk, hd, Hv, hdv, ps = 4, 2, 20, 1, 12, 4
    channels = (Hq + Hk) * hd + Hv * hdv
    n = 11
    u = torch.randn(n, channels, generator=g).to(dtype)
    other = torch.randn(3, channels, generator=g).to(dtype)
    w = torch.randn(channels, taps, generator=g) if taps else None
    freqs = torch.tensor([0.8 ** i for i in range(rot // 2)], dtype=torch.float32) if rot else None
    state = torch.full((4, max(taps - 1, 1), channels), float("nan"), device=DEV) if taps > 1 else None
    if state is not None:
        state[[1, 3]] = 0.0                                       # (the cache manager clears a slot when a request is admitted)
    k_cache = torch.zeros(8, Hk, ps, hd, dtype=dtype, device=DEV)
    v_cache = torch.zeros(8, Hv, hdv, ps, dtype=dtype, device=DEV)
    q_rows = []
    at = 0
    for step, count in enumerate([1, 4, 2, 4]):
        rows = torch.cat([u[at:at + count], other[step:step + 1]]) if step < 3 else u[at:at + count]
        m = rows.shape[0]
        places = list(range(at, at + count)) + ([step] if step < 3 else [])
        slots = list(range(at, at + count)) + ([16 + step] if step < 3 else [])
        q_out = torch.empty(m, Hq * hd, dtype=dtype, device=DEV)
        core.conv_prepare(rows.to(DEV), None if w is None else w.to(DEV), state, _i32([0, count, m]) if step < 3 else _i32([0, count]),
                          _i32([1, 3]) if step < 3 else _i32([1]), _i32([0] * count + ([1] if step < 3 else [])), _i32(places), _i32(slots),
                          q_out, k_cache, v_cache, Hq, Hk, hd, Hv, hdv, ps, None if freqs is None else freqs.to(DEV), pairing)
        q_rows.append(q_out[:count].double().cpu())
        at += count
    y = plain.short_convolution(u.double(), w.double()) if taps else u.double()
    q, k, v = y[:, :Hq * hd].reshape(n, Hq, hd), y[:, Hq * hd:(Hq + Hk) * hd].reshape(n, Hk, hd), y[:, (Hq + Hk) * hd:].reshape(n, Hv, hdv)
    if rot:
        # frequencies 0.8^i are base^(-2 i / rot) with base = 0.8^(-rot / 2)
        turn = plain.rotate_interleaved if pairing == "interleaved" else plain.rotate_halves
        q, k = turn(q, rot, 0.8 ** (-rot / 2.0)), turn(k, rot, 0.8 ** (-rot / 2.0))
    tol = _tol(dtype)
    assert torch.allclose(torch.cat(q_rows).view(n, Hq, hd), q, **tol)
    got_k = k_cache.double().cpu().permute(0, 2, 1, 3).reshape(-1, Hk, hd)[:n]
    got_v = v_cache.double().cpu().permute(0, 3, 1, 2).reshape(-1, Hv, hdv)[:n]
    assert torch.allclose(got_k, k, **tol) and torch.allclose(got_v, v, **tol)
    if taps > 1:
        assert torch.allclose(state[1].double().cpu(), u.double()[n - taps + 1:], **tol)


def _paged(rows, ps, pages_of):
    """``rows`` ``[n, ...]`` scattered into pages ``pages_of`` (a list of page numbers): ``[pages, ps, ...]``."""
    out = torch.full((max(pages_of) + 2, ps) + tuple(rows.shape[1:]), float("nan"), dtype=rows.dtype)
    for t in range(rows.shape[0]):
        out[pages_of[t // ps], t % ps] = rows[t]
    return out


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("hd, hdv, window, kept", [(20, 12, 7, 9), (32, 64, 24, 4), (64, 32, 40, 0), (16, 48, 1, 1), (28, 36, 33, 17)])
def test_two_maps_with_a_window_that_keeps_the_first_keys_kernel(hd, hdv, window, kept, dtype):
    """Two maps per head over one value head, queries at the end of a sequence of 70 in pages that are out of order; the
    keys between the kept ones and the window lie in pages filled with NaN. Then the combination of the maps."""
    from kestrel_amd.ops import core

    g = _gen(5)
    H, G, ps, length, n = 4, 2, 16, 70, 6
    q = torch.randn(n, H, 2, hd, generator=g).to(dtype)
    k = torch.randn(length, G, 2, hd, generator=g).to(dtype)
    v = torch.randn(length, G, hdv, generator=g).to(dtype)
    pages_of = [5, 2, 7, 0, 3]
    k_pages = _paged(k.reshape(length, 2 * G, hd), ps, pages_of).permute(0, 2, 1, 3).contiguous()            # [pages, 2G, ps, hd]
    v_pages = _paged(v, ps, pages_of).permute(0, 2, 3, 1).contiguous()                                       # [pages, G, hdv, ps]
    places = [length - n + i for i in range(n)]
    lo = [max(0, p - window + 1) for p in places]
    for page in range(len(pages_of)):                                # pages no query reads: poison
        first, last = page * ps, page * ps + ps - 1
        if first >= kept and last < min(lo):
            k_pages[pages_of[page]] = float("nan")
            v_pages[pages_of[page]] = float("nan")
    maps = torch.empty(n, 2 * H * hdv, dtype=torch.float32, device=DEV)
    scale = 0.3
    core.attention_generic(q.reshape(n, -1).to(DEV), k_pages.to(DEV), v_pages.to(DEV), _i32([pages_of + [-1]]), _i32([0] * n), _i32(lo),
                           _i32([p + 1 for p in places]), maps, scale, 2 * H, 2 * G, hd, hdv, keep_first=kept, maps=2)
    seen = plain.visible(length, window, kept)[places]
    want = torch.zeros(n, H, 2, hdv, dtype=F64)
    for head in range(H):
        for which in range(2):
            scores = (q.double()[:, head, which] @ k.double()[:, head // (H // G), which].T) * scale
            want[:, head, which] = plain.softmax_weights(scores[None], seen)[0] @ v.double()[:, head // (H // G)]
    assert torch.allclose(maps.double().cpu().view(n, H, 2, hdv), want, **_tol(dtype))
    out = torch.empty(n, H * hdv, dtype=dtype, device=DEV)
    core.maps_combine(maps, out, H, hdv, 0.37, 1e-5, 0.6)
    fp = maps.double().cpu().view(n, H, 2, hdv)
    assert torch.allclose(out.double().cpu().view(n, H, hdv), plain.rms_norm(fp[:, :, 0] - 0.37 * fp[:, :, 1], None, 1e-5) * 0.6, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("rank, dr", [(40, 8), (64, 16), (8, 2), (96, 32)])
def test_attention_over_latents_with_a_sink_per_head_kernel(rank, dr, dtype):
    """Heads of queries over one cached row per key whose first ``rank`` channels are also its value, with a sink per head
    (one of them dominating, one negligible); the first query sees one key only."""
    from kestrel_amd.ops import core

    g = _gen(6)
    H, ps, length = 5, 16, 37
    rows = torch.randn(length, rank + dr, generator=g).to(dtype)
    places = [0, 1, 15, 16, 36]
    n = len(places)
    q = torch.randn(n, H, rank + dr, generator=g).to(dtype)
    sinks = torch.tensor([2.0, -1.0, 0.3, 9.0, -30.0])
    pages_of = [4, 1, 2]
    cache = _paged(rows[:, None], ps, pages_of).permute(0, 2, 1, 3).contiguous()                              # [pages, 1, ps, rank + dr]
    out = torch.empty(n, H * rank, dtype=dtype, device=DEV)
    scale = 0.2
    core.attention_generic(q.reshape(n, -1).to(DEV), cache.to(DEV), None, _i32([pages_of]), _i32([0] * n), _i32([0] * n),
                           _i32([p + 1 for p in places]), out, scale, H, 1, rank + dr, rank, sinks=sinks.to(DEV), values_in_keys=True)
    scores = torch.einsum("ihd,jd->hij", q.double(), rows.double()) * scale
    weights = plain.softmax_weights(scores, plain.visible(length)[places], sinks.double())
    want = torch.einsum("hij,jd->ihd", weights, rows.double()[:, :rank])
    assert torch.allclose(out.double().cpu().view(n, H, rank), want, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_latent_rows_kernels(dtype):
    """The query latent normalised; the key/value latent normalised and the shared key part rotated by halves into the paged
    cache; the rotated tail of every query head moved behind the latent-sized part."""
    from kestrel_amd.ops import core

    g = _gen(7)
    n, qr, rank, dr, H, d, ps, eps = 5, 36, 40, 8, 3, 24, 4, 1e-4
    down = (torch.randn(n, qr + rank + dr + 7, generator=g) * 2).to(dtype)
    gq, gk = torch.randn(qr, generator=g), torch.randn(rank, generator=g)
    freqs = torch.tensor([0.7 ** i for i in range(dr // 2)], dtype=torch.float32)
    places = [3, 4, 5, 100, 0]
    slots = [3, 4, 5, 9, 12]
    cq = torch.empty(n, qr, dtype=dtype, device=DEV)
    cache = torch.zeros(4, 1, ps, rank + dr, dtype=dtype, device=DEV)
    core.latent_prepare(down.to(DEV), 0, qr, gq.to(DEV), cq, qr, rank, gk.to(DEV), dr, freqs.to(DEV), "halves", _i32(places), _i32(slots),
                        cache, eps)
    d64 = down.double()
    tol = _tol(dtype)
    assert torch.allclose(cq.double().cpu(), plain.rms_norm(d64[:, :qr], gq.double(), eps), **tol)
    base = 0.7 ** (-dr / 2.0)
    turned = torch.zeros(101, dr, dtype=F64)
    turned[places] = d64[:, qr + rank:qr + rank + dr]
    turned = plain.rotate_halves(turned, dr, base)[places]
    got = cache.double().cpu().reshape(-1, rank + dr)[slots]
    assert torch.allclose(got[:, :rank], plain.rms_norm(d64[:, qr:qr + rank], gk.double(), eps), **tol)
    assert torch.allclose(got[:, rank:], turned, **tol)
    src = torch.randn(n, H * (d + dr), generator=g).to(dtype)
    dst = torch.zeros(n, H * (rank + dr), dtype=dtype, device=DEV)
    core.rotate_tail(src.to(DEV), dst, H, d, dr, rank, freqs.to(DEV), "halves", _i32(places))
    tails = torch.zeros(101, H, dr, dtype=F64)
    tails[places] = src.double().view(n, H, d + dr)[:, :, d:]
    tails = plain.rotate_halves(tails, dr, base)[places]
    got = dst.double().cpu().view(n, H, rank + dr)
    assert torch.allclose(got[:, :, rank:], tails, **tol) and float(got[:, :, :rank].abs().max()) == 0.0


# ------------------------------------------------------------------------------------------------ the matrix-core attention's further forms
class _Packed:
    """Rows of keys in a paged cache with shuffled pages, and the packed queries of a step over them: row ``r`` has
    ``lengths[r]`` keys, of which the last ``lengths[r] - starts[r]`` places are this step's queries. Pages that a window
    has passed and that hold no kept key are given back (the table says -1 and the page holds NaN)."""

    def __init__(self, lengths, starts, window, kept, seed):
        from types import SimpleNamespace

        self.lengths, self.starts, self.window, self.kept = lengths, starts, window, kept
        gen = torch.Generator().manual_seed(seed)
        self.gen = gen
        n_pages = sum(-(-n // 16) for n in lengths) + 3
        order = torch.randperm(n_pages, generator=gen).tolist()
        self.n_pages = n_pages
        table = torch.full((len(lengths), max(-(-n // 16) for n in lengths) + 1), -1, dtype=torch.int32)
        for r, n in enumerate(lengths):
            for p in range(-(-n // 16)):
                table[r, p] = order.pop()
        self.full_table = table.clone()
        if window is not None:
            for r, s in enumerate(starts):
                for p in range(max(0, s + 1 - window) // 16):
                    if p * 16 >= kept:
                        table[r, p] = -1
        token_row, kv_lo, kv_hi, cu_q, rows, first = [], [], [], [0], [], []
        for r, (n, s) in enumerate(zip(lengths, starts)):
            for b in range(0, n - s, 32):
                rows.append(r)
                first.append(len(token_row) + b)
            for p in range(s, n):
                token_row.append(r)
                kv_hi.append(p + 1)
                kv_lo.append(0 if window is None else max(0, p + 1 - window))
            cu_q.append(len(token_row))
        self.n = len(token_row)
        self.token_row, self.kv_hi, self.cu_q = _i32(token_row), _i32(kv_hi), _i32(cu_q)
        self.kv_lo = _i32(kv_lo) if window is not None else None
        self.table = table.to(DEV)
        from kestrel_amd.engine.batch import Workspace

        # (with a workspace at hand a decode step of few rows deals a row's keys out over several workgroups)
        self.batch = SimpleNamespace(decode_only=all(n - s == 1 for n, s in zip(lengths, starts)),
                                     query_blocks={32: (_i32(rows), _i32(first))}, cu_q=self.cu_q,
                                     workspace=Workspace(torch.device(DEV)))

    def pages(self, per_row, transposed=False):
        """``per_row[r]`` ``[length, heads, channels]`` into pages ``[pages, heads, 16, channels]`` (or ``[pages, heads, channels, 16]``);
        pages given back hold NaN."""
        heads, channels = per_row[0].shape[1:]
        out = torch.full((self.n_pages, heads, 16, channels), float("nan"), dtype=per_row[0].dtype)
        for r, rows in enumerate(per_row):
            for p in range(-(-rows.shape[0] // 16)):
                if self.table[r, p] >= 0:
                    part = rows[p * 16:(p + 1) * 16]
                    out[self.full_table[r, p], :, :part.shape[0]] = part.transpose(0, 1)
        return (out.transpose(2, 3) if transposed else out).contiguous().to(DEV)


_CUTS = {"mixed": ([70, 133, 9, 2, 101, 64, 300], [0, 100, 7, 0, 100, 63, 267]), "decode": ([70, 133, 9, 1, 300], [69, 132, 8, 0, 299])}


@pytest.mark.parametrize("cut", list(_CUTS))
@pytest.mark.parametrize("window, kept", [(24, 4), (40, 0), (7, 9), (33, 17), (64, 40), (None, 0)])
@pytest.mark.parametrize("hd, hdv", [(32, 64), (64, 32), (48, 20), (128, 128), (80, 96), (160, 192), (64, 132)])
def test_two_maps_on_the_matrix_cores(hd, hdv, window, kept, cut):
    """The bf16 kernel for prompts, portions and single tokens: two maps per head over shared values, a window that keeps
    the first keys whose other pages were given back, fp32 outputs. (The last two size pairs: the kernel's wide form, queries
    in LDS and value channels in slices of 128.)"""
    from kestrel_amd.ops import fast

    lengths, starts = _CUTS[cut]
    case = _Packed(lengths, starts, window, kept, seed=hd + hdv)
    H, G, scale = 4, 2, 1.7 / math.sqrt(hd)
    bf = torch.bfloat16
    k = [torch.randn(n, 2 * G, hd, generator=case.gen).to(bf) for n in lengths]
    v = [torch.randn(n, G, hdv, generator=case.gen).to(bf) for n in lengths]
    q = [torch.randn(n - s, 2 * H, hd, generator=case.gen).to(bf) for n, s in zip(lengths, starts)]
    out = torch.full((case.n, 2 * H * hdv), float("nan"), dtype=torch.float32, device=DEV)
    done = fast.attention_maps_bf16(torch.cat(q).reshape(case.n, -1).to(DEV), case.pages(k), case.pages(v, transposed=True), case.table,
                                    case.token_row, case.kv_lo, case.kv_hi, out, scale, 2 * H, 2 * G, hd, hdv, kept, 2, case.batch)
    assert done, "the matrix-core kernel declined sizes it is meant to take"
    want = []
    for r, (n, s) in enumerate(zip(lengths, starts)):
        seen = plain.visible(n, window, kept)[s:]
        rows = torch.zeros(n - s, 2 * H, hdv, dtype=F64)
        for head in range(2 * H):
            which, g = head % 2, head // 2 // (H // G)
            scores = (q[r].double()[:, head] @ k[r].double()[:, 2 * g + which].T) * scale
            rows[:, head] = plain.softmax_weights(scores[None], seen)[0] @ v[r].double()[:, g]
        want.append(rows.reshape(n - s, -1))
    got, want = out.double().cpu(), torch.cat(want)
    err = (got - want).abs()
    assert bool((err <= 3e-2 + 2e-2 * want.abs()).all()), f"max error {float(err.max()):.3g}"


@pytest.mark.parametrize("cut", list(_CUTS))
@pytest.mark.parametrize("heads", [5, 40])
@pytest.mark.parametrize("rank, dr", [(64, 16), (80, 16), (48, 32), (96, 32), (20, 12), (128, 32), (512, 64), (260, 28)])
def test_latents_with_sinks_on_the_matrix_cores(rank, dr, heads, cut):
    """The bf16 kernel over cached rows that are key and value at once, a sink score per head; in a decode step more heads
    than one workgroup's columns. (Rows above 128 numbers: the kernel's wide form.)"""
    from kestrel_amd.ops import fast

    lengths, starts = _CUTS[cut]
    case = _Packed(lengths, starts, None, 0, seed=rank + dr + heads)
    scale = 1.5 / math.sqrt(rank + dr)
    bf = torch.bfloat16
    rows = [torch.randn(n, 1, rank + dr, generator=case.gen).to(bf) for n in lengths]
    q = [torch.randn(n - s, heads, rank + dr, generator=case.gen).to(bf) for n, s in zip(lengths, starts)]
    sinks = torch.linspace(-4.0, 6.0, heads)
    out = torch.full((case.n, heads * rank), float("nan"), dtype=bf, device=DEV)
    done = fast.attention_latent_bf16(torch.cat(q).reshape(case.n, -1).to(DEV), case.pages(rows), case.table, case.token_row, case.kv_hi,
                                      out, scale, heads, rank + dr, rank, sinks.to(DEV), case.batch)
    assert done, "the matrix-core kernel declined sizes it is meant to take"
    want = []
    for r, (n, s) in enumerate(zip(lengths, starts)):
        c = rows[r].double()[:, 0]
        scores = torch.einsum("ihd,jd->hij", q[r].double(), c) * scale
        weights = plain.softmax_weights(scores, plain.visible(n)[s:], sinks.double())
        want.append(torch.einsum("hij,jd->ihd", weights, c[:, :rank]).reshape(n - s, -1))
    got, want = out.double().cpu(), torch.cat(want)
    err = (got - want).abs()
    assert bool((err <= 3e-2 + 2e-2 * want.abs()).all()), f"max error {float(err.max()):.3g}"


def test_the_matrix_core_kernels_run_where_sizes_allow():
    """In bf16 the model whose sizes the matrix-core kernel takes runs it for both kinds of attention (and the model of
    odd sizes runs the generic one where they do not fit)."""
    from kestrel_amd.ops import fast

    calls = []
    original = fast.attention_biased_bf16

    def spy(*args, **kwargs):
        done = original(*args, **kwargs)
        calls.append((kwargs.get("maps", 1), bool(kwargs.get("values_in_keys")), done))
        return done

    fast.attention_biased_bf16 = spy
    try:
        for name, expect in (("P", True), ("Q", False)):
            calls.clear()
            folder = cases.model_dir(name)
            runner = _runner(folder, torch.bfloat16)
            reqs = {"r": Request("r", _ids(folder, 900, 40))}
            helpers.replay(runner, reqs, [[("r", 39)], [("r", 1)]])
            assert {(m, v) for m, v, _ in calls} == {(2, False), (1, True)}
            if expect:
                assert all(done for _, _, done in calls), calls
            else:                   # (maps of 20 and 28 channels and latent rows of 34; its first latent layer's rows of 48 the kernel takes)
                assert not any(done for m, _, done in calls if m == 2) and (1, True, False) in calls, calls
    finally:
        fast.attention_biased_bf16 = original


@pytest.mark.parametrize("n", [1, 8, 70, 300])
@pytest.mark.parametrize("heads, a_head, k, out_head, n_out", [(5, 72, 64, 88, 80), (3, 32, 32, 40, 40), (16, 96, 96, 64, 64),
                                                                 (2, 144, 128, 20, 20), (7, 16, 16, 8, 6)])
def test_a_linear_per_head_on_the_matrix_cores(heads, a_head, k, out_head, n_out, n):
    """Every head's own matrix in one launch: heads that read the first ``k`` channels of their part of a row and write the
    first ``n_out`` of theirs; what lies behind is left as it was."""
    from kestrel_amd.ops import fast

    g = _gen(8)
    bf = torch.bfloat16
    a = torch.randn(n, heads * a_head + 8, generator=g).to(bf)
    w = (torch.randn(heads, n_out, k, generator=g) / math.sqrt(k)).to(bf)
    out = torch.full((n, heads * out_head), 7.0, dtype=bf, device=DEV)
    assert fast.heads_linear_bf16(a.to(DEV)[:, :heads * a_head], a_head, k, w.to(DEV), out, out_head, n_out)
    got = out.double().cpu().view(n, heads, out_head)
    want = torch.einsum("nhk,hok->nho", a[:, :heads * a_head].double().view(n, heads, a_head)[:, :, :k], w.double())
    assert torch.allclose(got[:, :, :n_out], want, rtol=2e-2, atol=2e-2)
    assert bool((got[:, :, n_out:] == 7.0).all())
    # with a gate in a buffer of wider rows: times its sigmoid
    gate = (torch.randn(n, heads * out_head + 24, generator=g) * 2).to(bf)
    assert fast.heads_linear_bf16(a.to(DEV)[:, :heads * a_head], a_head, k, w.to(DEV), out, out_head, n_out, gate.to(DEV)[:, 24:])
    got = out.double().cpu().view(n, heads, out_head)
    want = want * torch.sigmoid(gate[:, 24:].double().view(n, heads, out_head)[:, :, :n_out])
    assert torch.allclose(got[:, :, :n_out], want, rtol=2e-2, atol=2e-2)
