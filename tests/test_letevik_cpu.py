"""Letevik on the host: its configuration reader, its plan, its caches and state, and the plain implementation's mechanisms."""

import copy
import math

import pytest
import torch

from kestrel_amd.cache.manager import CacheManager
from kestrel_amd.config.registry import read_model_dir, resolve
from kestrel_amd.models.decoder import DecoderModel
from kestrel_amd.models.letevik import LetevikConfig, build_plan
from kestrel_amd.parts.specs import CacheSpec
from tests import letevik_cases as cases
from tests.plain import letevik_plain as plain

F64 = torch.float64


def test_config_names_the_architecture_and_round_trips():
    for name, config in cases.CONFIGS.items():
        assert resolve(config).name == "letevik"
        typed = LetevikConfig.from_dict(config)
        again = LetevikConfig.from_dict(typed.to_dict())
        assert again.layers == typed.layers and (again.loop_start, again.loop_stop, again.loop_times) == \
            (typed.loop_start, typed.loop_stop, typed.loop_times), name


def test_tensor_names_and_shapes():
    params = DecoderModel(build_plan(LetevikConfig.from_dict(cases.CONFIGS["Q"]))).params()
    assert tuple(params["embed"].shape) == (211, 100) and tuple(params["bigram"].shape) == (54, 100)
    assert tuple(params["loop.step"].shape) == (3, 100) and tuple(params["final.norm"].shape) == (100,)
    assert "head" not in params                                                 # the head is the embedding table
    assert tuple(params["l0.mix.dq"].shape) == (36, 100) and tuple(params["l0.mix.dq.norm"].shape) == (36,)
    assert tuple(params["l0.mix.uq"].shape) == (5 * (24 + 8), 36) and tuple(params["l0.mix.dkv"].shape) == (40 + 8, 100)
    assert tuple(params["l0.mix.dkv.norm"].shape) == (40,) and tuple(params["l0.mix.uk"].shape) == (5 * 24, 40)
    assert tuple(params["l0.mix.uv"].shape) == (5 * 10, 40) and tuple(params["l0.mix.sink"].shape) == (5,)
    assert tuple(params["l0.mix.g"].shape) == (50, 100) and tuple(params["l0.mix.o"].shape) == (100, 50)
    assert "l0.mlp.gate" not in params and "l0.norm2" not in params
    assert tuple(params["l1.mix.q"].shape) == (6 * 2 * 20, 100) and tuple(params["l1.mix.k"].shape) == (3 * 2 * 20, 100)
    assert tuple(params["l1.mix.v"].shape) == (3 * 12, 100) and tuple(params["l1.mix.o"].shape) == (100, 6 * 12)
    assert tuple(params["l1.mix.q.conv"].shape) == (240, 2) and tuple(params["l1.mix.v.conv"].shape) == (36, 2)
    assert all(tuple(params[f"l1.mix.{n}"].shape) == (20,) for n in ("lq1", "lk1", "lq2", "lk2"))
    assert tuple(params["l1.mlp.gate"].shape) == (50, 100) and tuple(params["l1.mlp.down"].shape) == (100, 50)
    no_conv = DecoderModel(build_plan(LetevikConfig.from_dict(cases.CONFIGS["R"]))).params()
    assert "l0.mix.q.conv" in no_conv and "l1.mix.q.conv" not in no_conv and "loop.step" not in no_conv


def test_the_order_of_layers_and_the_passes_of_the_loop():
    for name, config in cases.CONFIGS.items():
        plan = build_plan(LetevikConfig.from_dict(config))
        want = plain.layer_order(config)
        assert [e.layer for e in plan.schedule] == [i for i, _ in want], name
        assert [(e.before is not None, e.passage if e.before else None) for e in plan.schedule] == \
            [(t is not None, t) for _, t in want], name
    # a loop that runs zero times leaves its layers out, an empty stretch leaves the vector out
    config = copy.deepcopy(cases.CONFIGS["Q"])
    config["loop"] = {"start": 1, "stop": 3, "times": 0}
    assert [e.layer for e in build_plan(LetevikConfig.from_dict(config)).schedule] == [0, 3]
    config["loop"] = {"start": 2, "stop": 2, "times": 4}
    plan = build_plan(LetevikConfig.from_dict(config))
    assert [e.layer for e in plan.schedule] == [0, 1, 2, 3] and not plan.junctions


def test_caches_and_state_by_layer():
    net = DecoderModel(build_plan(LetevikConfig.from_dict(cases.CONFIGS["P"])))
    needs = net.cache_needs()
    # 2 passes x (differential, latent), then differential and latent, then the pair embedding's state
    assert len(needs) == 7 and needs[-1][0] is None and needs[-1][1].dtype == "int32"
    assert [getattr(n[0], "window", None) for n in needs[:6]] == [24, None, 24, None, 40, None]
    assert [getattr(n[0], "keep_first", 0) for n in needs[:6]] == [4, 0, 4, 0, 0, 0]
    # the convolution's state: taps - 1 rows of q | k | v
    assert needs[0][1].shape == (2, 4 * 2 * 32 + 2 * 2 * 32 + 2 * 64) and needs[4][1].shape == (3, 2 * 2 * 64 + 2 * 2 * 64 + 2 * 32)
    assert needs[1][1] is None and needs[1][0].page_tensors(16) == {"k": (1, 16, 64 + 16)}
    # one tap and no convolution keep nothing
    other = DecoderModel(build_plan(LetevikConfig.from_dict(cases.CONFIGS["R"]))).cache_needs()
    assert other[0][1] is None and other[1][1] is None
    cache = CacheManager(needs, page_size=16, n_pages=8, max_requests=2)
    assert cache.free_slots == 2


def test_pages_of_kept_keys_stay_and_the_others_go_back():
    spec = CacheSpec(2, 8, 24, 8, keep_first=20)
    assert [spec.first_visible(p) for p in (0, 23, 24, 100)] == [0, 0, 1, 77]
    cache = CacheManager([(spec, None, None)], page_size=16, n_pages=6, max_requests=1)
    slot = cache.admit()
    held = []
    for length in range(1, 260):
        cache.ensure(slot, length)
        cache.trim(slot, length)
        cache.check()
        table = cache.block_table(0, slot)
        # every key the next query reads is still backed: the window's and the kept ones
        assert all(table[p // 16] >= 0 for p in range(spec.first_visible(length), length))
        assert all(table[p // 16] >= 0 for p in range(min(20, length)))
        held.append(sum(p >= 0 for p in table))
    assert max(held) <= 2 + 3 and held[-1] < 6
    cache.release(slot)
    assert cache.pages_available(0) == 6
    assert cache.pages_for(0, 1000, portion=1) <= 5


@pytest.mark.parametrize("bad, message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "dense"),
    (lambda c: c["layers"][0]["mlp"].update(limit=0), "limit"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=33), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=34), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["embedding"]["bigram"].pop("mul_cur"), "mul_cur"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_config_errors_name_the_key(bad, message):
    config = copy.deepcopy(cases.CONFIGS["P"])
    bad(config)
    with pytest.raises(ValueError, match=message):
        LetevikConfig.from_dict(config)


def test_model_folder_is_read_through_the_registry():
    spec, typed, plan = read_model_dir(cases.model_dir("S"))
    assert spec.name == "letevik" and plan.dim == 48 and len(plan.schedule) == 2 and plan.tied_head


# ------------------------------------------------------------------------------------------------ the plain implementation itself
def test_pair_rows_of_the_plain_implementation():
    assert plain.bigram_rows([5, 9, 9, 2], 11, 3, 4) == [11, (15 + 36) % 11, (27 + 36) % 11, (27 + 8) % 11]
    assert plain.bigram_rows([7], 1, 3, 5) == [1] and plain.bigram_rows([7, 8], 1, 3, 5) == [1, 0]


def test_short_convolution_of_the_plain_implementation():
    gen = torch.Generator().manual_seed(1)
    u, taps = torch.randn(9, 3, generator=gen, dtype=F64), torch.randn(3, 4, generator=gen, dtype=F64)
    y = plain.short_convolution(u, taps)
    for t in range(9):
        want = sum(taps[:, j] * u[t - 3 + j] for j in range(4) if t - 3 + j >= 0)
        assert torch.allclose(y[t], want, atol=1e-12)
    # the last tap weighs the token itself; one tap is a scaling
    assert torch.allclose(plain.short_convolution(u, taps[:, 3:]), u * taps[:, 3], atol=1e-12)
    # a sequence shorter than the taps
    assert torch.allclose(plain.short_convolution(u[:2], taps)[1], taps[:, 3] * u[1] + taps[:, 2] * u[0], atol=1e-12)


def test_rotations_of_the_plain_implementation():
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(6, 2, 10, generator=gen, dtype=F64)
    a = plain.rotate_interleaved(x, 6, 100.0)
    b = plain.rotate_halves(x, 6, 100.0)
    assert torch.equal(a[..., 6:], x[..., 6:]) and torch.equal(b[..., 6:], x[..., 6:]) and torch.equal(a[0], x[0])
    for i in range(3):
        angle = 5 * 100.0 ** (-2.0 * i / 6)
        u, v = x[5, 1, 2 * i], x[5, 1, 2 * i + 1]
        assert math.isclose(float(a[5, 1, 2 * i]), float(u * math.cos(angle) - v * math.sin(angle)), abs_tol=1e-12)
        assert math.isclose(float(a[5, 1, 2 * i + 1]), float(v * math.cos(angle) + u * math.sin(angle)), abs_tol=1e-12)
        u, v = x[5, 1, i], x[5, 1, i + 3]
        assert math.isclose(float(b[5, 1, i]), float(u * math.cos(angle) - v * math.sin(angle)), abs_tol=1e-12)
        assert math.isclose(float(b[5, 1, i + 3]), float(v * math.cos(angle) + u * math.sin(angle)), abs_tol=1e-12)
    # a rotation keeps a score a function of the distance
    q, k = torch.randn(1, 1, 8, generator=gen, dtype=F64), torch.randn(1, 1, 8, generator=gen, dtype=F64)
    rows = [plain.rotate_halves(t.expand(40, 1, 8).clone(), 8, 50.0) for t in (q, k)]
    assert math.isclose(float(rows[0][30, 0] @ rows[1][10, 0]), float(rows[0][25, 0] @ rows[1][5, 0]), abs_tol=1e-10)


def test_window_with_kept_first_keys_of_the_plain_implementation():
    seen = plain.visible(12, 4, 2)
    assert seen[3].tolist() == [True] * 4 + [False] * 8
    assert seen[9].tolist() == [True, True] + [False] * 4 + [True] * 4 + [False, False]
    assert plain.visible(5).tolist() == torch.tril(torch.ones(5, 5, dtype=torch.bool)).tolist()
    assert plain.visible(6, 1, 1)[4].tolist() == [True, False, False, False, True, False]


def test_sink_of_the_plain_implementation_counts_once_and_unscaled():
    scores = torch.tensor([[[0.3, -0.2, 1.1]]], dtype=F64)
    seen = torch.ones(1, 3, dtype=torch.bool)
    sink = torch.tensor([0.7], dtype=F64)
    w = plain.softmax_weights(scores, seen, sink)
    total = math.exp(0.3) + math.exp(-0.2) + math.exp(1.1) + math.exp(0.7)
    assert torch.allclose(w[0, 0], torch.tensor([math.exp(0.3), math.exp(-0.2), math.exp(1.1)], dtype=F64) / total, atol=1e-12)
    assert float(w.sum()) < 1.0
    # a very large sink takes all the weight: nothing overflows
    assert float(plain.softmax_weights(scores, seen, torch.tensor([800.0], dtype=F64)).sum()) < 1e-300


def test_feed_forward_of_the_plain_implementation_clamps_before_the_product():
    w = {"gate": torch.tensor([[10.0], [-10.0], [0.5]], dtype=F64), "up": torch.tensor([[10.0], [-10.0], [0.5]], dtype=F64),
         "down": torch.eye(3, dtype=F64)}
    y = plain.feed_forward(torch.tensor([[1.0]], dtype=F64), w, "", {"kind": "dense", "ff": 3, "limit": 2.0})
    sig = lambda z: 1.0 / (1.0 + math.exp(-z))
    want = [2.0 * sig(1.702 * 2.0) * 3.0, -10.0 * sig(-17.02) * (-2.0 + 1.0), 0.5 * sig(0.851) * 1.5]
    assert torch.allclose(y[0], torch.tensor(want, dtype=F64), atol=1e-12)


def test_differential_attention_of_the_plain_implementation_is_two_maps_of_one_value():
    """With equal weights for both maps and lambda = 1 the head's output vanishes before the norm; the norm has no gain and
    the factor behind it is 1 - diff."""
    gen = torch.Generator().manual_seed(4)
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 6, "scale": 0.5, "diff": 0.25, "rot": {"base": 10.0, "dims": 4}}
    width, n = 8, 7
    w = {"q": torch.randn(16, width, generator=gen, dtype=F64), "k": torch.randn(8, width, generator=gen, dtype=F64),
         "v": torch.randn(6, width, generator=gen, dtype=F64), "o": torch.eye(12, dtype=F64)}
    for name in ("lq1", "lk1", "lq2", "lk2"):
        w[name] = torch.zeros(4, dtype=F64)                      # lambda = exp(0) - exp(0) + diff = diff
    h = torch.randn(n, width, generator=gen, dtype=F64)
    out = plain.differential_attention(h, w, "", m, 1e-9).view(n, 2, 6)
    assert torch.allclose(out.pow(2).mean(dim=-1).sqrt(), torch.full((n, 2), 0.75, dtype=F64), atol=1e-6)
    # the first token sees itself alone: both maps give its value, o = (1 - lambda) v
    v0 = h[0] @ w["v"].T
    assert torch.allclose(out[0, 0], plain.rms_norm(0.75 * v0, None, 1e-9) * 0.75, atol=1e-9)
