"""Bokorax on the host: the configuration reader, the plan, what the cache manager makes of it, and the plain
implementation's functions on cases worked out by hand."""

import json
import math

import pytest
import torch

from kestrel_amd.cache.manager import CacheManager
from kestrel_amd.config.registry import resolve
from kestrel_amd.models import bokorax
from kestrel_amd.models.decoder import DecoderModel
from kestrel_amd.parts.rotary import rotary_frequencies
from kestrel_amd.parts.specs import LinearScaling
from tests import bokorax_cases as cases
from tests import helpers
from tests.plain import bokorax_plain as plain

F64 = torch.float64


def _plan(name):
    config = cases.CONFIGS[name]
    spec = resolve(config)
    assert spec.name == "bokorax"
    return spec.build_plan(spec.read_config(config))


def test_the_configuration_survives_a_round_trip():
    for name, config in cases.CONFIGS.items():
        typed = bokorax.BokoraxConfig.from_dict(config)
        assert typed.to_dict() == config, name


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "no multiple"),
    (lambda c: c["layers"][0].update(type="conv"), "this design has the mixers"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "no earlier attention_2 layer"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "no earlier attention_2 layer"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=32), "sizes differ"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=32), "the values are the keys"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even and at most dim"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "exceeds"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3), "must divide"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind 'moe'"),
    (lambda c: c["layers"][0]["mixer"].update(softcap=0), "softcap must be positive"),
    (lambda c: c.pop("norm"), "'norm' missing"),
])
def test_what_the_configuration_reader_refuses(edit, message):
    config = json.loads(json.dumps(cases.CONFIGS["P"]))
    edit(config)
    with pytest.raises(ValueError, match=message):
        bokorax.BokoraxConfig.from_dict(config)


def test_tensor_names_and_shapes():
    params = DecoderModel(_plan("P")).params()
    assert params["embed"].shape == (300, 128) and params["head"].shape == (300, 128) and params["final.norm"].shape == (128,)
    # a capped layer with keys and values of its own
    assert params["l0.mix.q"].shape == (128, 128) and params["l0.mix.k"].shape == (64, 128) and params["l0.mix.v"].shape == (128, 128)
    assert params["l0.mix.q.norm"].shape == (32,) and params["l0.mix.k.norm"].shape == (32,) and params["l0.mix.sink"].shape == (4,)
    assert params["l0.mix.g"].shape == (4, 128) and params["l0.mix.o"].shape == (128, 256)
    # the layer that reads its keys and values has none of their tensors
    assert "l3.mix.k" not in params and "l3.mix.v" not in params and "l3.mix.k.norm" not in params and params["l3.mix.q"].shape == (128, 128)
    # values that are the keys: no value projection, gains of the whole projection
    assert "l2.mix.v" not in params and params["l2.mix.q.norm"].shape == (256,) and params["l2.mix.k.norm"].shape == (64,)
    assert "l2.mix.g" not in params and "l2.mix.sink" not in params
    # the memory
    assert params["l1.mix.mu.w"].shape == (128,) and params["l1.mix.w1"].shape == (8, 128) and params["l1.mix.w2"].shape == (128, 8)
    assert params["l1.mix.u"].shape == (4, 32) and params["l1.mix.w0"].shape == (128,) and params["l1.mix.norm"].shape == (128,)
    # experts: identity experts have router rows and no tensors
    assert params["l0.mlp.router"].shape == (8, 128) and params["l0.mlp.correction"].shape == (8,) and "l0.mlp.e6.gate" not in params
    assert params["l0.mlp.e5.down"].shape == (128, 64) and params["l0.mlp.shared.sg"].shape == (1, 128)
    assert "l3.mlp.shared.gate" not in params and params["l2.mlp.shared.up"].shape == (64, 128)
    # the rank of the decay is left to the weights file where the configuration does not name it
    config = json.loads(json.dumps(cases.CONFIGS["P"]))
    config["layers"][1]["mixer"].pop("decay_rank")
    loose = DecoderModel(resolve(config).build_plan(bokorax.BokoraxConfig.from_dict(config))).params()
    assert loose["l1.mix.w1"].shape == (-1, 128) and loose["l1.mix.w2"].shape == (128, -1)


def test_schedule_cache_groups_and_state():
    plan = _plan("R")
    assert [e.reads_cache_of for e in plan.schedule] == [None, 0, None, None, 0]
    assert plan.embedding_scale == 2.0 and plan.logit_scale == 1.0 and all(layer.arrangement == "output_norms" for layer in plan.layers)
    model = DecoderModel(plan)
    needs = model.cache_needs()
    assert needs[2][0] is None and needs[2][1].shape == (2 * 128 * 128 + 256,) and needs[2][1].dtype == "float32"
    manager = CacheManager(needs, 16, 40, 3)
    assert len(manager.groups) == 2                                    # the capped layers share one, the windowed layer has its own
    caches = manager.layer_caches()
    assert caches[0].writes and not caches[1].writes and not caches[4].writes and caches[1].group == caches[0].group == caches[4].group
    assert caches[3].group != caches[0].group and caches[2].group is None


def test_a_window_gives_its_pages_back():
    manager = CacheManager(DecoderModel(_plan("P")).cache_needs(), 16, 30, 2)
    windowed = [g for g, group in enumerate(manager.groups) if group.spec.window == 40][0]
    full = 1 - windowed
    slot = manager.admit()
    manager.ensure(slot, 100)
    manager.trim(slot, 100)
    # the next query, at place 100, reads the keys 61 .. 100: pages 0 to 2 are behind it
    assert manager.block_table(windowed, slot)[:4] == [-1, -1, -1, manager.block_table(windowed, slot)[3]] and manager.block_table(windowed, slot)[3] >= 0
    assert all(p >= 0 for p in manager.block_table(full, slot))
    manager.release(slot)
    manager.check()


def test_frequencies_of_the_product_against_the_plain_ones():
    for rot in ({"dims": 16, "base": 10000.0, "scaling": {"factor": 2.0}}, {"dims": 64, "base": 500000.0, "scaling": {"factor": 4.0}},
                {"dims": 2, "base": 3.0}):
        scaling = LinearScaling(rot["scaling"]["factor"]) if "scaling" in rot else None
        assert rotary_frequencies(rot["dims"], rot["base"], scaling) == pytest.approx(plain.frequencies(rot), rel=1e-15)


# ---------------------------------------------------------------------------------------------- the plain functions themselves
def test_plain_norm_and_rotation_by_hand():
    y = torch.tensor([[3.0, 4.0]], dtype=F64)
    assert plain.norm_one_plus(y, torch.tensor([0.0, 1.0], dtype=F64), 0.0).tolist() == [[3 / math.sqrt(12.5), 2 * 4 / math.sqrt(12.5)]]
    x = torch.tensor([[[1.0, 2.0, 0.0, 0.0, 9.0]]], dtype=F64).repeat(2, 1, 1)        # channels 0, 1 pair with 2, 3; channel 4 stays
    out = plain.rotate_halves(x, [0, 1], [math.pi / 2, math.pi])
    assert out[0].tolist() == [[1.0, 2.0, 0.0, 0.0, 9.0]]
    assert out[1, 0].tolist() == pytest.approx([0.0, -2.0, 1.0, 0.0, 9.0], abs=1e-12)


def test_plain_window_and_softmax_with_a_sink():
    seen = plain.window_mask(5, 2)
    assert seen.tolist() == [[j in (i - 1, i) and j >= 0 for j in range(5)] for i in range(5)]
    w = plain.softmax_weights(torch.zeros(1, 3, dtype=F64), torch.tensor([[True, True, False]]), sink=math.log(2.0))
    assert w.tolist() == [[0.25, 0.25, 0.0]]                              # the sink counts once, with its own score, and has no value
    w = plain.softmax_weights(torch.tensor([[0.0, 1.0]], dtype=F64), torch.tensor([[True, True]]))
    assert float(w.sum()) == pytest.approx(1.0)


def test_plain_capped_scores_and_grouped_heads():
    q = torch.tensor([[[10.0], [0.0]]], dtype=F64)                        # one token, two heads of one channel, one kv head
    k, v = torch.tensor([[[1.0]]], dtype=F64), torch.tensor([[[5.0]]], dtype=F64)
    seen = torch.tensor([[True]])
    out = plain.grouped_attention(q, k, v, 1.0, seen, softcap=2.0, sinks=torch.tensor([2.0 * math.tanh(5.0), 0.0], dtype=F64))
    # head 0: the capped score 2 tanh(5) equals its sink: half of the value; head 1: score 0 = sink 0: half as well
    assert out.reshape(-1).tolist() == pytest.approx([2.5, 2.5])


def test_plain_token_shift_and_the_recurrence_cut_in_pieces():
    h = torch.tensor([[1.0, 2.0], [3.0, 6.0], [5.0, 0.0]], dtype=F64)
    mu = torch.tensor([0.0, 0.5], dtype=F64)
    assert plain.token_shift(h, mu).tolist() == [[1.0, 1.0], [3.0, 4.0], [5.0, 3.0]]
    assert plain.token_shift(h[1:], mu, before=h[0]).tolist() == [[3.0, 4.0], [5.0, 3.0]]
    gen = torch.Generator().manual_seed(0)
    r, k, decay = (torch.rand(9, 4, generator=gen, dtype=F64) for _ in range(3))
    v = torch.randn(9, 3, generator=gen, dtype=F64)
    u = torch.randn(4, generator=gen, dtype=F64)
    whole, state = plain.wkv_recurrence(r, k, v, decay, u)
    first, mid = plain.wkv_recurrence(r[:4], k[:4], v[:4], decay[:4], u)
    second, end = plain.wkv_recurrence(r[4:], k[4:], v[4:], decay[4:], u, mid)
    assert torch.allclose(torch.cat([first, second]), whole, atol=1e-14) and torch.allclose(end, state, atol=1e-14)
    # by hand: the first token reads only its own key through the bonus
    assert torch.allclose(whole[0], (r[0] * u * k[0]).sum() * v[0], atol=1e-14)
    assert torch.allclose(whole[1], ((r[1] * k[0]).sum()) * v[0] + (r[1] * u * k[1]).sum() * v[1], atol=1e-14)


def test_plain_router_by_hand():
    logits = torch.log(torch.tensor([[0.4, 0.1, 0.05, 0.05, 0.3, 0.1]], dtype=F64))
    pick = lambda r, c=None: plain.route(logits, torch.eye(6, dtype=F64), torch.zeros(6, dtype=F64) if c is None else c, r)
    chosen, weights = pick({"top": 2, "scale": 2.0})
    assert chosen.tolist() == [[0, 4]] and weights.tolist() == [pytest.approx([2 * 0.4 / 0.7, 2 * 0.3 / 0.7])]
    # three groups of two, one kept: group 0 wins (0.4), so the second choice comes from it too
    chosen, weights = pick({"top": 2, "groups": {"count": 3, "keep": 1}})
    assert sorted(chosen[0].tolist()) == [0, 1] and float(weights.sum()) == pytest.approx(1.0)
    # the correction moves the choice but not the weights; choice scores below zero still beat a group that is not kept
    correction = torch.tensor([-5.0, -5.0, -1.0, -1.0, -5.0, -5.0], dtype=F64)
    chosen, weights = pick({"top": 2, "groups": {"count": 3, "keep": 1}}, correction)
    assert sorted(chosen[0].tolist()) == [2, 3] and weights[0].tolist() == pytest.approx([0.5, 0.5])


def test_plain_identity_and_shared_experts():
    h = torch.tensor([[1.0, -2.0]], dtype=F64)
    w = {"m.router": torch.tensor([[0.0, 0.0], [9.0, 0.0]], dtype=F64), "m.correction": torch.zeros(2, dtype=F64),
         "m.e0.gate": torch.ones(1, 2, dtype=F64), "m.e0.up": torch.ones(1, 2, dtype=F64), "m.e0.down": torch.ones(2, 1, dtype=F64),
         "m.shared.gate": torch.zeros(1, 2, dtype=F64), "m.shared.up": torch.ones(1, 2, dtype=F64), "m.shared.down": torch.ones(2, 1, dtype=F64),
         "m.shared.sg": torch.zeros(1, 2, dtype=F64)}
    mlp = {"router": {"experts": 1, "identity": 1, "top": 1, "scale": 3.0}, "shared": {"ff": 1}}
    # the router prefers its second output, the identity expert: three times the input; the shared expert's gate is silu(0) = 0
    assert plain.routed_experts(h, w, "m.", mlp).tolist() == [[3.0, -6.0]]


def test_what_a_lost_mechanism_would_cost():
    """On the crafted folder the plain implementation itself says what the model-level tests can see: without the sinks,
    without the cap, without the bonus, without the identity experts, with a window that is one token longer or shorter, or
    with a far key lost, the logits move by more than the bounds of the model-level tests allow (1e-4 of a row's spread in
    float32, 4 % in bfloat16)."""
    base = cases.model_dir("P")
    folder = cases.crafted(base)
    config, weights = cases.config_of(folder), cases.stored_weights(folder)
    window = config["layers"][2]["mixer"]["mask"]["size"]
    length = 3 * window + 20
    at = length - 7

    def ids_with(distance):
        ids = list(range(10, 10 + length))
        ids[at] = cases.CALL
        if distance is not None:
            ids[at - distance] = cases.ECHO
        return ids

    def moved(a, b):
        d = a - b
        d = d - d.mean(dim=-1, keepdim=True)
        return float((d.pow(2).mean(dim=-1).sqrt() / a.std(dim=-1)).max())

    ids = ids_with(window - 1)
    want = plain.forward(config, weights, ids)
    no_sink = {k: (torch.full_like(v, -30.0) if k.endswith(".sink") else v) for k, v in weights.items()}
    assert moved(want, plain.forward(config, no_sink, ids)) > 0.05
    no_cap = json.loads(json.dumps(config))
    for layer in no_cap["layers"]:
        layer["mixer"].pop("softcap", None)
    assert moved(want, plain.forward(no_cap, weights, ids)) > 0.05
    no_bonus = {k: (torch.zeros_like(v) if k.endswith(".u") else v) for k, v in weights.items()}
    assert moved(want, plain.forward(config, no_bonus, ids)) > 0.05
    no_identity = {k: (torch.cat([v[:-2], torch.full_like(v[-2:], -9.0)]) if k.endswith("l0.mlp.correction") else v) for k, v in weights.items()}
    assert moved(want, plain.forward(config, no_identity, ids)) > 0.05
    # the window's edge, from either side, at the token that calls
    for size, distance in ((window + 1, window), (window - 1, window - 1)):
        other = json.loads(json.dumps(config))
        other["layers"][2]["mixer"]["mask"]["size"] = size
        ids = ids_with(distance)
        assert moved(plain.forward(config, weights, ids)[at], plain.forward(other, weights, ids)[at]) > 0.05
    # a far key, and the very first token, seen or not
    for distance in (2 * window + 5, at):
        assert moved(plain.forward(config, weights, ids_with(distance))[at], plain.forward(config, weights, ids_with(None))[at]) > 0.05
