"""Small Bokorax configurations for the tests, their model folders and crafted variants."""

from __future__ import annotations

import functools
import tempfile
from typing import Dict, Optional

import torch

from kestrel_amd.weights import InitRecipe, write_random_model
from tests.bogivik_cases import config_of, rewrite, stored_weights  # noqa: F401  (folders are read and edited the same way)


def experts(n, ff, top, scale=1.0, identity=0, groups=None, shared=None):
    router = {"experts": n, "top": top, "scale": scale, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def attention(heads, kv_heads, dim, scale, rot_dims, base, window, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": {"base": base, "dims": rot_dims}}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def attention_2(heads, kv_heads, dim, vdim, scale, rot_dims, base, factor=None, softcap=None, kv_from: Optional[int] = None, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if softcap is not None:
        mixer["softcap"] = softcap
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention_2", "mixer": mixer, "mlp": mlp}


def wkv(heads, dim, rank, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}, "mlp": mlp}


def _config(vocab, width, eps, layers, embedding_scale=1.0, logit_scale=1.0):
    return {"architecture": "Bokorax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embedding_scale},
            "logit_scale": logit_scale, "layers": layers}


CONFIGS: Dict[str, dict] = {
    # sizes the matrix-core kernels take; a capped layer first whose keys a later layer reads; a window of two and a half pages
    "P": _config(300, 128, 1e-5, [
        attention_2(4, 2, 32, 64, 0.2, 16, 10000.0, 2.0, 30.0, None, experts(6, 64, 3, 1.5, 2, (4, 2), 32)),
        wkv(4, 32, 8, experts(6, 64, 3, 1.5, 2, (4, 2), 32)),
        attention(4, 1, 64, 0.15, 32, 500.0, 40, experts(4, 48, 2, 2.0, 0, None, 64)),
        attention_2(4, 2, 32, 64, 0.25, 16, 10000.0, 2.0, 20.0, 0, experts(6, 64, 3, 1.5, 2, (4, 2), None)),
    ], embedding_scale=0.7, logit_scale=0.5),
    # sizes that fit none of the fast kernels' alignments: a window shorter than a page, fewer rotated channels than a head has,
    # no scaling of frequencies, no cap, as many kv heads as heads, one choice among experts without identity experts or groups,
    # layers without a feed-forward, no shared expert
    "Q": _config(211, 100, 1e-6, [
        wkv(5, 20, 6, None),
        attention(6, 3, 24, 0.3, 12, 50.0, 7, experts(5, 24, 1)),
        attention_2(3, 3, 20, 12, 0.25, 20, 300.0, None, None, None, experts(3, 40, 2, 0.5, 3, (3, 2), 20)),
        attention_2(6, 3, 20, 12, 0.4, 20, 300.0, None, 5.0, 2, None),
        wkv(2, 44, 3, experts(5, 24, 1)),
    ]),
    # the largest head sizes; one kv head; a window of whole pages; every channel rotated; two layers that read the same keys;
    # many experts in five groups of which two are kept
    "R": _config(190, 256, 1e-3, [
        attention_2(2, 1, 128, 128, 0.09, 128, 1e6, 8.0, 50.0, None, experts(16, 144, 4, 2.5, 4, (5, 2), 80)),
        attention_2(4, 1, 128, 128, 0.07, 128, 1e6, 8.0, 15.0, 0, None),
        wkv(2, 128, 32, experts(16, 144, 4, 2.5, 4, (5, 2), 80)),
        attention(2, 2, 128, 0.1, 128, 1e4, 64, experts(8, 80, 2, 1.0, 0, (2, 1), 144)),
        attention_2(2, 1, 128, 128, 0.09, 128, 1e6, 8.0, 50.0, 0, None),
    ], embedding_scale=2.0),
    # one head everywhere, a window of one key, one expert and one identity expert that are both always chosen, one group
    "S": _config(77, 48, 1e-5, [
        attention(1, 1, 16, 0.5, 2, 3.0, 1, experts(1, 40, 2, 1.0, 1, (1, 1), 8)),
        wkv(1, 48, 1, experts(1, 40, 1, 3.0, 0)),
        attention_2(1, 1, 16, 16, 0.3, 16, 30.0, 1.0, 1.0, None, experts(2, 16, 1, 1.0, 1, (3, 1), None)),
    ], logit_scale=2.0),
}
RECIPE = InitRecipe(std=0.08, bias_std=0.5, gain_std=0.2, shift_std=0.2)
SEEDS = {"P": 31, "Q": 32, "R": 33, "S": 34}


@functools.lru_cache(maxsize=None)
def model_dir(name: str) -> str:
    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_bokorax{name}_")
    write_random_model(folder, CONFIGS[name], SEEDS[name], RECIPE, store_dtype="bfloat16")
    return folder


@functools.lru_cache(maxsize=None)
def steady(base: str) -> str:
    """A variant of a folder whose routers always choose the same experts: corrections three units apart, which no score
    (a number between 0 and 1) can bridge. The weights of the chosen experts still follow the scores. For runs in bfloat16:
    a router's choice is a step function of its scores, and where two choice scores lie closer than rounding moves them the
    step falls either way: with corrections drawn at random that happens to a few tokens of every sequence, and the row
    then differs from the plain implementation by an expert, not by rounding."""
    def edit(weights):
        for name in [k for k in weights if k.endswith(".mlp.correction")]:
            count = weights[name].numel()
            order = torch.randperm(count, generator=torch.Generator().manual_seed(count + len(name) + int(name[1:name.index(".")])))
            weights[name] = (3.0 * order.float()).to(weights[name].dtype)

    return rewrite(base, edit)


def folder_for(name: str, dtype) -> str:
    """The model folder a run in ``dtype`` is tested on: as written for float32, with steady routers for bfloat16."""
    folder = model_dir(name)
    return steady(folder) if dtype in (torch.bfloat16, "bfloat16") else folder


CALL, ECHO = 5, 6


@functools.lru_cache(maxsize=None)
def crafted(base: str) -> str:
    """A variant of a folder in which a repeated token stands out: query weights equal to key weights (times three) in every
    attention layer, a memory that forgets slowly and reads with its keys' weights, sinks of several units that differ by
    head, a cap on the scores that bites, and an embedding large enough to dominate the stream."""
    config = config_of(base)

    def edit(weights):
        # token ECHO is token CALL twice as large: behind a norm its key is CALL's (a query of CALL finds it as it finds
        # itself), while what it adds as a value, or to a memory, is not
        weights["embed"][ECHO] = 2 * weights["embed"][CALL]
        for i, layer in enumerate(config["layers"]):
            p = f"l{i}.mix."
            m = layer["mixer"]
            if layer["type"] == "wkv":
                weights[p + "w0"] = torch.full_like(weights[p + "w0"], -4.0)
                weights[p + "w2"] = weights[p + "w2"] * 0.1
                weights[p + "r"] = weights[p + "k"].clone()
                weights[p + "mu.r"] = weights[p + "mu.k"].clone()
                continue
            heads, kv_heads, d = m["heads"], m["kv_heads"], m["dim"]
            source = m.get("kv_from")
            k = weights[(p if source is None else f"l{source}.mix.") + "k"].float().reshape(kv_heads, d, -1)
            if source is None:
                k = k * 3
                weights[p + "k"] = k.reshape(kv_heads * d, -1).to(torch.bfloat16)
            weights[p + "q"] = k.repeat_interleave(heads // kv_heads, dim=0).reshape(heads * d, -1).to(torch.bfloat16)
            if "mask" in m:
                # (the windowed layer speaks as loudly as the embedding)
                weights[f"l{i}.norm1"] = torch.full_like(weights[f"l{i}.norm1"], 7.0)
            if layer["type"] == "attention_2":
                weights[p + "sink"] = torch.tensor([(-1.0) ** a * (2.0 + a) for a in range(heads)], dtype=torch.bfloat16)

    def caps(edited):
        for layer in edited["layers"]:
            if "softcap" in layer["mixer"]:
                layer["mixer"]["softcap"] = 4.0               # (low enough that the cap decides the repeated token's score)
            if "mask" in layer["mixer"]:
                # (slow angles: the echo's key keeps most of its likeness to the query over the window's length, where with
                # fast ones the query's own key, which is not turned against it, would take all the weight)
                layer["mixer"]["rot"]["base"] = 1e9
        # every sublayer's output enters the stream with a root mean square near one: the embedding must stand above that
        # for a token to be recognised as itself in the later layers
        edited["embedding"]["scale"] = 100.0

    return rewrite(base, edit, caps)
