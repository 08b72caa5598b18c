"""Small Letevik configurations for the tests, their model folders and crafted variants."""

from __future__ import annotations

import functools
import json
import tempfile
from typing import Dict

import torch

from kestrel_amd.weights import InitRecipe, write_random_model


def differential(heads, kv_heads, dim, vdim, scale, diff, conv, mask, rot, ff=None, limit=2.0):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
             "rot": {"base": rot[1], "dims": rot[0]}}
    if conv is not None:
        mixer["conv"] = conv
    if mask is not None:
        mixer["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, ff=None, limit=2.0):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
             "rot": {"base": base, "dims": rot_dim}}
    return {"type": "latent_attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def _config(vocab, width, eps, bigram, layers, loop=None):
    out = {"architecture": "Letevik", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}, "layers": layers}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


CONFIGS: Dict[str, dict] = {
    # sizes the matrix-core kernels take; a window of one and a half pages that keeps four keys; the loop over the first two layers
    "P": _config(300, 64, 1e-5, (97, 7, 13), [
        differential(4, 2, 32, 64, 0.2, 0.4, 3, (24, 4), (32, 8000.0), 128, 1.5),
        latent(4, 32, 16, 32, 48, 64, 0.15, 50000.0, 128, 3.0),
        differential(2, 2, 64, 32, 0.12, 0.7, 4, (40, 0), (16, 500.0), None),
        latent(2, 64, 32, 64, 32, 128, 0.1, 1e4, 128, 2.0),
    ], (0, 2, 2)),
    # sizes that fit no alignment: odd heads and ranks, two taps, a window shorter than a page with more kept keys than a window,
    # fewer rotated channels than a map has, a loop in the middle that runs three times, layers without a feed-forward
    "Q": _config(211, 100, 1e-6, (53, 31, 17), [
        latent(5, 24, 8, 10, 36, 40, 0.2, 300.0, None),
        differential(6, 3, 20, 12, 0.25, 0.3, 2, (7, 9), (12, 500.0), 50, 0.8),
        latent(3, 12, 6, 20, 20, 28, 0.3, 77.0, 90, 5.0),
        differential(3, 1, 28, 36, 0.2, 0.55, 5, (33, 1), (28, 20.0), None),
    ], (1, 3, 3)),
    # no loop at all, one tap (a convolution without state), no convolution, no mask, kept keys beyond a page, a window of whole pages
    "R": _config(190, 128, 1e-3, (769, 1, 1), [
        differential(2, 1, 64, 128, 0.09, 0.5, 1, (32, 17), (64, 1e6), 136, 2.0),
        differential(4, 4, 32, 32, 0.18, 0.2, None, None, (8, 1e4), 136, 2.5),
        latent(8, 48, 16, 64, 96, 80, 0.12, 30000.0, 136, 2.0),
    ]),
    # one of everything: one head, one pass of the loop, a window of one key that keeps one, one bucket
    "S": _config(77, 48, 1e-5, (1, 3, 5), [
        differential(1, 1, 16, 48, 0.5, 0.9, 2, (1, 1), (2, 3.0), 40, 1.0),
        latent(1, 16, 2, 48, 8, 8, 0.4, 3.0, 40, 1.0),
    ], (0, 1, 1)),
}
RECIPE = InitRecipe(std=0.08, bias_std=0.5, gain_std=0.2)
SEEDS = {"P": 31, "Q": 32, "R": 33, "S": 34}


# With one standard deviation for all matrices the mixers would add little to the stream beside the feed-forwards (a latent
# mixer is a chain of five products, and a softmax over many keys averages values out), and a fault in a mask, a sink or a
# cache would move the logits by less than rounding does. Their output projections are therefore made larger.
OUTPUT_BOOST = {"attention": 2.0, "latent_attention": 8.0}


@functools.lru_cache(maxsize=None)
def model_dir(name: str) -> str:
    from safetensors.torch import save_file

    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_letevik{name}_")
    write_random_model(folder, CONFIGS[name], SEEDS[name], RECIPE, store_dtype="bfloat16")
    weights = stored_weights(folder)
    for i, layer in enumerate(CONFIGS[name]["layers"]):
        key = f"l{i}.mix.o"
        weights[key] = (weights[key].float() * OUTPUT_BOOST[layer["type"]]).to(torch.bfloat16)
    save_file({k: v.contiguous() for k, v in weights.items()}, folder + "/model.safetensors")
    return folder


def stored_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(folder + "/model.safetensors")


def config_of(folder: str) -> dict:
    with open(folder + "/config.json") as handle:
        return json.load(handle)


def rewrite(folder: str, edit, edit_config=None) -> str:
    """A copy of a model folder whose weights went through ``edit(weights dict)`` (and its configuration through
    ``edit_config(config dict)``)."""
    from safetensors.torch import save_file

    weights = stored_weights(folder)
    edit(weights)
    config = config_of(folder)
    if edit_config is not None:
        edit_config(config)
    out = tempfile.mkdtemp(prefix="kestrel_amd_letevik_edit_")
    save_file({k: v.contiguous() for k, v in weights.items()}, out + "/model.safetensors")
    with open(out + "/config.json", "w") as handle:
        json.dump(config, handle)
    return out


# For tests that make one key's score stand out: the latent layer's two ranks are equal, so that its queries can be given
# its keys' weights; the window of the differential layer is one and a half pages and keeps four keys; both layers loop.
CONFIGS["T"] = _config(400, 64, 1e-5, (211, 5, 3), [
    differential(2, 1, 32, 32, 0.25, 0.3, 3, (24, 4), (32, 10000.0), 96, 2.0),
    latent(2, 32, 16, 32, 64, 64, 0.2, 10000.0, 96, 2.0),
], (0, 2, 2))
SEEDS["T"] = 35


def stand_out(weights: Dict[str, torch.Tensor], config: dict, factor: float = 3.0, embed: float = 4.0) -> None:
    """The token embedding is made ``embed`` times larger (a token then looks much the same whatever stood before it), and queries get the keys' weights (times ``factor``), so that a token's query scores highest against the key of the same token
    wherever it stands: in differential layers on the first map only and with convolutions that pass q and k through unchanged, in
    latent layers (whose ranks must be equal) on the unrotated part."""
    weights["embed"] = (weights["embed"].float() * embed).to(torch.bfloat16)
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            k = weights[p + "k"].float().reshape(G, 2, d, -1)
            q = weights[p + "q"].float().reshape(H, 2, d, -1).clone()
            q[:, 0] = factor * k[:, 0].repeat_interleave(H // G, dim=0)
            weights[p + "q"] = q.reshape(H * 2 * d, -1).to(torch.bfloat16)
            if m.get("conv"):
                for name in ("q", "k"):
                    taps = torch.zeros_like(weights[p + name + ".conv"])
                    taps[:, -1] = 1.0
                    weights[p + name + ".conv"] = taps
        else:
            H, d, dr, rank = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
            assert m["q_rank"] == rank
            weights[p + "dq"] = weights[p + "dkv"][:rank].clone()
            weights[p + "dq.norm"] = weights[p + "dkv.norm"].clone()
            uq = weights[p + "uq"].float().reshape(H, d + dr, rank).clone()
            uq[:, :d] = factor * weights[p + "uk"].float().reshape(H, d, rank)
            weights[p + "uq"] = uq.reshape(H * (d + dr), rank).to(torch.bfloat16)
