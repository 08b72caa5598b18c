"""Decode and prefill throughput of the engine on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints one JSON line. A step is one
decode step of the default batch (8 requests, each holding ``context`` tokens: a block of
prefix embeddings and text ids) through the engine's step function with greedy sampling
on the GPU. The model has the layer sizes of the Moondream 2 text decoder with seeded
random weights N(0, 0.02) in bf16; inputs are synthetic. Besides ``value`` (decoded tokens
a second) the line carries a 2,048-token prefill, the decode step's HBM roofline and
decode throughput at batch 1 and 64. Beside the nominal peaks the line names what this GPU reaches on a plain
read stream and on a loop of matrix instructions (``peak_measured``; ``--no-peaks`` leaves that out).

``--workload waves256`` and ``--workload mixed48`` (the latter meant for ``--sizes phi2``) measure
the whole engine instead: a model folder is written with seeded random weights, loaded through the
loader, and requests go through ``InferenceEngine`` (scheduler, sampler, paged cache under
pressure); the line then reports generated tokens a second. With ``--check N`` (meant for ``--layers 2``) the first N
greedy requests of such a run are compared, token by token, with the plain implementation under ``tests/``.

``--workload compare-vimesun`` measures the Vimesun design beside the Moondream decoder at equal sizes (width,
feed-forward, heads, head size, runs of layers, vocabulary; random weights): a prompt alone and decode steps at batch 1,
8 and 64 through the same step function, each with its share of the roofline (``--compare-sizes``, ``--compare-model``).
``--workload compare-bogivik`` does the same for the Bogivik design (layers of attention with a distance bias and a
layer of chunked attention beside a matrix memory) at sizes of its own (``BOGIVIK_SIZES``), and
``--workload compare-bokorax`` for the Bokorax design (two kinds of attention, a decaying matrix memory, routed experts),
``--workload compare-letevik`` for the Letevik design (differential attention behind short convolutions and latent
attention in a looped stretch of layers; ``LETEVIK_SIZES``).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Layer sizes of the benchmark model (Moondream 2 text decoder) and its workload.
MODEL = {"dim": 2048, "ff_dim": 8192, "n_layers": 24, "vocab_size": 51200, "max_context": 2048, "n_heads": 32,
         "n_kv_heads": 32, "rope_theta": 10000.0, "prefix_attn": 730, "layer_norm_eps": 1e-5}
# Another member of the family for measurements beside the default: Phi-2's layer sizes (head size 80).
SIZES = {
    "moondream2": MODEL,
    "phi2": {"dim": 2560, "ff_dim": 10240, "n_layers": 32, "vocab_size": 51200, "max_context": 2048, "n_heads": 32,
             "n_kv_heads": 32, "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5, "rotary_dim": 32},
}
LABELS = {"moondream2": ("Moondream 2 text decoder sizes", "moondream2-text"), "phi2": ("Phi-2 layer sizes", "phi2-sizes")}
CONTEXT = 1024          # tokens each request holds when decoding starts (730 prefix + 294 text)
PREFILL_TOKENS = 2048
PAGE_SIZE = 16
SEED = 2
PEAK_HBM = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def build_model(layers: int, dtype, device, sizes=None):
    """The benchmark model with random weights drawn on the GPU (nothing is read from disk)."""
    import torch

    from kestrel_amd.config import get_spec
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.weights import InitRecipe, random_tensor

    spec = get_spec("moondream2")
    typed = spec.read_config({"text": dict(sizes or MODEL, n_layers=layers)})
    net = DecoderModel(spec.build_plan(typed))
    recipe = InitRecipe(std=0.02)
    store = torch.bfloat16
    tensors = {name: random_tensor(name, pspec, SEED, recipe, device=device).to(store if dtype == torch.bfloat16 else dtype)
               for name, pspec in net.params().items()}
    net.bind(tensors, dtype, device)
    return net, typed


def build_from_config(config: dict, model: str, dtype, device):
    """A model of any registered architecture from its ``config.json`` dictionary, random weights drawn on the GPU."""
    import torch

    from kestrel_amd.config import get_spec
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.weights import InitRecipe, random_tensor

    spec = get_spec(model)
    typed = spec.read_config(config)
    net = DecoderModel(spec.build_plan(typed))
    recipe = InitRecipe(std=0.02)
    tensors = {name: random_tensor(name, pspec, SEED, recipe, device=device).to(torch.bfloat16 if dtype == torch.bfloat16 else dtype)
               for name, pspec in net.params().items()}
    net.bind(tensors, dtype, device)
    return net, typed


# Sizes at which the two designs are measured side by side: (label, width, feed-forward, heads, kv heads, head size,
# value head size of Vimesun, window of Vimesun or None for its position limit, layers, looped stretch and passes).
# Moondream gets as many layers as Vimesun has runs of layers; its values have the keys' size.
COMPARE_SIZES = {
    "w2048": dict(width=2048, ff=8192, heads=32, kv_heads=32, head=64, vdim=64, window=None, layers=4, loop=(1, 3, 2)),
    "w2048-window": dict(width=2048, ff=8192, heads=32, kv_heads=32, head=64, vdim=64, window=512, layers=4, loop=(1, 3, 2)),
    "w4096-gqa": dict(width=4096, ff=11008, heads=32, kv_heads=8, head=128, vdim=128, window=None, layers=3, loop=(1, 2, 2)),
    "w2560-v": dict(width=2560, ff=10240, heads=32, kv_heads=8, head=64, vdim=96, window=1024, layers=4, loop=(1, 3, 2)),
}
COMPARE_VOCAB = 51200


def compare_models(size: dict, positions: int):
    """``{name: (config dict, registry name, facts)}`` of the two designs at one size; ``facts`` is what the roofline
    needs: runs of layers, and per run the linears' weights and the attention's sizes."""
    from types import SimpleNamespace

    start, stop, times = size["loop"]
    runs = size["layers"] + (stop - start) * (times - 1)
    mixer = {"heads": size["heads"], "kv_heads": size["kv_heads"], "dim": size["head"], "vdim": size["vdim"],
             "scale": size["head"] ** -0.5}
    if size["window"]:
        mixer["mask"] = {"size": size["window"]}
    else:
        mixer["mask"] = {"size": positions}
    vimesun = {"architecture": "Vimesun", "vocab": COMPARE_VOCAB, "width": size["width"], "max_positions": positions,
               "norm": {"eps": 1e-5}, "residual_mult": 0.5, "loop": dict(zip(("start", "stop", "times"), size["loop"])),
               "layers": [{"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": size["ff"]}}
                          for _ in range(size["layers"])]}
    moondream = {"text": {"dim": size["width"], "ff_dim": size["ff"], "n_layers": runs, "vocab_size": COMPARE_VOCAB,
                          "max_context": positions, "n_heads": size["heads"], "n_kv_heads": size["kv_heads"],
                          "head_dim": size["head"], "rotary_dim": size["head"] // 2, "rope_theta": 10000.0,
                          "prefix_attn": 0, "layer_norm_eps": 1e-5}}
    w, h, g, d = size["width"], size["heads"], size["kv_heads"], size["head"]

    def facts(dv, window, junctions):
        linear = w * (h * d + g * d + g * dv) + h * dv * w + 2 * w * size["ff"]        # weights of one run's linears
        return SimpleNamespace(runs=runs, linear=linear, extra=junctions * 2 * w * w, heads=h, kv_heads=g, d=d, dv=dv,
                               window=window, width=w, vocab=COMPARE_VOCAB)

    return {"vimesun": (vimesun, "vimesun", facts(size["vdim"], size["window"], times)),
            "moondream2": (moondream, "moondream2", facts(d, None, 0))}


def compare_flops(f, tokens: int) -> float:
    """Multiply-adds x 2 of a prompt of ``tokens`` places: linears, score and value products over the keys each
    place sees, the head at the last place."""
    seen = sum(min(p + 1, f.window or p + 1) for p in range(tokens))
    return 2.0 * tokens * (f.runs * f.linear + f.extra) + 2.0 * f.runs * f.heads * (f.d + f.dv) * seen + 2.0 * f.width * f.vocab


def compare_decode_bytes(f, batch: int, context: int, size: int) -> float:
    """Bytes a decode step must read: every weight once, and of every row the keys and values it sees."""
    keys = min(context, f.window or context)
    return size * (f.runs * f.linear + f.extra + f.width * f.vocab + batch * f.runs * f.kv_heads * (f.d + f.dv) * keys)


def run_compare(args, dtype, device) -> dict:
    """Vimesun beside the Moondream decoder at equal sizes, through the same step function."""
    from types import SimpleNamespace

    import torch

    size_bytes = 2 if dtype == torch.bfloat16 else 4
    context, tokens = args.context, args.prefill_tokens
    positions = max(context + args.steps + args.warmup + 16, tokens)
    out = {}
    for label in args.compare_sizes.split(","):
        size = COMPARE_SIZES[label]
        out[label] = {}
        for name, (config, registry_name, f) in compare_models(size, positions).items():
            if args.compare_model not in ("both", name):
                continue
            net, _typed = build_from_config(config, registry_name, dtype, device)
            # (what the timing harness asks of a typed configuration)
            shim = SimpleNamespace(prefix_attn=0, dim=f.width, vocab_size=f.vocab, n_kv_heads=f.kv_heads,
                                   head_dim=(f.d + f.dv) / 2, n_layers=f.runs)
            entry = {}
            seconds, best = time_prefill(net, shim, tokens, repeats=5)
            flops = compare_flops(f, tokens)
            entry["prefill"] = {"tokens": tokens, "ms": round(seconds * 1e3, 3), "best_ms": round(best * 1e3, 3),
                                "tok_s": round(tokens / seconds, 1), "frac_of_peak_flops": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
            for batch in (1, 8, 64):
                steps = args.steps if batch < 64 else max(16, args.steps // 4)
                elapsed, _kv = time_decode(net, shim, batch, context, steps, min(args.warmup, 4))
                moved = compare_decode_bytes(f, batch, context, size_bytes)
                entry[f"decode_b{batch}"] = {"ms_per_step": round(elapsed / steps * 1e3, 4), "tok_s": round(batch * steps / elapsed, 1),
                                             "frac_of_peak_hbm": round(moved / (elapsed / steps) / PEAK_HBM, 4)}
            out[label][name] = entry
            del net
            torch.cuda.empty_cache()
    first = out[args.compare_sizes.split(",")[0]]
    lead = first.get("vimesun") or next(iter(first.values()))
    return {"metric": f"Vimesun beside the Moondream decoder at equal sizes: decode tok/s at batch 8, context {context} ({args.compare_sizes.split(',')[0]})",
            "value": lead["decode_b8"]["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": lead["decode_b8"]["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": args.dtype, "data": "synthetic (seeded random token ids, random weights N(0,0.02))",
            "config": {"model": "vimesun and moondream2-text at equal sizes", "sizes": {k: COMPARE_SIZES[k] for k in out},
                       "global_batch": 8, "seq_len": context, "vocab_size": COMPARE_VOCAB, "parallelism": "single-gpu"},
            "compare": out}


# Sizes at which Bogivik is measured beside the Moondream decoder: width, gated feed-forward (Moondream's plain one gets
# one and a half times the hidden size: the same weights), heads, kv heads, head size (keys and values), the chunk of the
# chunked branch, heads and head sizes of the matrix memory, and the order of layers (a: attention, p: parallel).
BOGIVIK_SIZES = {
    "w2048": dict(width=2048, ff=5632, heads=32, kv_heads=8, head=64, chunk=1024, memory=(8, 64, 256), order="aapa"),
    "w4096": dict(width=4096, ff=7168, heads=32, kv_heads=8, head=128, chunk=2048, memory=(16, 64, 256), order="apa"),
}


def bogivik_models(size: dict, positions: int):
    """``{name: (config dict, registry name)}`` of Bogivik and of the Moondream decoder at one size."""
    h, g, d, w = size["heads"], size["kv_heads"], size["head"], size["width"]
    mlp = {"kind": "dense", "ff": size["ff"]}
    attention = {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "bias_max": 128, "buckets": 32,
                 "q_temp": {"coef": 0.5, "every": 64}, "v_mix": True}
    mh, md, mdv = size["memory"]
    parallel = {"left": {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": size["chunk"]},
                         "rot": {"base": 10000.0, "dims": d, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}},
                "right": {"heads": mh, "dim": md, "vdim": mdv, "gate_cap": 15.0}}
    layers = [{"type": "attention", "mixer": dict(attention), "mlp": mlp} if kind == "a" else
              {"type": "parallel", "mixer": parallel, "mlp": mlp} for kind in size["order"]]
    bogivik = {"architecture": "Bogivik", "vocab": COMPARE_VOCAB, "width": w, "norm": {"eps": 1e-6}, "max_positions": positions,
               "layers": layers}
    moondream = {"text": {"dim": w, "ff_dim": size["ff"] * 3 // 2, "n_layers": len(size["order"]), "vocab_size": COMPARE_VOCAB,
                          "max_context": positions, "n_heads": h, "n_kv_heads": g, "head_dim": d, "rotary_dim": d // 2,
                          "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5}}
    return {"bogivik": (bogivik, "bogivik"), "moondream2": (moondream, "moondream2")}


def design_facts(net):
    """What the roofline of any model of the package needs, read off its plan: the weights of its linears (every matrix
    but the embedding table), and per layer of its attention ``(multiply-adds a query spends per key it sees, numbers
    the cache holds per key, window, chunk, kept first keys)`` and the sizes of its matrix memory (heads, key and value size)."""
    from types import SimpleNamespace

    plan = net.plan
    embedding = plan.names["embedding"]
    linear = sum(int(__import__("math").prod(p.shape)) for name, p in net.params().items() if p.role == "matrix" and name != embedding)
    attention, memory, experts = [], [], []

    def walk(spec):
        kind = getattr(spec, "kind", None)
        if kind == "attention":
            dv = spec.head_dim if getattr(spec, "value_dim", None) is None else spec.value_dim
            attention.append((spec.n_heads * (spec.head_dim + dv), spec.n_kv_heads * (spec.head_dim + dv),
                              getattr(spec, "window", None), getattr(spec, "chunk", None), 0))
        elif kind == "differential_attention":
            # two maps per head, each a score and a value product; the cache holds two keys and one value per kv head
            mask = spec.mask
            attention.append((2 * spec.n_heads * (spec.head_dim + spec.value_dim), spec.n_kv_heads * (2 * spec.head_dim + spec.value_dim),
                              mask.size if mask is not None else None, None, mask.keep_first if mask is not None else 0))
        elif kind == "latent_attention":
            # per head a score over the plain and the rotated part and a value product; the cache holds the latent and
            # the shared rotated key part
            attention.append((spec.n_heads * (spec.head_dim + spec.rot_dim + spec.value_dim), spec.kv_rank + spec.rot_dim, None, None, 0))
        elif kind == "matrix_memory":
            memory.append((spec.n_heads, spec.head_dim, spec.value_dim))
        elif kind == "decayed_memory":
            memory.append((spec.n_heads, spec.head_dim, spec.head_dim))
        elif kind == "branches":
            for branch in spec.branches:
                walk(branch)

    for entry in plan.schedule:
        walk(plan.layers[entry.layer].mixer)
        ff = plan.layers[entry.layer].feed_forward
        if getattr(ff, "kind", None) == "routed_experts":
            # routed experts: a token multiplies with `top` of them, and a step reads those that its tokens chose; they are
            # counted apart from the weights that every token uses
            size = 3 * ff.dim * ff.hidden_dim
            experts.append((ff.n_experts, ff.top, size))
            linear -= ff.n_experts * size
    return SimpleNamespace(linear=linear, attention=attention, memory=memory, experts=experts, width=plan.dim, vocab=plan.vocab_size)


def _keys_seen(place: int, window, chunk, keep_first: int = 0) -> int:
    lo = 0
    if window is not None:
        lo = max(lo, place + 1 - window)
    if chunk is not None:
        lo = max(lo, place // chunk * chunk)
    return place + 1 - lo + min(keep_first, lo)


def design_flops(f, tokens: int) -> float:
    """Multiply-adds x 2 of a prompt of ``tokens`` places: the linears (the head at the last place only), score and value
    products over the keys each place sees, the matrix memory's update and read-out (two multiply-adds a number of state)."""
    total = 2.0 * tokens * (f.linear - f.width * f.vocab) + 2.0 * f.width * f.vocab
    for per_key, _held, window, chunk, kept in f.attention:
        total += 2.0 * per_key * sum(_keys_seen(p, window, chunk, kept) for p in range(tokens))
    for h, d, dv in f.memory:
        total += 2.0 * 2.0 * h * d * dv * tokens
    for _count, top, size in getattr(f, "experts", ()):
        total += 2.0 * tokens * top * size
    return total


def design_decode_bytes(f, batch: int, context: int, size: int) -> float:
    """Bytes a decode step must move: every weight once, of every row the keys and values it sees, and its matrix
    memories' fp32 state read and written."""
    total = float(size) * f.linear
    for _per_key, held, window, chunk, kept in f.attention:
        total += size * batch * held * _keys_seen(context, window, chunk, kept)
    for h, d, dv in f.memory:
        total += 2.0 * 4 * batch * h * (d * dv + d + 1)
    for count, top, expert_size in getattr(f, "experts", ()):
        total += float(size) * min(count, batch * top) * expert_size          # (at most: rows may choose the same experts)
    return total


# Sizes at which Letevik is measured beside the Moondream decoder: width, gated feed-forward (Moondream's plain one gets
# one and a half times the hidden size: the same weights), the differential layers' heads, kv heads, size of a map and of
# a value, taps, window and kept keys, the latent layers' heads, plain and rotated key size, value size and the two
# ranks, the order of layers (d: differential, l: latent) and the looped stretch with its passes. Moondream gets as many
# layers as Letevik has runs of layers, and heads of the size of a pair of maps. "w2048" has latent rows of 128 numbers
# (what the matrix-core attention kernel takes), "w4096" rows of 576 (the sizes of latent attention as published
# models have them; the generic kernel runs).
LETEVIK_SIZES = {
    "w2048": dict(width=2048, ff=5632, diff=dict(heads=16, kv_heads=4, dim=64, vdim=128, conv=4, window=1024, keep=4),
                  latent=dict(heads=16, dim=64, rot_dim=32, vdim=64, q_rank=512, kv_rank=96), order="dlld", loop=(0, 2, 2),
                  moondream=dict(heads=32, kv_heads=8, head=64)),
    "w4096": dict(width=4096, ff=7168, diff=dict(heads=16, kv_heads=4, dim=128, vdim=128, conv=4, window=2048, keep=16),
                  latent=dict(heads=32, dim=128, rot_dim=64, vdim=128, q_rank=1536, kv_rank=512), order="dl", loop=(0, 2, 2),
                  moondream=dict(heads=32, kv_heads=8, head=128)),
}


def letevik_models(size: dict, positions: int):
    """``{name: (config dict, registry name)}`` of Letevik and of the Moondream decoder at one size."""
    w, d, m = size["width"], size["diff"], size["latent"]
    mlp = {"kind": "dense", "ff": size["ff"], "limit": 7.0}
    differential = {"heads": d["heads"], "kv_heads": d["kv_heads"], "dim": d["dim"], "vdim": d["vdim"], "scale": d["dim"] ** -0.5,
                    "diff": 0.5, "conv": d["conv"], "mask": {"size": d["window"], "keep_first": d["keep"]},
                    "rot": {"base": 10000.0, "dims": d["dim"]}}
    latent = {"heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "q_rank": m["q_rank"],
              "kv_rank": m["kv_rank"], "scale": (m["dim"] + m["rot_dim"]) ** -0.5, "rot": {"base": 50000.0, "dims": m["rot_dim"]}}
    layers = [{"type": "attention", "mixer": dict(differential), "mlp": mlp} if kind == "d" else
              {"type": "latent_attention", "mixer": dict(latent), "mlp": mlp} for kind in size["order"]]
    start, stop, times = size["loop"]
    letevik = {"architecture": "Letevik", "vocab": COMPARE_VOCAB, "width": w, "norm": {"eps": 1e-6}, "max_positions": positions,
               "embedding": {"bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 17}}, "layers": layers,
               "loop": {"start": start, "stop": stop, "times": times}}
    md = size["moondream"]
    runs = len(size["order"]) + (stop - start) * (times - 1)
    moondream = {"text": {"dim": w, "ff_dim": size["ff"] * 3 // 2, "n_layers": runs, "vocab_size": COMPARE_VOCAB,
                          "max_context": positions, "n_heads": md["heads"], "n_kv_heads": md["kv_heads"], "head_dim": md["head"],
                          "rotary_dim": md["head"] // 2, "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5}}
    return {"letevik": (letevik, "letevik"), "moondream2": (moondream, "moondream2")}


# Sizes at which Bokorax is measured beside the Moondream decoder: width, heads, kv heads and head size of both kinds of
# attention, the window of the first kind, heads and head size of the decaying memory, the routed experts (how many, their
# hidden size, choices per token, identity experts, groups and kept groups) and the shared expert, and the order of layers
# (2: capped attention with sinks, w: the decaying memory, 1: windowed attention whose values are its keys, s: capped
# attention that reads the keys and values of the first capped layer). A token multiplies with `top` experts and the shared
# one: as many feed-forward weights as Moondream's plain feed-forward of one and a half times `ff`.
BOKORAX_SIZES = {
    "w2048": dict(width=2048, ff=5632, heads=32, kv_heads=8, head=64, window=1024, memory=(32, 64), rank=64,
                  experts=dict(n=30, ff=704, top=4, identity=2, groups=(4, 2), shared=2816), order="2w1s"),
    "w4096": dict(width=4096, ff=7168, heads=32, kv_heads=8, head=128, window=2048, memory=(64, 64), rank=128,
                  experts=dict(n=62, ff=896, top=6, identity=2, groups=(8, 4), shared=1792), order="w21"),
}


def bokorax_models(size: dict, positions: int):
    """``{name: (config dict, registry name)}`` of Bokorax and of the Moondream decoder at one size."""
    h, g, d, w = size["heads"], size["kv_heads"], size["head"], size["width"]
    e = size["experts"]
    mlp = {"kind": "moe", "expert": {"ff": e["ff"]}, "shared": {"ff": e["shared"]},
           "router": {"experts": e["n"], "top": e["top"], "identity": e["identity"], "scale": 2.5,
                      "groups": {"count": e["groups"][0], "keep": e["groups"][1]}}}
    first = {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": size["window"]},
             "rot": {"base": 10000.0, "dims": d // 2}}
    second = {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "softcap": 50.0,
              "rot": {"base": 500000.0, "dims": d, "scaling": {"factor": 8.0}}}
    memory = {"heads": size["memory"][0], "dim": size["memory"][1], "decay_rank": size["rank"]}
    layers, source = [], None
    for i, kind in enumerate(size["order"]):
        if kind == "w":
            layers.append({"type": "wkv", "mixer": dict(memory), "mlp": mlp})
        elif kind == "1":
            layers.append({"type": "attention", "mixer": dict(first), "mlp": mlp})
        else:
            mixer = dict(second)
            if kind == "s":
                mixer["kv_from"] = source
            else:
                source = i if source is None else source
            layers.append({"type": "attention_2", "mixer": mixer, "mlp": mlp})
    bokorax = {"architecture": "Bokorax", "vocab": COMPARE_VOCAB, "width": w, "norm": {"eps": 1e-6}, "max_positions": positions,
               "embedding": {"scale": 1.0}, "logit_scale": 1.0, "layers": layers}
    moondream = {"text": {"dim": w, "ff_dim": size["ff"] * 3 // 2, "n_layers": len(size["order"]), "vocab_size": COMPARE_VOCAB,
                          "max_context": positions, "n_heads": h, "n_kv_heads": g, "head_dim": d, "rotary_dim": d // 2,
                          "rope_theta": 10000.0, "prefix_attn": 0, "layer_norm_eps": 1e-5}}
    return {"bokorax": (bokorax, "bokorax"), "moondream2": (moondream, "moondream2")}


def run_compare_bokorax(args, dtype, device) -> dict:
    """Bokorax beside the Moondream decoder at equal sizes, through the same step function."""
    return run_compare_design(args, dtype, device, "bokorax", BOKORAX_SIZES, bokorax_models)


def run_compare_bogivik(args, dtype, device) -> dict:
    """Bogivik beside the Moondream decoder at equal sizes, through the same step function."""
    return run_compare_design(args, dtype, device, "bogivik", BOGIVIK_SIZES, bogivik_models)


def run_compare_letevik(args, dtype, device) -> dict:
    """Letevik beside the Moondream decoder at equal sizes, through the same step function."""
    return run_compare_design(args, dtype, device, "letevik", LETEVIK_SIZES, letevik_models)


def run_compare_design(args, dtype, device, design: str, sizes: dict, models) -> dict:
    """A design beside the Moondream decoder at the sizes of ``sizes`` (``models(size, positions)`` gives both configurations),
    through the same step function."""
    from types import SimpleNamespace

    import torch

    size_bytes = 2 if dtype == torch.bfloat16 else 4
    context, tokens = args.context, args.prefill_tokens
    positions = max(context + args.steps + args.warmup + 16, tokens)
    labels = (args.compare_sizes or ",".join(sizes)).split(",")
    out = {}
    for label in labels:
        out[label] = {}
        for name, (config, registry_name) in models(sizes[label], positions).items():
            if args.compare_model not in ("both", name):
                continue
            net, _typed = build_from_config(config, registry_name, dtype, device)
            f = design_facts(net)
            shim = SimpleNamespace(prefix_attn=0, dim=f.width, vocab_size=f.vocab, n_kv_heads=1, head_dim=1, n_layers=1)
            entry = {}
            if not args.skip_prefill:
                seconds, best = time_prefill(net, shim, tokens, repeats=5)
                flops = design_flops(f, tokens)
                entry["prefill"] = {"tokens": tokens, "ms": round(seconds * 1e3, 3), "best_ms": round(best * 1e3, 3),
                                    "tok_s": round(tokens / seconds, 1), "frac_of_peak_flops": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
            for batch in [int(b) for b in args.compare_batches.split(",") if b]:
                steps = args.steps if batch < 64 else max(16, args.steps // 4)
                elapsed, _kv = time_decode(net, shim, batch, context, steps, min(args.warmup, 4))
                moved = design_decode_bytes(f, batch, context, size_bytes)
                entry[f"decode_b{batch}"] = {"ms_per_step": round(elapsed / steps * 1e3, 4), "tok_s": round(batch * steps / elapsed, 1),
                                             "frac_of_peak_hbm": round(moved / (elapsed / steps) / PEAK_HBM, 4)}
            out[label][name] = entry
            del net
            torch.cuda.empty_cache()
    first = out[labels[0]]
    lead = first.get(design) or next(iter(first.values()))
    key = "decode_b8" if "decode_b8" in lead else next((k for k in lead if k.startswith("decode")), None)
    return {"metric": f"{design.capitalize()} beside the Moondream decoder at equal sizes: decode tok/s at batch 8, context {context} ({labels[0]})",
            "value": lead[key]["tok_s"] if key else None, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": lead[key]["ms_per_step"] if key else None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": args.dtype, "data": "synthetic (seeded random token ids, random weights N(0,0.02))",
            "config": {"model": f"{design} and moondream2-text at equal sizes", "sizes": {k: sizes[k] for k in out},
                       "global_batch": 8, "seq_len": context, "vocab_size": COMPARE_VOCAB, "parallelism": "single-gpu"},
            "compare": out}


def model_bytes(net, dtype_size: int) -> int:
    """Bytes of weights a decode step reads once: every linear, norm and the head (the
    embedding table is read only at the rows of the batch)."""
    total = 0
    emb = net.plan.names["embedding"]
    for name, pspec in net.params().items():
        if name == emb:
            continue
        count = 1
        for s in pspec.shape:
            count *= s
        total += count * dtype_size
    return total


def prefill_flops(typed, tokens: int, prefix: int) -> float:
    """Multiply-adds x 2 of one prompt of ``tokens`` positions whose first ``prefix`` are a
    bidirectional block; the head runs on the last position only."""
    d, ff, hd = typed.dim, typed.ff_dim, typed.head_dim
    qkv = (typed.n_heads + 2 * typed.n_kv_heads) * hd
    per_token_linear = 2 * (d * qkv + typed.n_heads * hd * d + 2 * d * ff)
    pairs = prefix * prefix + sum(q + 1 for q in range(prefix, tokens))
    attention = 4 * hd * typed.n_heads * pairs
    return typed.n_layers * (tokens * per_token_linear + attention) + 2 * d * typed.vocab_size


class DecodeBench:
    """A batch of requests prefilled to ``context`` tokens, then decoded step by step."""

    def __init__(self, net, typed, batch: int, context: int, steps_total: int):
        import torch

        from kestrel_amd.engine.loading import make_runner
        from kestrel_amd.engine.step import PENDING_TOKEN, StepEntry
        from kestrel_amd.sampling import Sampler

        self.torch, self.StepEntry, self.PENDING = torch, StepEntry, PENDING_TOKEN
        self.net, self.typed, self.batch, self.context = net, typed, batch, context
        pages_per_request = -(-(context + steps_total + 1) // PAGE_SIZE)
        self.runner = make_runner(net, PAGE_SIZE, batch * pages_per_request, batch, max_tokens_per_step=max(4096, context),
                                  enable_graphs=True)
        self.sampler = Sampler(net.device, pending=self.runner.pending)
        self.host = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.unread = None                      # (event, pinned tokens) of the step launched last
        self.n_steps = 0
        gen = torch.Generator().manual_seed(SEED)
        prefix = min(typed.prefix_attn, context - 1)
        self.slots = []
        last = []
        for _ in range(batch):
            slot = self.runner.admit()
            embeds = torch.randn(prefix, typed.dim, generator=gen)
            ids = torch.randint(0, typed.vocab_size, (context - prefix,), generator=gen).tolist()
            entry = StepEntry(slot, [-1] * prefix + ids, want=[context - 1], embeds=embeds.to(net.device),
                              bidirectional=[(0, prefix)] if prefix else [])
            logits = self.runner.step([entry])
            last.append(int(self.sampler.greedy(logits, slots=[slot])[0]))
            self.slots.append(slot)
        self.last = last

    def step(self):
        """One decode step as the scheduler runs it with two steps in flight: the next step is
        launched with the tokens that sampling left on the device, then the tokens of the step
        before are read on the host."""
        torch = self.torch
        entries = [self.StepEntry(slot, [self.PENDING], want=[0]) for slot in self.slots]
        logits = self.runner.step(entries)
        host = self.host[self.n_steps % 2]
        self.sampler.greedy(logits, out=host, slots=self.runner.logit_slots)      # (the kernel writes into the pinned memory)
        event = torch.cuda.Event()
        event.record()
        if self.unread is not None:
            self.unread[0].synchronize()
            self.last = self.unread[1].tolist()
        self.unread = (event, host)
        self.n_steps += 1

    def kv_bytes_now(self, dtype_size: int) -> int:
        t = self.typed
        per_token = 2 * t.n_kv_heads * t.head_dim * dtype_size * t.n_layers
        return per_token * sum(self.runner.held[s] for s in self.slots)

    def close(self):
        for slot in self.slots:
            self.runner.release(slot)
        self.runner = None


def time_decode(net, typed, batch, context, steps, warmup):
    import torch

    bench = DecodeBench(net, typed, batch, context, steps + warmup)
    for _ in range(warmup):
        bench.step()
    torch.cuda.synchronize()
    kv_start = bench.kv_bytes_now(2)
    started = time.perf_counter()
    for _ in range(steps):
        bench.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    kv_end = bench.kv_bytes_now(2)
    bench.close()
    torch.cuda.empty_cache()
    return elapsed, 0.5 * (kv_start + kv_end)


def time_prefill(net, typed, tokens, repeats=8):
    import torch

    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry

    # (as the engine runs it: a step short enough for the host's launches to take longer than its kernels is a replayed graph)
    runner = make_runner(net, PAGE_SIZE, -(-tokens // PAGE_SIZE) + 1, 1, max_tokens_per_step=tokens, enable_graphs=True)
    gen = torch.Generator().manual_seed(SEED + 1)
    prefix = min(typed.prefix_attn, tokens - 1)
    embeds = torch.randn(prefix, typed.dim, generator=gen).to(net.device)
    ids = torch.randint(0, typed.vocab_size, (tokens - prefix,), generator=gen).tolist()
    times = []
    for i in range(repeats + 1):
        slot = runner.admit()
        entry = StepEntry(slot, [-1] * prefix + ids, want=[tokens - 1], embeds=embeds,
                          bidirectional=[(0, prefix)] if prefix else [])
        torch.cuda.synchronize()
        started = time.perf_counter()
        runner.step([entry])
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        runner.release(slot)
        if i > 0:                      # the first run warms up
            times.append(elapsed)
    times.sort()
    return times[len(times) // 2], times[0]          # the median of the runs, and the best of them


def write_model_folder(sizes: dict, layers: int, seed: int) -> str:
    """A model folder (config.json, model.safetensors) with seeded random weights N(0, 0.02)."""
    import tempfile

    from kestrel_amd.weights import InitRecipe, write_random_model

    folder = tempfile.mkdtemp(prefix="kestrel_amd_bench_")
    write_random_model(folder, {"text": dict(sizes, n_layers=layers)}, seed, InitRecipe(std=0.02))
    return folder


def check_greedy(args, sizes: dict, folder: str, greedy: dict, results, prefix) -> int:
    """``--check N``: the first N greedy requests of a workload against the plain implementation under ``tests/``
    (float64, whole sequences, no cache): every token the engine generated must be the plain model's choice
    after the engine's own earlier tokens, up to what the precision leaves of a near tie (twice the bound the
    tests put on a bf16 logit: 3 % of the row's spread + 1 % of the value). Returns how many were compared;
    raises if a token is not."""
    if args.check <= 0:
        return 0
    from safetensors.torch import load_file

    from tests.plain import moondream_plain as plain

    weights = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    cfg = dict(sizes, n_layers=args.layers)
    done = 0
    for index in sorted(greedy)[:args.check]:
        ids, tokens = greedy[index], results[index].tokens
        logits = plain.forward(cfg, weights, list(ids) + tokens[:-1], prefix)
        first = (0 if prefix is None else prefix.shape[0]) + len(ids) - 1
        for i, token in enumerate(tokens):
            row = logits[first + i]
            gap, allowed = float(row.max() - row[token]), 2 * float(0.03 * row.std() + 0.01 * row.max().abs())
            if args.dtype == "fp32":
                allowed = 1e-4
            if gap > allowed:
                raise AssertionError(f"request {index}: token {i} is {token}, the plain implementation prefers "
                                     f"{int(row.argmax())} by {gap:.3g} (allowed {allowed:.3g})")
        done += 1
    return done


def run_workload(args, sizes: dict) -> dict:
    """Requests through the entry point. ``waves256``: 256 requests in 4 waves, each a block of 730
    given embeddings and 32 to 128 ids, 128 new tokens, half greedy and half at temperature 1, in
    a cache pool of about 60 GB. ``mixed48``: 48 requests with prompts of 64 to 1,536 ids fed in
    portions of at most 512 tokens beside the decoded tokens of the others, 128 new tokens each at
    temperature 0.7."""
    import random
    import shutil

    import torch

    from kestrel_amd import InferenceEngine, RuntimeConfig

    waves = args.workload == "waves256"
    seed = 4 if waves else 3
    started = time.perf_counter()
    folder = write_model_folder(sizes, args.layers, seed)
    written = time.perf_counter() - started
    n_requests, n_new = (256, 128) if waves else (48, 128)
    if waves:
        cfg = RuntimeConfig(model_path=folder, dtype=args.dtype, max_batch_size=args.max_batch_size or 64,
                            kv_cache_bytes=60 * 10 ** 9 * args.layers // sizes["n_layers"], max_seq_len=2048, seed=seed,
                            tune_linears=args.tune_linears)
    else:
        cfg = RuntimeConfig(model_path=folder, dtype=args.dtype, max_batch_size=args.max_batch_size or 48,
                            max_num_batched_tokens=512, max_seq_len=2048, seed=seed, tune_linears=args.tune_linears)
    started = time.perf_counter()
    engine = InferenceEngine.create_sync(cfg)
    loaded = time.perf_counter() - started
    try:
        rng = random.Random(seed)
        vocab, dim = sizes["vocab_size"], sizes["dim"]
        prefix = torch.randn(730, dim, generator=torch.Generator().manual_seed(seed)).to("cuda:0") if waves else None

        greedy = {}                    # index of a timed greedy request -> its prompt ids

        def submit(i):
            if waves:
                ids = [rng.randrange(0, vocab) for _ in range(rng.randint(32, 128))]
                options = dict(temperature=1.0, top_p=1.0, seed=i) if i % 2 else {}
                if not options and i < 1000:
                    greedy[i] = ids
                return engine.submit_sync(ids, max_new_tokens=n_new, prefix_embeds=prefix, stop_ids=(), **options)
            ids = [rng.randrange(0, vocab) for _ in range(rng.randint(64, 1536))]
            if i < args.check:             # (to be compared with the plain implementation: these decode greedily)
                greedy[i] = ids
                return engine.submit_sync(ids, max_new_tokens=n_new, stop_ids=())
            return engine.submit_sync(ids, max_new_tokens=n_new, temperature=0.7, top_p=1.0, seed=i, stop_ids=())

        for future in [submit(1000 + i) for i in range(8 if waves else 4)]:      # warm-up: graphs, workspaces
            future.result()
        steps_before = engine.scheduler.steps
        started = time.perf_counter()
        futures = []
        for wave in range(4 if waves else 1):
            count = n_requests // 4 if waves else n_requests
            futures += [submit(wave * count + j) for j in range(count)]
            if waves:
                time.sleep(0.05)
        results = [f.result() for f in futures]
        elapsed = time.perf_counter() - started
        steps = engine.scheduler.steps - steps_before
        pages = engine.runner.cache.n_pages
        checked = check_greedy(args, sizes, folder, greedy, results, None if prefix is None else prefix.cpu())
    finally:
        engine.shutdown_sync()
        shutil.rmtree(folder, ignore_errors=True)
    generated = sum(len(r.tokens) for r in results)
    prompt = sum(r.metrics.input_tokens for r in results)
    what = ("256 requests in 4 waves, 730 given embeddings + 32-128 ids each, 128 new tokens, half greedy half T=1" if waves
            else "48 requests, prompts of 64-1536 ids in portions of at most 512 beside decodes, 128 new tokens at T=0.7")
    return {
        "metric": f"generated tok/s through the entry point ({LABELS[args.sizes][0]}; {what})",
        "value": round(generated / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 8 if waves else 4,
        "ms_per_step": round(elapsed / max(steps, 1) * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic (seeded random token ids and prefix embeddings; a folder of random weights N(0,0.02) read by the loader)",
        "config": {"model": LABELS[args.sizes][1], "workload": args.workload, "n_layers": args.layers,
                   "n_layers_full": sizes["n_layers"], "dim": sizes["dim"], "ff_dim": sizes["ff_dim"],
                   "n_heads": sizes["n_heads"], "vocab_size": sizes["vocab_size"], "requests": n_requests,
                   "max_batch_size": cfg.max_batch_size, "max_num_batched_tokens": cfg.max_num_batched_tokens,
                   "kv_cache_pages": pages, "page_size": PAGE_SIZE, "parallelism": "single-gpu"},
        "seconds": round(elapsed, 3), "generated_tokens": generated, "prompt_tokens": prompt,
        "all_tokens_per_second": round((generated + prompt) / elapsed, 1),
        "finish_reasons": sorted({r.finish_reason for r in results}), "checked_against_plain": checked,
        "setup_seconds": {"write_folder": round(written, 1), "load": round(loaded, 1)},
    }


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--sizes", default="moondream2", choices=sorted(SIZES), help="layer sizes (the default is the benchmark's)")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--context", type=int, default=CONTEXT, help="tokens each request holds when decoding starts")
    parser.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="length of the timed prompt")
    parser.add_argument("--skip-points", action="store_true", help="only the default batch (no batch 1 / 64, no prefill)")
    parser.add_argument("--only-prefill", action="store_true", help="only the 2,048-token prefill (for profiling)")
    parser.add_argument("--peaks", action=argparse.BooleanOptionalAction, default=True,
                        help="also measure a plain read stream and a loop of matrix instructions on this GPU and report "
                             "against them (about 0.1 s; --no-peaks leaves it out)")
    parser.add_argument("--tune-linears", type=int, default=0,
                        help="with --workload: RuntimeConfig.tune_linears (time the vendor library's algorithms at warm-up)")
    parser.add_argument("--check", type=int, default=0,
                        help="with --workload: compare this many greedy requests with the plain implementation (for --layers 2)")
    parser.add_argument("--workload", default="decode", choices=["decode", "waves256", "mixed48", "compare-vimesun", "compare-bogivik", "compare-letevik", "compare-bokorax"],
                        help="decode: the benchmark's decode step (default); waves256 and mixed48 run requests through "
                             "InferenceEngine; compare-vimesun, compare-bogivik and compare-letevik measure that design beside the Moondream "
                             "decoder at equal sizes")
    parser.add_argument("--compare-sizes", default=None,
                        help="with --workload compare-*: which of its sizes, with commas between them "
                             "(default: all of them)")
    parser.add_argument("--compare-model", default="both", choices=["both", "vimesun", "bogivik", "letevik", "bokorax", "moondream2"],
                        help="with --workload compare-*: one of the two designs only (for profiling)")
    parser.add_argument("--compare-batches", default="1,8,64", help="with --workload compare-bogivik or compare-letevik: batch sizes of the decode steps")
    parser.add_argument("--skip-prefill", action="store_true", help="with --workload compare-bogivik or compare-letevik: decode steps only")
    parser.add_argument("--max-batch-size", type=int, default=None, help="for the workloads through the entry point")
    parser.add_argument("--linears", default="library", choices=["library", "own"],
                        help="linears of more than 64 rows (a prompt's): through hipBLASLt (the engine's default) or "
                             "through this package's tiled kernels only")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible")
        return 1
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from kestrel_amd.ops import fast

    fast.LIBRARY_LINEAR = args.linears == "library"
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    size = 2 if dtype == torch.bfloat16 else 4
    sizes = dict(SIZES[args.sizes])
    # a longer context than the model's own is measured with its position table made longer
    sizes["max_context"] = max(sizes["max_context"], args.context + max(args.steps, 16) + args.warmup + 8, args.prefill_tokens)
    if args.layers is None:
        args.layers = sizes["n_layers"]
    if args.workload == "compare-vimesun":
        args.compare_sizes = args.compare_sizes or ",".join(COMPARE_SIZES)
        print(json.dumps(run_compare(args, dtype, device)))
        return 0
    if args.workload == "compare-bogivik":
        print(json.dumps(run_compare_bogivik(args, dtype, device)))
        return 0
    if args.workload == "compare-bokorax":
        print(json.dumps(run_compare_bokorax(args, dtype, device)))
        return 0
    if args.workload == "compare-letevik":
        print(json.dumps(run_compare_letevik(args, dtype, device)))
        return 0
    if args.workload != "decode":
        print(json.dumps(run_workload(args, dict(SIZES[args.sizes]))))
        return 0
    net, typed = build_model(args.layers, dtype, device, sizes)
    weights = model_bytes(net, size)

    if args.only_prefill:
        seconds, best = time_prefill(net, typed, args.prefill_tokens)
        print(json.dumps({"prefill_ms": round(seconds * 1e3, 3), "best_ms": round(best * 1e3, 3), "tokens": args.prefill_tokens,
                          "dtype": args.dtype}))
        return 0
    elapsed, kv_bytes = time_decode(net, typed, args.batch, args.context, args.steps, args.warmup)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    step_bytes = weights + kv_bytes * (size / 2) + args.batch * typed.dim * size
    achieved = step_bytes / (elapsed / args.steps)
    record = {
        "metric": f"decode tok/s ({LABELS[args.sizes][0]}, batch {args.batch}, context {args.context})",
        "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random token ids and prefix embeddings, random weights N(0,0.02))",
        "config": {"model": LABELS[args.sizes][1], "n_layers": args.layers, "n_layers_full": sizes["n_layers"],
                   "dim": typed.dim, "ff_dim": typed.ff_dim, "n_heads": typed.n_heads, "n_kv_heads": typed.n_kv_heads,
                   "head_dim": typed.head_dim, "rotary_dim": typed.rotary_dim, "vocab_size": typed.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "prefix_attn": typed.prefix_attn,
                   "page_size": PAGE_SIZE, "parallelism": "single-gpu",
                   "prompt_linears": "hipblaslt" if args.linears == "library" else "own"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
    }
    if not args.skip_points:
        seconds, best = time_prefill(net, typed, args.prefill_tokens)         # the median of eight runs, and the best
        flops = prefill_flops(typed, args.prefill_tokens, min(typed.prefix_attn, args.prefill_tokens - 1))
        record["prefill"] = {"value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
                             "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
                             "best_ms": round(best * 1e3, 3)}
        points, detail = {}, {}
        for batch, steps in ((1, args.steps), (64, max(16, args.steps // 4))):
            e, kv = time_decode(net, typed, batch, args.context, steps, min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(batch * steps / e, 1)
            moved = weights + kv * (size / 2) + batch * typed.dim * size
            detail[f"decode_b{batch}"] = {"ms_per_step": round(e / steps * 1e3, 4), "steps": steps,
                                          "frac": round(moved / (e / steps) / PEAK_HBM, 4)}
        record["points"] = points
        record["points_detail"] = detail
    if args.peaks:
        from kestrel_amd.ops import core

        peaks = core.measured_peaks(device)
        record["roofline"]["peak_measured"] = round(peaks["hbm_read_gbs"], 1)
        record["roofline"]["frac_measured"] = round(achieved / 1e9 / peaks["hbm_read_gbs"], 4)
        if "prefill" in record and args.dtype == "bf16":
            record["prefill"]["peak_measured"] = round(peaks["mfma_bf16_tflops"], 1)
            record["prefill"]["frac_measured"] = round(flops / seconds / 1e12 / peaks["mfma_bf16_tflops"], 4)
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
