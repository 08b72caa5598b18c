"""Letevik: a small decoder with a token-pair embedding, a looped stretch of layers, and two kinds of attention:
differential attention behind short convolutions with a window that keeps the first tokens, and latent attention with a
per-head sink and an output gate.

The design, in this file's notation (``w`` the width, ``eps`` the one epsilon of all norms, ``rms(x) = x / sqrt(mean(x^2) + eps)``):

* ``x = embed[token] + bigram[r]`` with ``r = (previous token * mul_prev + token * mul_cur) mod buckets`` and ``r = buckets``
  (the table's last row) for the first token of a sequence.
* The layers ``start .. stop - 1`` of ``loop`` run ``times`` times in a row with the same weights and a cache of their own
  each time; every such pass begins with ``x <- x + loop.step[pass]``.
* A layer: ``x <- x + mix(rms(x) norm1)``, then ``x <- x + mlp(rms(x) norm2)``; a layer whose ``mlp`` is null has the first half only.
* Layer type ``attention``: ``parts/differential_attention.py`` with a convolution of ``conv`` taps, an interleaved rotation
  of the first ``rot.dims`` channels of every map, and the mask ``i - j < mask.size or j < mask.keep_first``.
* Layer type ``latent_attention``: ``parts/latent_attention.py``; the ``rot_dim`` part is rotated by halves.
* ``mlp`` (``kind`` ``dense``): ``down(g sigmoid(1.702 g) (u + 1))`` with ``g = min(gate h, limit)``, ``u = clamp(up h, -limit, limit)``.
* Logits: ``embed (rms(x) final.norm)``: the head is the embedding table.

Every size and constant above that is not a literal comes from ``config.json`` or from a tensor's shape. Tensor names:
``embed``, ``bigram``, ``loop.step``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{q,k,v,o}``, ``l<i>.mix.{q,k,v}.conv``,
``l<i>.mix.{lq1,lk1,lq2,lk2}``, ``l<i>.mix.{dq,uq,dkv,uk,uv,g,sink}``, ``l<i>.mix.{dq,dkv}.norm``, ``l<i>.mlp.{gate,up,down}``,
``final.norm``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.registry import ModelSpec, register
from ..parts.specs import (ClampedGatedFeedForwardSpec, DifferentialAttentionSpec, LatentAttentionSpec, LayerSpec, ModelPlan, NormSpec,
                           PairEmbeddingSpec, PassVectorSpec, PositionSpec, ScheduleEntry, WindowWithKeptFirst)

NAME = "letevik"
GATE_SLOPE = 1.702             # the feed-forward's gate is g * sigmoid(1.702 g)
VALUE_SHIFT = 1.0              # and multiplies u + 1
DIFFERENTIAL_PAIRING = "interleaved"
LATENT_PAIRING = "halves"
# The design has no longest sequence of its own (angles are computed, no table depends on one). ``config.json`` may name a
# bound (``max_positions``); without one this stands, and the engine's ``max_seq_len`` narrows it.
DEFAULT_MAX_POSITIONS = 1 << 17


def _positive_int(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"config.json: {where} must be a positive integer, got {value!r}")
    return value


def _natural(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ValueError(f"config.json: {where} must be an integer that is not negative, got {value!r}")
    return value


def _number(where: str, value) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ValueError(f"config.json: {where} must be a number, got {value!r}")
    return float(value)


def _object(where: str, value, keys=()) -> dict:
    if not isinstance(value, dict):
        raise ValueError(f"config.json: {where} must be an object")
    for key in keys:
        if key not in value:
            raise ValueError(f"config.json: {where}.{key} missing")
    return value


def _rotation(where: str, m: dict, most: int) -> Tuple[int, float]:
    rot = _object(f"{where}.rot", m.get("rot"), ("base", "dims"))
    dims = _positive_int(f"{where}.rot.dims", rot["dims"])
    if dims % 2 or dims > most:
        raise ValueError(f"config.json: {where}.rot.dims must be even and at most {most}, got {dims}")
    return dims, _number(f"{where}.rot.base", rot["base"])


@dataclass(frozen=True)
class LetevikDifferential:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: Optional[int]
    window: Optional[int]
    keep_first: int
    rot_dims: int
    rot_base: float

    @classmethod
    def read(cls, where: str, m: dict) -> "LetevikDifferential":
        _object(where, m, ("heads", "kv_heads", "dim", "vdim", "scale", "diff"))
        heads, kv_heads = _positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.kv_heads", m["kv_heads"])
        if heads % kv_heads:
            raise ValueError(f"config.json: {where}: {heads} heads are no multiple of {kv_heads} kv_heads")
        dim = _positive_int(f"{where}.dim", m["dim"])
        window, keep_first = None, 0
        if m.get("mask") is not None:
            mask = _object(f"{where}.mask", m["mask"], ("size",))
            window = _positive_int(f"{where}.mask.size", mask["size"])
            keep_first = _natural(f"{where}.mask.keep_first", mask.get("keep_first", 0))
        conv = m.get("conv")
        if conv is not None:
            conv = _positive_int(f"{where}.conv", conv)
        rot_dims, rot_base = _rotation(where, m, dim)
        return cls(heads, kv_heads, dim, _positive_int(f"{where}.vdim", m["vdim"]), _number(f"{where}.scale", m["scale"]),
                   _number(f"{where}.diff", m["diff"]), conv, window, keep_first, rot_dims, rot_base)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                               "diff": self.diff, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.conv is not None:
            out["conv"] = self.conv
        if self.window is not None:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out


@dataclass(frozen=True)
class LetevikLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_dims: int
    rot_base: float

    @classmethod
    def read(cls, where: str, m: dict) -> "LetevikLatent":
        _object(where, m, ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale"))
        rot_dim = _positive_int(f"{where}.rot_dim", m["rot_dim"])
        rot_dims, rot_base = _rotation(where, m, rot_dim)
        return cls(_positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.dim", m["dim"]), rot_dim,
                   _positive_int(f"{where}.vdim", m["vdim"]), _positive_int(f"{where}.q_rank", m["q_rank"]),
                   _positive_int(f"{where}.kv_rank", m["kv_rank"]), _number(f"{where}.scale", m["scale"]), rot_dims, rot_base)

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class LetevikLayer:
    kind: str                                  # "attention" or "latent_attention"
    mixer: Any                                 # LetevikDifferential or LetevikLatent
    ff: Optional[int]                          # hidden size of the feed-forward; None: the layer has none
    limit: Optional[float]                     # its clamp


@dataclass(frozen=True)
class LetevikConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: Tuple[LetevikLayer, ...]
    loop_start: int
    loop_stop: int
    loop_times: Optional[int]          # None: no stretch of layers is repeated and there is no ``loop.step``
    raw: Any = None

    @classmethod
    def from_dict(cls, config: Dict[str, Any]) -> "LetevikConfig":
        for key in ("layers", "vocab", "width", "norm", "embedding"):
            if key not in config:
                raise ValueError(f"config.json: key {key!r} missing")
        eps = _number("norm.eps", _object("norm", config["norm"], ("eps",))["eps"])
        if not eps >= 0:
            raise ValueError("config.json: norm.eps must not be negative")
        bigram = _object("embedding.bigram", _object("embedding", config["embedding"], ("bigram",))["bigram"],
                         ("buckets", "mul_prev", "mul_cur"))
        listed = config["layers"]
        if not isinstance(listed, list) or not listed:
            raise ValueError("config.json: 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            _object(where, entry, ("type", "mixer"))
            kind = entry["type"]
            mixer = _object(f"{where}.mixer", entry["mixer"])
            if kind == "attention":
                mixer = LetevikDifferential.read(f"{where}.mixer", mixer)
            elif kind == "latent_attention":
                mixer = LetevikLatent.read(f"{where}.mixer", mixer)
            else:
                raise ValueError(f"config.json: {where}.type is {kind!r}; this design has the mixers 'attention' and 'latent_attention'")
            mlp = entry.get("mlp")
            ff = limit = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ValueError(f"config.json: {where}.mlp must be null or an object of kind 'dense'")
                ff = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
                limit = _number(f"{where}.mlp.limit", mlp.get("limit"))
                if not limit > 0:
                    raise ValueError(f"config.json: {where}.mlp.limit must be positive")
            layers.append(LetevikLayer(kind, mixer, ff, limit))
        loop = config.get("loop")
        start = stop = 0
        times = None
        if loop is not None:
            _object("loop", loop, ("start", "stop", "times"))
            start, stop, times = (_natural(f"loop.{key}", loop[key]) for key in ("start", "stop", "times"))
            if not start <= stop <= len(layers):
                raise ValueError(f"config.json: loop {start} .. {stop} does not lie within the {len(layers)} layers")
        positions = config.get("max_positions", DEFAULT_MAX_POSITIONS)
        return cls(vocab=_positive_int("vocab", config["vocab"]), width=_positive_int("width", config["width"]), eps=eps,
                   max_positions=_positive_int("max_positions", positions),
                   buckets=_positive_int("embedding.bigram.buckets", bigram["buckets"]),
                   mul_prev=_natural("embedding.bigram.mul_prev", bigram["mul_prev"]),
                   mul_cur=_natural("embedding.bigram.mul_cur", bigram["mul_cur"]), layers=tuple(layers),
                   loop_start=start, loop_stop=stop, loop_times=times, raw=config)

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"type": layer.kind, "mixer": layer.mixer.to_dict(),
                   "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff, "limit": layer.limit}} for layer in self.layers]
        out = {"architecture": "Letevik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "embedding": {"bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur}}, "layers": layers}
        if self.loop_times is not None:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out


def build_plan(cfg: LetevikConfig) -> ModelPlan:
    layers = []
    ignored = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        names = {"norm.weight": p + "norm1"}
        x = p + "mix."
        if layer.kind == "attention":
            mixer = DifferentialAttentionSpec(
                "differential_attention", cfg.width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.diff, cfg.eps,
                PositionSpec("rotary", rotary_dim=m.rot_dims, theta=m.rot_base, pairing=DIFFERENTIAL_PAIRING), conv_taps=m.conv,
                mask=WindowWithKeptFirst(m.window, m.keep_first) if m.window is not None else None)
            names.update({"mixer.q.weight": x + "q", "mixer.k.weight": x + "k", "mixer.v.weight": x + "v", "mixer.proj.weight": x + "o",
                          "mixer.lq1": x + "lq1", "mixer.lk1": x + "lk1", "mixer.lq2": x + "lq2", "mixer.lk2": x + "lk2"})
            if m.conv is not None:
                names.update({"mixer.q.conv": x + "q.conv", "mixer.k.conv": x + "k.conv", "mixer.v.conv": x + "v.conv"})
        else:
            mixer = LatentAttentionSpec(
                "latent_attention", cfg.width, m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank, m.scale, cfg.eps,
                PositionSpec("rotary", rotary_dim=m.rot_dims, theta=m.rot_base, pairing=LATENT_PAIRING))
            names.update({"mixer.dq.weight": x + "dq", "mixer.dq_norm.weight": x + "dq.norm", "mixer.uq.weight": x + "uq",
                          "mixer.dkv.weight": x + "dkv", "mixer.dkv_norm.weight": x + "dkv.norm", "mixer.uk.weight": x + "uk",
                          "mixer.uv.weight": x + "uv", "mixer.sink": x + "sink", "mixer.gate.weight": x + "g",
                          "mixer.proj.weight": x + "o"})
        feed_forward = norm2 = None
        if layer.ff is not None:
            feed_forward = ClampedGatedFeedForwardSpec("clamped_gated_dense", cfg.width, layer.ff, layer.limit, GATE_SLOPE, VALUE_SHIFT)
            norm2 = NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False)
            names.update({"norm2.weight": p + "norm2", "feed_forward.gate.weight": p + "mlp.gate", "feed_forward.up.weight": p + "mlp.up",
                          "feed_forward.down.weight": p + "mlp.down"})
        else:
            ignored.append(p + "norm2")        # (a layer without a feed-forward has no use for a second norm)
        layers.append(LayerSpec(arrangement="sequential", norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False), mixer=mixer,
                                feed_forward=feed_forward, norm2=norm2, names=names))
    names = {"embedding": "embed", "position.table": "bigram", "final_norm.weight": "final.norm"}
    if cfg.loop_times is None:
        schedule = [ScheduleEntry(i) for i in range(len(cfg.layers))]
        ignored.append("loop.step")
        junctions = {}
    else:
        schedule = [ScheduleEntry(i) for i in range(cfg.loop_start)]
        for t in range(cfg.loop_times):
            # every pass keeps a cache of its own and begins at the junction, with the pass's own vector
            schedule += [ScheduleEntry(i, before="loop_step" if i == cfg.loop_start else None, passage=t)
                         for i in range(cfg.loop_start, cfg.loop_stop)]
        schedule += [ScheduleEntry(i) for i in range(cfg.loop_stop, len(cfg.layers))]
        if cfg.loop_times > 0 and cfg.loop_stop > cfg.loop_start:
            junctions = {"loop_step": PassVectorSpec("pass_vector", cfg.width, cfg.loop_times)}
            names["junction.loop_step.steps"] = "loop.step"
        else:
            junctions = {}
            ignored.append("loop.step")
        if cfg.loop_times == 0:
            # (layers that never run own no tensors the model needs)
            ignored.extend(f"l{i}." for i in range(cfg.loop_start, cfg.loop_stop))
    return ModelPlan(
        architecture=NAME, vocab_size=cfg.vocab, dim=cfg.width, max_positions=cfg.max_positions, layers=tuple(layers),
        schedule=tuple(schedule), final_norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False), head_bias=False, tied_head=True,
        names=names, position=PairEmbeddingSpec("pair_embedding", cfg.width, cfg.buckets, cfg.mul_prev, cfg.mul_cur, cfg.vocab),
        junctions=junctions, ignored_prefixes=tuple(ignored),
    )


def _claims(config: Dict[str, Any]) -> bool:
    layers = config.get("layers")
    return isinstance(layers, list) and bool(layers) and "width" in config and "residual_mult" not in config and \
        isinstance(config.get("embedding"), dict) and "bigram" in config["embedding"] and \
        all(isinstance(e, dict) and e.get("type") in ("attention", "latent_attention") and "mixer" in e for e in layers)


register(ModelSpec(
    name=NAME,
    read_config=LetevikConfig.from_dict,
    build_plan=build_plan,
    aliases=("Letevik",),
    claims=_claims,
    filename="model.safetensors",
))
