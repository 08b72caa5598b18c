"""Bokorax: a small decoder whose layers mix tokens by one of two kinds of attention or by a decaying matrix memory,
each followed by a routed mixture of experts, with the norms behind the sublayers.

The design, in this file's notation (``w`` the width, ``eps`` the one epsilon of all norms, ``rms(y) = y / sqrt(mean(y^2) + eps)``):

* ``x = embed[token] * embedding.scale``; a layer is ``x <- x + rms(mix(x)) (1 + norm1)``, then
  ``x <- x + rms(mlp(x)) (1 + norm2)``: the sublayers read the stream itself, the norm (its weight stored around zero) stands
  behind them; a layer whose ``mlp`` is null has the first half only. Logits are ``head(rms(x) (1 + final.norm)) * logit_scale``.
* Layer type ``attention``: ``heads`` query heads over ``kv_heads`` key heads of ``dim`` channels, no biases, no value
  projection: the values are the keys as projected. All queries of a token are normalised together, ``rms(W_q x) * q.norm`` over
  the whole projection, likewise the keys; then the first ``rot.dims`` channels of every head are rotated (channel ``i`` with
  ``i + dims / 2``, angle ``place * base^(-2i / dims)``). Score ``scale * (q . k)``; place ``i`` sees ``j`` with ``0 <= i - j < mask.size``
  (no ``mask``: every ``j <= i``); an ordinary softmax.
* Layer type ``attention_2``: projections of q, k and v (values of ``vdim`` channels); every query and key head normalised by
  itself with one gain of a head's size; the same rotation with every frequency divided by ``rot.scaling.factor``; score
  ``softcap * tanh(scale * (q . k) / softcap)``; every ``j <= i`` is seen; ``exp(sink_h)`` in the softmax's denominator, a learned
  number per head; head ``h``'s output times ``sigmoid(W_g x)_h``, one number per head. A layer that says ``kv_from: j`` has no key
  and value tensors and reads layer ``j``'s cached keys and values with its own queries.
* Layer type ``wkv``: the decaying matrix memory of ``parts/decayed_memory.py``.
* ``mlp`` (``kind`` ``moe``): the routed experts of ``parts/experts.py`` (silu), with ``router.identity`` identity experts,
  ``router.groups``, the weights times ``router.scale``, and a shared expert behind a gate of one number per token.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.registry import ModelSpec, register
from ..parts.specs import (AttentionSpec, DecayedMemorySpec, LayerSpec, LinearScaling, ModelPlan, NormSpec, PositionSpec, QKNorm,
                           RoutedExpertsSpec, ScheduleEntry)

NAME = "bokorax"
EXPERT_ACTIVATION = "silu"
NORM_OFFSET = 1.0                      # the layers' norms multiply by one plus the stored weight
# The design has no longest sequence of its own (no table depends on one). ``config.json`` may name a bound
# (``max_positions``); without one this stands, and the engine's ``max_seq_len`` narrows it.
DEFAULT_MAX_POSITIONS = 1 << 17


def _positive_int(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"config.json: {where} must be a positive integer, got {value!r}")
    return value


def _count(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ValueError(f"config.json: {where} must be a non-negative integer, got {value!r}")
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


@dataclass(frozen=True)
class BokoraxAttention:
    """Sizes of either kind of attention; what a kind does not have is ``None``."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    rot_factor: Optional[float] = None        # every frequency divided by it (``attention_2``)
    window: Optional[int] = None              # ``attention``
    softcap: Optional[float] = None           # ``attention_2``
    kv_from: Optional[int] = None             # ``attention_2``

    @classmethod
    def read(cls, where: str, m: dict, second: bool) -> "BokoraxAttention":
        _object(where, m, ("heads", "kv_heads", "dim", "scale", "rot"))
        heads, kv_heads = _positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.kv_heads", m["kv_heads"])
        if heads % kv_heads:
            raise ValueError(f"config.json: {where}: {heads} heads are no multiple of {kv_heads} kv_heads")
        dim = _positive_int(f"{where}.dim", m["dim"])
        vdim = _positive_int(f"{where}.vdim", m.get("vdim", dim))
        rot = _object(f"{where}.rot", m["rot"], ("base", "dims"))
        dims = _positive_int(f"{where}.rot.dims", rot["dims"])
        if dims % 2 or dims > dim:
            raise ValueError(f"config.json: {where}.rot.dims must be even and at most dim, got {dims}")
        common = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_number(f"{where}.scale", m["scale"]), rot_dims=dims,
                      rot_base=_number(f"{where}.rot.base", rot["base"]))
        if not second:
            if vdim != dim:
                raise ValueError(f"config.json: {where}: the values are the keys, vdim {vdim} must be dim {dim}")
            mask = m.get("mask")
            window = None if mask is None else _positive_int(f"{where}.mask.size", _object(f"{where}.mask", mask, ("size",))["size"])
            return cls(**common, window=window)
        factor = None
        if rot.get("scaling") is not None:
            factor = _number(f"{where}.rot.scaling.factor", _object(f"{where}.rot.scaling", rot["scaling"], ("factor",))["factor"])
            if not factor > 0:
                raise ValueError(f"config.json: {where}.rot.scaling.factor must be positive")
        cap = m.get("softcap")
        if cap is not None:
            cap = _number(f"{where}.softcap", cap)
            if not cap > 0:
                raise ValueError(f"config.json: {where}.softcap must be positive")
        source = m.get("kv_from")
        if source is not None:
            source = _count(f"{where}.kv_from", source)
        return cls(**common, rot_factor=factor, softcap=cap, kv_from=source)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                               "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.rot_factor is not None:
            out["rot"]["scaling"] = {"factor": self.rot_factor}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class BokoraxMemory:
    heads: int
    dim: int
    decay_rank: Optional[int] = None           # (not a key of the design: only the writer of random weights needs it)

    @classmethod
    def read(cls, where: str, m: dict) -> "BokoraxMemory":
        _object(where, m, ("heads", "dim"))
        rank = m.get("decay_rank")
        return cls(_positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.dim", m["dim"]),
                   None if rank is None else _positive_int(f"{where}.decay_rank", rank))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        return out


@dataclass(frozen=True)
class BokoraxExperts:
    experts: int
    ff: int
    top: int
    scale: float
    identity: int
    groups: Optional[Tuple[int, int]]          # (count, keep)
    shared_ff: Optional[int]

    @classmethod
    def read(cls, where: str, m: dict) -> "BokoraxExperts":
        if not isinstance(m, dict) or m.get("kind") != "moe":
            raise ValueError(f"config.json: {where} must be null or an object of kind 'moe'")
        _object(where, m, ("expert", "router"))
        ff = _positive_int(f"{where}.expert.ff", _object(f"{where}.expert", m["expert"], ("ff",))["ff"])
        r = _object(f"{where}.router", m["router"], ("experts", "top"))
        experts, top = _positive_int(f"{where}.router.experts", r["experts"]), _positive_int(f"{where}.router.top", r["top"])
        identity = _count(f"{where}.router.identity", r.get("identity", 0))
        groups = r.get("groups")
        if groups is not None:
            _object(f"{where}.router.groups", groups, ("count", "keep"))
            groups = (_positive_int(f"{where}.router.groups.count", groups["count"]), _positive_int(f"{where}.router.groups.keep", groups["keep"]))
            if (experts + identity) % groups[0] or groups[1] > groups[0]:
                raise ValueError(f"config.json: {where}.router.groups: {groups[0]} groups must divide the {experts + identity} router "
                                 f"outputs and hold the {groups[1]} that are kept")
        if top > experts + identity:
            raise ValueError(f"config.json: {where}.router.top {top} exceeds the {experts + identity} router outputs")
        shared = m.get("shared")
        shared_ff = None if shared is None else _positive_int(f"{where}.shared.ff", _object(f"{where}.shared", shared, ("ff",))["ff"])
        return cls(experts, ff, top, _number(f"{where}.router.scale", r.get("scale", 1.0)), identity, groups, shared_ff)

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top, "scale": self.scale, "identity": self.identity}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class BokoraxLayer:
    kind: str                                  # "attention", "attention_2" or "wkv"
    attention: Optional[BokoraxAttention]
    memory: Optional[BokoraxMemory]
    mlp: Optional[BokoraxExperts]


KINDS = ("attention", "attention_2", "wkv")


@dataclass(frozen=True)
class BokoraxConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    logit_scale: float
    max_positions: int
    layers: Tuple[BokoraxLayer, ...]
    raw: Any = None

    @classmethod
    def from_dict(cls, config: Dict[str, Any]) -> "BokoraxConfig":
        for key in ("layers", "vocab", "width", "norm"):
            if key not in config:
                raise ValueError(f"config.json: key {key!r} missing")
        eps = _number("norm.eps", _object("norm", config["norm"], ("eps",))["eps"])
        if not eps >= 0:
            raise ValueError("config.json: norm.eps must not be negative")
        listed = config["layers"]
        if not isinstance(listed, list) or not listed:
            raise ValueError("config.json: 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            _object(where, entry, ("type", "mixer"))
            kind = entry["type"]
            mixer = _object(f"{where}.mixer", entry["mixer"])
            if kind not in KINDS:
                raise ValueError(f"config.json: {where}.type is {kind!r}; this design has the mixers {', '.join(KINDS)}")
            attention = memory = None
            if kind == "wkv":
                memory = BokoraxMemory.read(f"{where}.mixer", mixer)
            else:
                attention = BokoraxAttention.read(f"{where}.mixer", mixer, second=kind == "attention_2")
            mlp = entry.get("mlp")
            layers.append(BokoraxLayer(kind, attention, memory, None if mlp is None else BokoraxExperts.read(f"{where}.mlp", mlp)))
        for i, layer in enumerate(layers):
            a = layer.attention
            if a is None or a.kv_from is None:
                continue
            j = a.kv_from
            owner = layers[j].attention if j < i and layers[j].kind == "attention_2" else None
            if owner is None or owner.kv_from is not None:
                raise ValueError(f"config.json: layers[{i}].mixer.kv_from names layer {j}, which is no earlier attention_2 layer with "
                                 f"keys and values of its own")
            if (owner.kv_heads, owner.dim, owner.vdim) != (a.kv_heads, a.dim, a.vdim):
                raise ValueError(f"config.json: layers[{i}] reads the keys and values of layer {j}, whose sizes differ")
        embedding = config.get("embedding") or {}
        positions = config.get("max_positions", DEFAULT_MAX_POSITIONS)
        return cls(vocab=_positive_int("vocab", config["vocab"]), width=_positive_int("width", config["width"]), eps=eps,
                   embedding_scale=_number("embedding.scale", _object("embedding", embedding).get("scale", 1.0)),
                   logit_scale=_number("logit_scale", config.get("logit_scale", 1.0)),
                   max_positions=_positive_int("max_positions", positions), layers=tuple(layers), raw=config)

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"type": layer.kind, "mixer": (layer.memory if layer.kind == "wkv" else layer.attention).to_dict(),
                   "mlp": None if layer.mlp is None else layer.mlp.to_dict()} for layer in self.layers]
        out = {"architecture": "Bokorax", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale, "layers": layers}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out


def _mixer(cfg: BokoraxConfig, i: int, layer: BokoraxLayer, names: Dict[str, str]):
    p = f"l{i}.mix."
    if layer.kind == "wkv":
        m = layer.memory
        names.update({f"mixer.mu.{s}": p + "mu." + s for s in "rkvgw"})
        names.update({f"mixer.{s}.weight": p + s for s in ("r", "k", "v", "g")})
        names.update({"mixer.w1.weight": p + "w1", "mixer.w2.weight": p + "w2", "mixer.w0": p + "w0", "mixer.u": p + "u",
                      "mixer.norm.weight": p + "norm", "mixer.proj.weight": p + "o"})
        return DecayedMemorySpec("decayed_memory", cfg.width, m.heads, m.dim, cfg.eps, decay_rank=m.decay_rank)
    a = layer.attention
    names.update({"mixer.q.weight": p + "q", "mixer.proj.weight": p + "o", "mixer.q_norm.weight": p + "q.norm"})
    if a.kv_from is None:
        names.update({"mixer.k.weight": p + "k", "mixer.k_norm.weight": p + "k.norm"})
    if layer.kind == "attention":
        rotation = PositionSpec("rotary", rotary_dim=a.rot_dims, theta=a.rot_base, pairing="halves")
        return AttentionSpec("attention", cfg.width, a.heads, a.kv_heads, a.dim, rotation, bias=False, scale=a.scale, window=a.window,
                             split_projections=True, qk_norm=QKNorm("projection", cfg.eps), values_from_keys=True)
    if a.kv_from is None:
        names["mixer.v.weight"] = p + "v"
    names.update({"mixer.gate.weight": p + "g", "mixer.sinks": p + "sink"})
    rotation = PositionSpec("rotary", rotary_dim=a.rot_dims, theta=a.rot_base, pairing="halves",
                            scaling=None if a.rot_factor is None else LinearScaling(a.rot_factor))
    return AttentionSpec("attention", cfg.width, a.heads, a.kv_heads, a.dim, rotation, bias=False, scale=a.scale, value_dim=a.vdim,
                         split_projections=True, qk_norm=QKNorm("head", cfg.eps), output_gate=True, gate_per_head=True,
                         softcap=a.softcap, head_sinks=True, shares_kv=a.kv_from is not None)


def build_plan(cfg: BokoraxConfig) -> ModelPlan:
    layers = []
    schedule = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        names = {"norm.weight": p + "norm1"}
        mixer = _mixer(cfg, i, layer, names)
        feed_forward = norm2 = None
        if layer.mlp is not None:
            e = layer.mlp
            feed_forward = RoutedExpertsSpec("routed_experts", cfg.width, e.experts, e.ff, e.top, scale=e.scale, n_identity=e.identity,
                                             n_groups=e.groups[0] if e.groups else 0, keep_groups=e.groups[1] if e.groups else 0,
                                             activation=EXPERT_ACTIVATION, shared_hidden=e.shared_ff, shared_gate=True)
            for j in range(e.experts):
                names.update({f"feed_forward.e{j}.{s}.weight": f"{p}mlp.e{j}.{s}" for s in ("gate", "up", "down")})
            names.update({"feed_forward.router.weight": p + "mlp.router", "feed_forward.correction": p + "mlp.correction"})
            if e.shared_ff is not None:
                names.update({f"feed_forward.shared.{s}.weight": f"{p}mlp.shared.{s}" for s in ("gate", "up", "down", "sg")})
            norm2 = NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False, offset=NORM_OFFSET)
            names["norm2.weight"] = p + "norm2"
        layers.append(LayerSpec(arrangement="output_norms", norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False, offset=NORM_OFFSET),
                                mixer=mixer, feed_forward=feed_forward, norm2=norm2, names=names))
        source = layer.attention.kv_from if layer.attention is not None else None
        schedule.append(ScheduleEntry(i, reads_cache_of=source))
    return ModelPlan(
        architecture=NAME, vocab_size=cfg.vocab, dim=cfg.width, max_positions=cfg.max_positions, layers=tuple(layers),
        schedule=tuple(schedule), final_norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False, offset=NORM_OFFSET),
        head_bias=False, tied_head=False, names={"embedding": "embed", "final_norm.weight": "final.norm", "head.weight": "head"},
        embedding_scale=cfg.embedding_scale, logit_scale=cfg.logit_scale,
    )


def _claims(config: Dict[str, Any]) -> bool:
    layers = config.get("layers")
    return isinstance(layers, list) and bool(layers) and "width" in config and \
        all(isinstance(e, dict) and e.get("type") in KINDS and "mixer" in e for e in layers) and \
        any(e.get("type") in ("wkv", "attention_2") for e in layers)


register(ModelSpec(
    name=NAME,
    read_config=BokoraxConfig.from_dict,
    build_plan=build_plan,
    aliases=("Bokorax",),
    claims=_claims,
    filename="model.safetensors",
))
