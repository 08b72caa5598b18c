"""Attention over the paged cache with a fused q|k|v projection."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.attention import paged_attention
from ..ops.linear import linear
from .base import LayerCache, Mixer, build_part, register_mixer
from .specs import AttentionSpec, CacheSpec, ParamSpec


class PagedAttention(Mixer):
    """``proj(softmax(q k^T scale + mask) v)`` with grouped kv heads.

    One linear gives ``[q (H hd) | k (Hkv hd) | v (Hkv hd)]`` per token
    (``kestrel/models/moondream/text.py:101-121``); the position encoding is applied to
    q and k, k and v go into the paged cache first and attention then reads the cache
    (``text.py:123-135``); query head ``h`` reads kv head ``h // (H / Hkv)``; the scale is
    ``hd ** -0.5`` unless given (``text.py:158-185``); the output projection adds into the
    residual (``text.py:187-193``). Which keys a token sees comes with the batch
    (``kv_hi``, and the group's ``kv_lo`` for a window).

    Positions: the part built from ``spec.position`` is asked for a ``Rotation`` (a cos|sin table
    and the pairing of channels); ``None`` means q and k go into attention as they are. Nothing
    else is understood here: an encoding that needs more (several axes, a learned table added to
    the input) is refused when the weights are bound, not silently turned the rotary way.

    Further forms, each switched on by its field of the specification and all of them together or alone:
    values of another size than keys (``value_dim``: the cache's value pages and the output projection follow);
    queries and keys divided head by head by their root mean square before the scores (``qk_unit_norm_eps``);
    scores lowered by a head's slope times the distance ``i - j`` between query and key (``distance_slopes``);
    a term in the softmax's denominator that has a score but no value (``sink``), so that a query may attend to
    nothing; the three projections stored as three tensors (``split_projections``). With any of the middle four
    the mixer takes no rotation, and runs through kernels of its own (``ops.core.unit_norm_cache`` and the
    attention kernels that know these terms).

    A third family of forms is made ready by one kernel (``ops.core.qkv_prepare``: norm, rotation, factor, blend and cache
    write in one pass over the projected rows), again each by its field and in any combination: queries and keys
    normalised with learned gains over a head or over the whole projection (``qk_norm``); a rotation given by
    frequencies, with either pairing of channels (a position encoding that offers ``Rotation.frequencies``); queries
    times a factor that grows with the place (``query_growth``); a learned bias per bucket of distance and head
    (``distance_buckets``, tensor ``rel``, turned into a table by distance when the weights are bound); values blended
    with those of another layer of the same step (``value_blend``, tensor ``vmix``); the heads multiplied by the sigmoid
    of a further projection of the input before the output projection (``output_gate``, tensor ``gate.weight``, which
    rides in the launch of the q|k|v projection). ``chunk`` is a mask like ``window``: it only changes which keys a
    token reads (``kv_lo``) and which pages go back.

    And four more, again by their fields: values that are the keys as projected (``values_from_keys``: no value
    projection, the prepare kernel writes the unnormalised, unrotated keys into the value pages); scores capped by
    ``softcap * tanh(score / softcap)``; a learned sink score per head (``head_sinks``, tensor ``sinks``); a gate of one
    number per head (``gate_per_head``); and a layer without keys and values of its own (``shares_kv``: it projects
    queries, and the gate, alone, and its schedule entry reads another entry's cache).
    """

    replays_every_step = True

    def __init__(self, spec: AttentionSpec) -> None:
        super().__init__(spec)
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} query heads cannot share {spec.n_kv_heads} kv heads")
        self.position = build_part("position", spec.position)
        self.scale = float(spec.scale) if spec.scale is not None else float(spec.head_dim) ** -0.5
        self.value_dim = int(spec.head_dim if getattr(spec, "value_dim", None) is None else spec.value_dim)
        self.shares_kv = bool(getattr(spec, "shares_kv", False))
        self.values_from_keys = bool(getattr(spec, "values_from_keys", False))
        if self.values_from_keys and self.value_dim != spec.head_dim:
            raise ValueError("values that are the keys have the keys' size")
        self.q_dim = spec.n_heads * spec.head_dim
        self.kv_dim = 0 if self.shares_kv else spec.n_kv_heads * spec.head_dim
        self.v_dim = 0 if (self.shares_kv or self.values_from_keys) else spec.n_kv_heads * self.value_dim
        self.qkv_dim = self.q_dim + self.kv_dim + self.v_dim
        self.out_dim = spec.n_heads * self.value_dim
        self.softcap = getattr(spec, "softcap", None)
        self.head_sinks = bool(getattr(spec, "head_sinks", False))
        self.gate_per_head = bool(getattr(spec, "gate_per_head", False))
        self._sinks: Optional[torch.Tensor] = None
        self.unit_norm_eps = getattr(spec, "qk_unit_norm_eps", None)
        self.sink = getattr(spec, "sink", None)
        self.distance = getattr(spec, "distance_slopes", None)
        # the forms that the kernels of the rotary path know nothing of
        self.qk_norm = getattr(spec, "qk_norm", None)
        self.growth = getattr(spec, "query_growth", None)
        self.buckets = getattr(spec, "distance_buckets", None)
        self.blend = getattr(spec, "value_blend", None)
        self.gated = bool(getattr(spec, "output_gate", False))
        if self.qk_norm is not None and (self.qk_norm.scope not in ("head", "projection") or self.unit_norm_eps is not None):
            raise ValueError("qk_norm takes the scope 'head' or 'projection' and stands instead of qk_unit_norm_eps")
        if self.blend is not None and self.blend.role not in ("source", "blend"):
            raise ValueError(f"a value blend has the role 'source' or 'blend', got {self.blend.role!r}")
        self.extended = self.value_dim != spec.head_dim or self.unit_norm_eps is not None or self.sink is not None \
            or self.distance is not None or self.buckets is not None or self.softcap is not None or self.head_sinks \
            or (self.gated and self.gate_per_head)
        # the forms that ``ops.core.qkv_prepare`` makes ready (a rotation by frequencies, found when the weights are bound, too)
        self.prepared = self.qk_norm is not None or self.growth is not None or self.buckets is not None \
            or self.blend is not None or self.gated or self.shares_kv or self.values_from_keys or self.softcap is not None \
            or self.head_sinks
        if (self.shares_kv or self.values_from_keys) and (self.unit_norm_eps is not None or self.blend is not None):
            raise ValueError("a layer without values of its own takes neither unit-norm keys nor blended values")
        if self.head_sinks and self.sink is not None:
            raise ValueError("a sink is one number (sink) or one per head (head_sinks), not both")
        self.gate_dim = (spec.n_heads if self.gate_per_head else self.out_dim) if self.gated else 0
        self.in_dim = self.qkv_dim + self.gate_dim
        self._slopes: Optional[torch.Tensor] = None
        self._bias_table: Optional[torch.Tensor] = None
        self._q_gain = self._k_gain = self._blend_weight = self._freqs = None
        self.qkv_weight = self.qkv_bias = self.proj_weight = self.proj_bias = None
        self.dtype: Optional[torch.dtype] = None
        self._table = None
        self._pairing = "halves"

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        pieces = {name: rows for name, rows in (("q", self.q_dim), ("k", self.kv_dim), ("v", self.v_dim)) if rows} \
            if getattr(spec, "split_projections", False) else {"qkv": self.qkv_dim}
        out = {f"{name}.weight": ParamSpec((rows, spec.dim)) for name, rows in pieces.items()}
        out["proj.weight"] = ParamSpec((spec.dim, self.out_dim))
        if self.gated:
            out["gate.weight"] = ParamSpec((self.gate_dim, spec.dim))
        if self.qk_norm is not None and self.qk_norm.gain:
            per_head = self.qk_norm.scope == "head"
            out["q_norm.weight"] = ParamSpec((spec.head_dim if per_head else self.q_dim,), "vector", "gain")
            if not self.shares_kv:
                out["k_norm.weight"] = ParamSpec((spec.head_dim if per_head else self.kv_dim,), "vector", "gain")
        if self.head_sinks:
            out["sinks"] = ParamSpec((spec.n_heads,), "vector", "bias")
        if self.buckets is not None:
            out["rel"] = ParamSpec((-1 if self.buckets.buckets is None else self.buckets.buckets, spec.n_heads), "matrix", "bias")
        if self.blend is not None:
            out["vmix"] = ParamSpec((), "vector", "fraction")
        if spec.bias:
            out.update({f"{name}.bias": ParamSpec((rows,), "vector", "bias") for name, rows in pieces.items()})
            out["proj.bias"] = ParamSpec((spec.dim,), "vector", "bias")
        return out

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window,
                         self.value_dim if self.value_dim != self.spec.head_dim else None, getattr(self.spec, "chunk", None))

    def bind(self, tensors, dtype, device) -> None:
        spec = self.spec
        self.dtype = dtype
        split = getattr(spec, "split_projections", False)

        def fused(what: str) -> torch.Tensor:
            # (rows of q, then k, then v: the order of a fused projection's outputs)
            if split:
                return torch.cat([tensors[f"{name}.{what}"].to(device) for name in ("q", "k", "v") if f"{name}.{what}" in tensors], dim=0)
            return tensors[f"qkv.{what}"].to(device)

        self.qkv_weight = fused("weight").contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()
        if self.spec.bias:
            self.qkv_bias = fused("bias").to(dtype=torch.float32).contiguous()
            self.proj_bias = tensors["proj.bias"].to(device=device, dtype=torch.float32).contiguous()
        if self.gated:
            # the gate's rows behind those of q, k and v: one launch projects all four (the gate has no bias)
            self.qkv_weight = torch.cat([self.qkv_weight, tensors["gate.weight"].to(device)], dim=0).contiguous()
            if self.qkv_bias is not None:
                self.qkv_bias = torch.cat([self.qkv_bias, torch.zeros(self.gate_dim, dtype=torch.float32, device=device)]).contiguous()
        if self.qk_norm is not None and self.qk_norm.gain:
            self._q_gain = tensors["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            if not self.shares_kv:
                self._k_gain = tensors["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        if self.head_sinks:
            self._sinks = tensors["sinks"].to(device=device, dtype=torch.float32).contiguous()
        if self.buckets is not None:
            # rel [buckets, H] -> the bias by distance [H, distances]: the kernels look a distance up, not its bucket
            buckets = self.buckets.sized(tensors["rel"].shape[0])
            index = torch.tensor([buckets.bucket(n) for n in range(buckets.distances())], dtype=torch.long, device=device)
            self._bias_table = tensors["rel"].to(device=device, dtype=torch.float32)[index].t().contiguous()
        if self.blend is not None:
            self._blend_weight = tensors["vmix"].to(device=device, dtype=torch.float32).reshape(1).contiguous()
        if self.distance is not None:
            self._slopes = torch.tensor(self.distance.values(spec.n_heads), dtype=torch.float32, device=device)
        if int(getattr(self.position, "axes", 1)) != 1:
            raise ValueError(f"attention rotates by a token's place in the sequence; the position encoding "
                             f"{getattr(spec.position, 'kind', '?')!r} takes {self.position.axes} numbers per token")
        rotation = self.position.rotation(device)
        if rotation is None and callable(getattr(self.position, "table", None)) and self.position.table(device) is not None:
            raise ValueError(f"the position encoding {getattr(spec.position, 'kind', '?')!r} holds a table but offers no "
                             f"rotation(): attention would not know which channels to pair")
        if rotation is not None and getattr(rotation, "frequencies", None) is not None:
            freqs = rotation.frequencies
            if rotation.pairing not in core.ROTARY_PAIRINGS:
                raise ValueError(f"attention cannot apply a rotation with pairing {rotation.pairing!r}; known: "
                                 f"{', '.join(sorted(core.ROTARY_PAIRINGS))}")
            if freqs.dtype != torch.float32 or freqs.dim() != 1 or 2 * freqs.numel() > spec.head_dim:
                raise ValueError(f"a rotation's frequencies must be fp32 [R / 2] with R at most the head size {spec.head_dim}")
            if self.unit_norm_eps is not None or self.sink is not None or self.distance is not None:
                raise ValueError("attention with unit-norm queries and keys, distance slopes or a one-number sink takes no rotation")
            self._freqs, self._pairing, self._table = freqs.to(device).contiguous(), rotation.pairing, None
            self.prepared = True
        elif rotation is not None:
            table = rotation.table
            if rotation.pairing not in core.ROTARY_PAIRINGS:
                raise ValueError(f"attention cannot apply a rotation with pairing {rotation.pairing!r}; known: "
                                 f"{', '.join(sorted(core.ROTARY_PAIRINGS))}")
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] % 2 or table.shape[1] > self.spec.head_dim:
                raise ValueError(f"a rotation's table must be fp32 [positions, R] with R even and at most the head size "
                                 f"{self.spec.head_dim}, got {tuple(table.shape)} {table.dtype}")
            if self.extended or self.prepared:
                raise ValueError("attention with values of another size, normalised queries and keys, a distance bias, a sink, "
                                 "blended values or an output gate takes no rotation from a table (one from frequencies it does)")
            self._table, self._pairing = table.to(device).contiguous(), rotation.pairing
        else:
            self._table, self._pairing = None, "halves"

    def query_tile(self) -> Optional[int]:
        if self.dtype != torch.bfloat16:
            return None                     # the generic kernel takes tokens one by one
        from ..ops import fast
        if self.extended:
            return fast.biased_query_block(self.spec.head_dim, self.value_dim)
        return fast.prefill_query_block(self.spec.head_dim)

    # The three stages are also offered one by one, so that a block may fuse the first with its
    # norm and the last with its feed-forward (see ``Mixer.input_projection``).
    def input_projection(self):
        return self.qkv_weight, self.qkv_bias, self.in_dim

    def output_projection(self):
        return self.proj_weight, self.proj_bias

    def _decodes_fused(self, batch, cache: LayerCache) -> bool:
        """One token per row in bf16 with a rotation by halves: the decode kernel then rotates q and
        k and stores k and v itself."""
        return self.dtype == torch.bfloat16 and batch.decode_only and cache.writes and self._table is not None and not self.extended \
            and not self.prepared \
            and self._pairing == "halves"          # the MFMA-path kernels turn halves; the generic one any pairing

    def takes_beside(self, job, batch, cache: LayerCache) -> bool:
        if not self._decodes_fused(batch, cache):
            return False
        from ..ops import fast
        return fast.attention_decode_takes(job, job.a.shape[0], self.spec.n_heads, self.spec.head_dim, cache.k.shape[2],
                                           batch.max_kv)

    def attend(self, qkv, batch, cache: LayerCache, beside=None):
        """Position encoding, cache write and attention on the projected input ``[n, q|k|v]``."""
        spec = self.spec
        n = qkv.shape[0]
        group = batch.groups[cache.group]
        out = batch.workspace.get("attn.out", (n, self.out_dim), self.dtype)
        if self.prepared:
            if beside is not None:
                self._alone(beside)
            return self._attend_prepared(qkv, batch, cache, group, out)
        if self.extended:
            if beside is not None:
                self._alone(beside)
            return self._attend_extended(qkv, batch, cache, group, out)
        halves = self._pairing == "halves"
        if qkv.dtype == torch.bfloat16 and self._decodes_fused(batch, cache):
            from ..ops import fast
            k_new = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            v_new = qkv[:, self.q_dim + self.kv_dim:]
            operands = (qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                        self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, batch)
            fuse = (k_new, v_new, self._table, group.slots)
            if beside is not None and fast.attention_decode_bf16(*operands, fuse=fuse, beside=beside):
                return out
            if beside is not None:
                self._alone(beside)
                beside = None
            if fast.attention_decode_bf16(*operands, fuse=fuse):
                return out
        if beside is not None:
            self._alone(beside)
        slots = group.slots if cache.writes else None
        done = False
        if qkv.dtype == torch.bfloat16 and halves:
            from ..ops import fast
            done = fast.rope_cache_bf16(qkv, batch.positions, slots, self._table, cache.k, cache.v, spec.n_heads,
                                        spec.n_kv_heads, spec.head_dim, group.page_size,
                                        runs=getattr(batch, "page_runs", None))
        if not done:
            core.rope_cache(qkv, batch.positions, slots, self._table, cache.k, cache.v, spec.n_heads, spec.n_kv_heads,
                            spec.head_dim, group.page_size, self._pairing)
        paged_attention(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                        self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, batch)
        return out

    def _attend_extended(self, qkv, batch, cache: LayerCache, group, out):
        """Queries and keys to unit norm, the cache write, then attention with the terms the specification names."""
        spec = self.spec
        slots = group.slots if cache.writes else None
        # (a decode step's tokens are each a run of their own: nothing to gain from the lists there)
        core.unit_norm_cache(qkv, slots, cache.k, cache.v, spec.n_heads, spec.n_kv_heads, spec.head_dim, self.value_dim,
                             group.page_size, self.unit_norm_eps,
                             runs=None if batch.decode_only else getattr(batch, "page_runs", None))
        if qkv.dtype == torch.bfloat16:
            from ..ops import fast
            if fast.attention_biased_bf16(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi,
                                          out, self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, self.value_dim,
                                          batch.positions, self._slopes, self.sink, batch):
                return out
        core.attention_generic(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                               self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, self.value_dim, batch.positions,
                               self._slopes, self.sink)
        return out

    def _attend_prepared(self, projected, batch, cache: LayerCache, group, out):
        """Queries, keys and values made ready by one kernel (norms, rotation, factor, blend, cache write), attention with
        the distance table where there is one, then the output gate. ``projected``: ``[n, q | k | v (| gate)]``."""
        spec = self.spec
        n = projected.shape[0]
        qkv = projected[:, :self.qkv_dim] if self.gated else projected
        slots = group.slots if cache.writes else None
        other = None
        if self.blend is not None:
            # the source layer's values of this step's tokens: scratch of the step, at a fixed address under graphs
            other = batch.workspace.get("shared." + self.blend.name, (n, self.v_dim), self.dtype)
        norm = self.qk_norm
        if self.shares_kv and cache.writes:
            raise RuntimeError("a layer without keys and values of its own must read another layer's cache (ScheduleEntry.reads_cache_of)")
        core.qkv_prepare(qkv, batch.positions, slots, cache.k, cache.v, spec.n_heads, 0 if self.shares_kv else spec.n_kv_heads,
                         spec.head_dim, self.value_dim, group.page_size, norm.scope if norm is not None else None, self._q_gain,
                         self._k_gain, float(norm.eps) if norm is not None else 0.0, self._freqs, self._pairing,
                         (self.growth.coef, self.growth.every) if self.growth is not None else None,
                         self.blend.role if self.blend is not None else None, other, self._blend_weight,
                         values_from_keys=self.values_from_keys)
        gate = projected[:, self.qkv_dim:] if self.gated else None
        more = dict(sinks=self._sinks, softcap=self.softcap, gate_per_head=self.gate_per_head)
        done = gated = False          # (gated: the attention kernel has applied the output gate in its epilogue)
        if qkv.dtype == torch.bfloat16:
            from ..ops import fast
            if self.extended:
                done = gated = fast.attention_biased_bf16(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo,
                                                          batch.kv_hi, out, self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim,
                                                          self.value_dim, batch.positions, None, None, batch,
                                                          bias_table=self._bias_table, gate=gate, **more)
            else:
                paged_attention(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                                self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, batch)
                done = True
        if not done:
            core.attention_generic(qkv, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, out,
                                   self.scale, spec.n_heads, spec.n_kv_heads, spec.head_dim, self.value_dim, batch.positions,
                                   None, None, bias_table=self._bias_table, gate=gate, **more)
            gated = True
        if self.gated and not gated:
            core.gate_mul(out, gate)
        return out

    @staticmethod
    def _alone(job) -> None:
        """A job that was promised a place in the attention launch and did not get one after all."""
        linear(job.a, job.weight, job.bias, job.out, act=job.act)

    def mix(self, h, batch, cache: LayerCache, out, accumulate: bool) -> None:
        """The mixer's output written into (or added to) fp32 ``out``."""
        qkv = batch.workspace.get("attn.qkv", (h.shape[0], self.in_dim), self.dtype)
        linear(h, self.qkv_weight, self.qkv_bias, qkv)
        mixed = self.attend(qkv, batch, cache)
        linear(mixed, self.proj_weight, self.proj_bias, out, accumulate=accumulate)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        self.mix(h, batch, cache, residual, True)


register_mixer("attention", PagedAttention)
