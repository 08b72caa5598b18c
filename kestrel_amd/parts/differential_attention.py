"""Differential attention: two softmax maps per head over the same values, subtracted and normalised."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import linear
from .base import LayerCache, Mixer, build_part, register_mixer
from .specs import CacheSpec, DifferentialAttentionSpec, ParamSpec, StateSpec


class DifferentialAttention(Mixer):
    """Per head two attentions ``a1``, ``a2`` with queries and keys of their own over the same values:

        o = a1 - lambda a2,   lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init   (one number for the layer)
        out = o / sqrt(mean(o^2) + eps) * (1 - lambda_init)                          (over a head's values, no gain)

    Queries are ``[H, 2, hd]`` and keys ``[G, 2, hd]``, head by head as ``[map 1, map 2]``; values ``[G, hdv]``; query head ``h``
    reads key/value head ``h // (H / G)``. To the kernels a map is a head: ``2 H`` query heads read ``2 G`` key heads, and the two
    key heads of a pair share one value head (``ops.core.attention_generic`` with ``maps = 2``). The maps leave the attention
    kernel in fp32 and are combined in fp32.

    Right after the projections comes an optional short causal convolution over time on every channel of q, k and v
    (tensors ``q.conv``, ``k.conv``, ``v.conv`` ``[channels, taps]``): the last ``taps - 1`` projected rows of a sequence are
    per-request state. Convolution, rotation (``spec.position``) and the cache write are one kernel (``ops.core.conv_prepare``).

    The mask is a window that keeps the first keys: the cache manager never gives back the pages of the first
    ``keep_first`` positions, the step's ``kv_lo`` is the window's start, and the attention kernel reads ``[0, min(keep_first,
    kv_lo))`` and ``[kv_lo, kv_hi)``."""

    replays_every_step = True

    def __init__(self, spec: DifferentialAttentionSpec) -> None:
        super().__init__(spec)
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} query heads cannot share {spec.n_kv_heads} kv heads")
        self.position = build_part("position", spec.position)
        self.q_dim = spec.n_heads * 2 * spec.head_dim
        self.k_dim = spec.n_kv_heads * 2 * spec.head_dim
        self.v_dim = spec.n_kv_heads * spec.value_dim
        self.in_dim = self.q_dim + self.k_dim + self.v_dim
        self.out_dim = spec.n_heads * spec.value_dim
        self.taps = int(spec.conv_taps) if spec.conv_taps else 0
        self.window = spec.mask.size if spec.mask is not None else None
        self.keep_first = int(spec.mask.keep_first) if spec.mask is not None else 0
        self.in_weight = self.proj_weight = self._taps = self._freqs = None
        self._pairing = "halves"
        self.map_weight = 0.0
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"q.weight": ParamSpec((self.q_dim, spec.dim)), "k.weight": ParamSpec((self.k_dim, spec.dim)),
               "v.weight": ParamSpec((self.v_dim, spec.dim)), "proj.weight": ParamSpec((spec.dim, self.out_dim))}
        for name in ("lq1", "lk1", "lq2", "lk2"):
            out[name] = ParamSpec((spec.head_dim,), "vector", "bias")
        if self.taps:
            out.update({"q.conv": ParamSpec((self.q_dim, self.taps), "matrix", "normal"),
                        "k.conv": ParamSpec((self.k_dim, self.taps), "matrix", "normal"),
                        "v.conv": ParamSpec((self.v_dim, self.taps), "matrix", "normal")})
        return out

    def cache_spec(self) -> CacheSpec:
        spec = self.spec
        return CacheSpec(2 * spec.n_kv_heads, spec.head_dim, self.window, spec.value_dim, keep_first=self.keep_first,
                         value_heads=spec.n_kv_heads)

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.taps - 1, self.in_dim), "float32") if self.taps > 1 else None

    def bind(self, tensors, dtype, device) -> None:
        spec = self.spec
        self.dtype = dtype
        self.in_weight = torch.cat([tensors[f"{name}.weight"].to(device) for name in ("q", "k", "v")], dim=0).contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()
        if self.taps:
            self._taps = torch.cat([tensors[f"{name}.conv"].to(device=device, dtype=torch.float32) for name in ("q", "k", "v")],
                                   dim=0).contiguous()
        fp = {name: tensors[name].to(device=device, dtype=torch.float32) for name in ("lq1", "lk1", "lq2", "lk2")}
        weight = torch.exp((fp["lq1"] * fp["lk1"]).sum()) - torch.exp((fp["lq2"] * fp["lk2"]).sum()) + \
            torch.tensor(float(spec.lambda_init), dtype=torch.float32, device=device)
        self.map_weight = float(weight.item())
        if int(getattr(self.position, "axes", 1)) != 1:
            raise ValueError("differential attention rotates by a token's place in the sequence")
        rotation = self.position.rotation(device)
        if rotation is not None:
            if getattr(rotation, "frequencies", None) is None:
                raise ValueError("differential attention takes a rotation given by frequencies")
            if rotation.pairing not in core.ROTARY_PAIRINGS or 2 * rotation.frequencies.numel() > spec.head_dim:
                raise ValueError(f"differential attention cannot apply this rotation to heads of {spec.head_dim} channels")
            self._freqs, self._pairing = rotation.frequencies.to(device).contiguous(), rotation.pairing

    def query_tile(self) -> Optional[int]:
        if self.dtype != torch.bfloat16:
            return None                     # the generic kernel takes tokens one by one
        from ..ops import fast
        return fast.biased_query_block(self.spec.head_dim, self.spec.value_dim)

    def input_projection(self):
        return self.in_weight, None, self.in_dim

    def output_projection(self):
        return self.proj_weight, None

    def attend(self, projected, batch, cache: LayerCache, beside=None) -> torch.Tensor:
        """Convolution, rotation, cache write, both maps, their combination; returns the input of the output projection."""
        spec = self.spec
        n = projected.shape[0]
        ws = batch.workspace
        group = batch.groups[cache.group]
        if self.taps > 1 and cache.state is None:
            raise RuntimeError("the convolution needs its per-request state from the cache manager")
        q = ws.get("diff.q", (n, self.q_dim), self.dtype)
        slots = group.slots if cache.writes else None
        core.conv_prepare(projected, self._taps, cache.state, batch.cu_q, batch.row_slot, batch.token_row, batch.positions, slots, q,
                          cache.k, cache.v, 2 * spec.n_heads, 2 * spec.n_kv_heads, spec.head_dim, spec.n_kv_heads, spec.value_dim,
                          group.page_size, self._freqs, self._pairing)
        maps = ws.get("diff.maps", (n, 2 * self.out_dim), torch.float32)
        done = False
        if self.dtype == torch.bfloat16:
            from ..ops import fast
            done = fast.attention_maps_bf16(q, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, maps,
                                            float(spec.scale), 2 * spec.n_heads, 2 * spec.n_kv_heads, spec.head_dim, spec.value_dim,
                                            self.keep_first, 2, batch)
        if not done:
            core.attention_generic(q, cache.k, cache.v, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, maps,
                                   float(spec.scale), 2 * spec.n_heads, 2 * spec.n_kv_heads, spec.head_dim, spec.value_dim,
                                   keep_first=self.keep_first, maps=2)
        out = ws.get("diff.out", (n, self.out_dim), self.dtype)
        core.maps_combine(maps, out, spec.n_heads, spec.value_dim, self.map_weight, spec.eps, 1.0 - float(spec.lambda_init))
        return out

    def mix(self, h, batch, cache: LayerCache, out, accumulate: bool) -> None:
        projected = batch.workspace.get("diff.in", (h.shape[0], self.in_dim), self.dtype)
        linear(h, self.in_weight, None, projected)
        linear(self.attend(projected, batch, cache), self.proj_weight, None, out, accumulate=accumulate)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        self.mix(h, batch, cache, residual, True)


register_mixer("differential_attention", DifferentialAttention)
