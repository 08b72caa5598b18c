"""Latent attention: queries, keys and values through low-rank latents; the cache holds the latent."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import linear
from .base import LayerCache, Mixer, build_part, register_mixer
from .specs import LatentAttentionSpec, LatentCacheSpec, ParamSpec


class LatentAttention(Mixer):
    """With ``rms(x) = x / sqrt(mean(x^2) + eps)``:

        c_q = rms(W_dq h) g_q,   q = W_uq c_q                 per head [hd plain | dr rotated]
        [c' | k_r] = W_dkv h,    c = rms(c') g_kv             c: the latent (kv_rank), k_r: dr channels shared by all heads
        k_h = [W_uk,h c | rot(k_r)],   v_h = W_uv,h c
        score = scale * (q_plain . W_uk,h c + rot(q_rot) . rot(k_r)),   softmax over j <= i with exp(sink_h) in the denominator
        out = W_o (concat_h(sum_j w_j v_h,j) * sigmoid(W_g h))

    Only ``[c | rot(k_r)]`` is cached, one row of ``kv_rank + dr`` channels per token (``LatentCacheSpec``). The per-head
    up-projections are moved to the query's side: ``q_plain . W_uk,h c = (W_uk,h^T q_plain) . c``, so every head's query
    becomes ``[W_uk,h^T q_plain | rot(q_rot)]`` against the cached row, and ``sum_j w_j W_uv,h c_j = W_uv,h sum_j w_j c_j``,
    so the attention kernel returns weighted sums of latents (the cached row's first ``kv_rank`` channels are its value)
    that ``W_uv,h`` then lifts to the head's values. To the kernel this is attention of ``H`` query heads over one key
    head whose values lie inside its keys (``ops.core.attention_generic`` with ``values_in_keys``)."""

    replays_every_step = True

    def __init__(self, spec: LatentAttentionSpec) -> None:
        super().__init__(spec)
        self.position = build_part("position", spec.position)
        self.q_head = spec.head_dim + spec.rot_dim
        self.q_dim = spec.n_heads * self.q_head
        self.row_dim = spec.kv_rank + spec.rot_dim              # a cached row, and a query head as the kernel sees it
        self.out_dim = spec.n_heads * spec.value_dim
        self.gated = bool(spec.output_gate)
        self.down_dim = spec.q_rank + self.row_dim + (self.out_dim if self.gated else 0)
        self.down_weight = self.uq_weight = self.absorb = self.lift = self.proj_weight = None
        self._q_gain = self._kv_gain = self._sinks = self._freqs = None
        self._pairing = "halves"
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"dq.weight": ParamSpec((spec.q_rank, spec.dim)), "dq_norm.weight": ParamSpec((spec.q_rank,), "vector", "gain"),
               "uq.weight": ParamSpec((self.q_dim, spec.q_rank)), "dkv.weight": ParamSpec((self.row_dim, spec.dim)),
               "dkv_norm.weight": ParamSpec((spec.kv_rank,), "vector", "gain"),
               "uk.weight": ParamSpec((spec.n_heads * spec.head_dim, spec.kv_rank)),
               "uv.weight": ParamSpec((self.out_dim, spec.kv_rank)), "proj.weight": ParamSpec((spec.dim, self.out_dim))}
        if spec.head_sinks:
            out["sink"] = ParamSpec((spec.n_heads,), "vector", "bias")
        if self.gated:
            out["gate.weight"] = ParamSpec((self.out_dim, spec.dim))
        return out

    def cache_spec(self) -> LatentCacheSpec:
        return LatentCacheSpec(self.spec.kv_rank, self.spec.rot_dim)

    def bind(self, tensors, dtype, device) -> None:
        spec = self.spec
        self.dtype = dtype
        names = ["dq.weight", "dkv.weight"] + (["gate.weight"] if self.gated else [])
        # one launch projects the query latent, the key/value latent with the shared key part, and the gate
        self.down_weight = torch.cat([tensors[name].to(device) for name in names], dim=0).contiguous()
        self.uq_weight = tensors["uq.weight"].to(device).contiguous()
        # W_uk per head, transposed: [H, kv_rank, hd] (a linear's weight for q_plain -> latent space)
        self.absorb = tensors["uk.weight"].to(device).view(spec.n_heads, spec.head_dim, spec.kv_rank).transpose(1, 2).contiguous()
        self.lift = tensors["uv.weight"].to(device).view(spec.n_heads, spec.value_dim, spec.kv_rank).contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()
        self._q_gain = tensors["dq_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        self._kv_gain = tensors["dkv_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        if spec.head_sinks:
            self._sinks = tensors["sink"].to(device=device, dtype=torch.float32).contiguous()
        if int(getattr(self.position, "axes", 1)) != 1:
            raise ValueError("latent attention rotates by a token's place in the sequence")
        rotation = self.position.rotation(device)
        if rotation is not None:
            if getattr(rotation, "frequencies", None) is None:
                raise ValueError("latent attention takes a rotation given by frequencies")
            if rotation.pairing not in core.ROTARY_PAIRINGS or 2 * rotation.frequencies.numel() > spec.rot_dim:
                raise ValueError(f"latent attention cannot apply this rotation to a part of {spec.rot_dim} channels")
            self._freqs, self._pairing = rotation.frequencies.to(device).contiguous(), rotation.pairing

    def query_tile(self) -> Optional[int]:
        if self.dtype != torch.bfloat16:
            return None                     # the generic kernel takes tokens one by one
        from ..ops import fast
        return fast.biased_query_block(self.row_dim, self.spec.kv_rank)

    def input_projection(self):
        return self.down_weight, None, self.down_dim

    def output_projection(self):
        return self.proj_weight, None

    def attend(self, down, batch, cache: LayerCache, beside=None) -> torch.Tensor:
        """From the projected row ``[c_q' | c' | k_r | gate]`` to the gated heads, the input of the output projection."""
        spec = self.spec
        n = down.shape[0]
        ws = batch.workspace
        group = batch.groups[cache.group]
        slots = group.slots if cache.writes else None
        cq = ws.get("latent.cq", (n, spec.q_rank), self.dtype)
        core.latent_prepare(down, 0, spec.q_rank, self._q_gain, cq, spec.q_rank, spec.kv_rank, self._kv_gain, spec.rot_dim,
                            self._freqs, self._pairing, batch.positions, slots, cache.k, spec.eps)
        q = ws.get("latent.q", (n, self.q_dim), self.dtype)
        linear(cq, self.uq_weight, None, q)
        full = ws.get("latent.q_full", (n, spec.n_heads * self.row_dim), self.dtype)
        core.rotate_tail(q, full, spec.n_heads, spec.head_dim, spec.rot_dim, spec.kv_rank, self._freqs, self._pairing, batch.positions)
        self._per_head(q, self.q_head, spec.head_dim, self.absorb, full, self.row_dim, spec.kv_rank)
        mixed = ws.get("latent.mixed", (n, spec.n_heads * spec.kv_rank), self.dtype)
        gate = down[:, spec.q_rank + self.row_dim:] if self.gated else None
        done = False
        if self.dtype == torch.bfloat16:
            from ..ops import fast
            done = fast.attention_latent_bf16(full, cache.k, group.block_table, batch.token_row, batch.kv_hi, mixed, float(spec.scale),
                                              spec.n_heads, self.row_dim, spec.kv_rank, self._sinks, batch)
        if not done:
            core.attention_generic(full, cache.k, None, group.block_table, batch.token_row, group.kv_lo, batch.kv_hi, mixed,
                                   float(spec.scale), spec.n_heads, 1, self.row_dim, spec.kv_rank, sinks=self._sinks,
                                   values_in_keys=True)
        heads = ws.get("latent.heads", (n, self.out_dim), self.dtype)
        if not self._per_head(mixed, spec.kv_rank, spec.kv_rank, self.lift, heads, spec.value_dim, spec.value_dim, gate) \
                and gate is not None:
            core.gate_mul(heads, gate)
        return heads

    def _per_head(self, a, a_head: int, k: int, weights, out, out_head: int, n_out: int, gate=None) -> bool:
        """``out[:, h, :n_out] = a[:, h, :k] @ weights[h].T`` for every head (rows of ``a`` hold heads of ``a_head`` channels, rows of
        ``out`` heads of ``out_head``). True: the outputs were also multiplied by the sigmoid of ``gate``."""
        if self.dtype == torch.bfloat16:
            from ..ops import fast
            if fast.heads_linear_bf16(a, a_head, k, weights, out, out_head, n_out, gate):
                return gate is not None
        for h in range(self.spec.n_heads):
            linear(a[:, h * a_head:h * a_head + k], weights[h], None, out[:, h * out_head:h * out_head + n_out])
        return False

    def mix(self, h, batch, cache: LayerCache, out, accumulate: bool) -> None:
        down = batch.workspace.get("latent.down", (h.shape[0], self.down_dim), self.dtype)
        linear(h, self.down_weight, None, down)
        linear(self.attend(down, batch, cache), self.proj_weight, None, out, accumulate=accumulate)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        self.mix(h, batch, cache, residual, True)


register_mixer("latent_attention", LatentAttention)
