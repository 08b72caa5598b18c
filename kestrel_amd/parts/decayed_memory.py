"""A recurrent mixer whose state decays channel by channel: time mixing in the manner of RWKV."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import activation_code, linear
from .base import LayerCache, Mixer, register_mixer
from .specs import DecayedMemorySpec, ParamSpec, StateSpec

# the five projections that each read a token-shifted mix of their own, in the order the mixes are laid out
MIXES = ("r", "k", "v", "g", "w")


class DecayedMemory(Mixer):
    """Per head a state ``S`` ``[d, d]`` (key channel by value channel), fp32, zero for a new request and carried from token
    to token in the request's state slot, together with the stream's row of the request's last token.

    With ``x'`` the stream's row of the token before (zeros before the first token), each of the five projections reads a
    mix of its own, ``m_s = x + (x' - x) * mu_s``. Then ``r = W_r m_r``, ``k = W_k m_k``, ``v = W_v m_v`` (heads of ``d``),
    ``gate = silu(W_g m_g)``, and the decay ``w = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))`` per head and key channel. Per head

        o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t            S_t = diag(w_t) S_(t-1) + k_t v_t^T

    (the bonus ``u`` counts for the token's own key only). Every head's ``o`` is divided by its root mean square (``eps``);
    the heads are concatenated, multiplied by the gain ``norm.weight`` and by the gate, and go through the output
    projection.

    The mixer reads the fp32 stream itself (``reads_stream``): the mixes are computed in fp32 and rounded once to the
    activation type. The five projections are linears of that type; the second linear of the decay writes fp32 (with
    ``w0`` as its bias) and the exponentials are taken in the recurrence kernel, so that everything that enters the
    recurrence besides the projections is fp32. One kernel walks over every row's tokens in order and a second normalises the read-outs
    (``ops.core.decayed_memory``), whatever the step holds: a prompt, a portion, single tokens. Rows without a request
    (the padding of a replayed step) write zeros and touch no state."""

    replays_every_step = True
    reads_stream = True

    def __init__(self, spec: DecayedMemorySpec) -> None:
        super().__init__(spec)
        self.width = spec.n_heads * spec.head_dim
        self.rank = -1 if getattr(spec, "decay_rank", None) is None else int(spec.decay_rank)
        self.mu = self.w_r = self.w_k = self.w_v = self.w_g = self.w_1 = self.w_2 = self.w_0 = None
        self.u = self.gain = self.proj_weight = None
        self.dtype: Optional[torch.dtype] = None
        self._tanh, self._silu = activation_code("tanh"), activation_code("silu")

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {f"mu.{s}": ParamSpec((spec.dim,), "vector", "fraction") for s in MIXES}
        out.update({f"{s}.weight": ParamSpec((self.width, spec.dim)) for s in ("r", "k", "v", "g")})
        out.update({"w1.weight": ParamSpec((self.rank, spec.dim)), "w2.weight": ParamSpec((self.width, self.rank)),
                    "w0": ParamSpec((self.width,), "vector", "bias"), "u": ParamSpec((spec.n_heads, spec.head_dim), "matrix", "bias"),
                    "norm.weight": ParamSpec((self.width,), "vector", "gain"), "proj.weight": ParamSpec((spec.dim, self.width))})
        return out

    def state_spec(self) -> StateSpec:
        spec = self.spec
        return StateSpec((self.width * spec.head_dim + spec.dim,), "float32")

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        if not core.decayed_memory_supported(self.spec.head_dim):
            raise ValueError(f"the decaying memory's kernel takes heads of up to 256 channels, got {self.spec.head_dim}")
        f32 = dict(device=device, dtype=torch.float32)
        self.mu = torch.stack([tensors[f"mu.{s}"].to(**f32) for s in MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (tensors[f"{s}.weight"].to(device).contiguous() for s in ("r", "k", "v", "g"))
        self.w_1 = tensors["w1.weight"].to(device).contiguous()
        self.w_2 = tensors["w2.weight"].to(device).contiguous()
        if self.w_1.shape[0] != self.w_2.shape[1]:
            raise ValueError(f"the decay's two linears meet in {self.w_1.shape[0]} and {self.w_2.shape[1]} channels")
        self.w_0 = tensors["w0"].to(**f32).reshape(-1).contiguous()
        self.u = tensors["u"].to(**f32).reshape(-1).contiguous()
        self.gain = tensors["norm.weight"].to(**f32).contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()

    def read(self, x, batch, cache: LayerCache) -> torch.Tensor:
        """The recurrence over the step's tokens for the fp32 stream ``x``; returns the input of the output projection."""
        spec = self.spec
        n = x.shape[0]
        ws = batch.workspace
        if cache.state is None:
            raise RuntimeError("the decaying memory needs its per-request state from the cache manager")
        if x.dtype != torch.float32:
            raise RuntimeError("the decaying memory reads the fp32 stream")
        state = cache.state
        kept = state[:, self.width * spec.head_dim:]
        mixes = ws.get("decay.mixes", (len(MIXES), n, spec.dim), self.dtype)
        core.token_shift(x, kept, self.mu, batch.token_row, batch.cu_q, batch.row_slot, mixes)
        rkvg = ws.get("decay.rkvg", (n, 4 * self.width), self.dtype)
        for i, (weight, act) in enumerate(((self.w_r, 0), (self.w_k, 0), (self.w_v, 0), (self.w_g, self._silu))):
            linear(mixes[i], weight, None, rkvg[:, i * self.width:(i + 1) * self.width], act=act)
        low = ws.get("decay.low", (n, self.w_1.shape[0]), self.dtype)
        linear(mixes[4], self.w_1, None, low, act=self._tanh)
        pre = ws.get("decay.pre", (n, self.width), torch.float32)
        linear(low, self.w_2, self.w_0, pre)
        out = ws.get("decay.out", (n, self.width), self.dtype)
        r, k, v, g = (rkvg[:, i * self.width:(i + 1) * self.width] for i in range(4))
        raw = ws.get("decay.raw", (n, self.width), torch.float32)
        core.decayed_memory(r, k, v, g, pre, self.u, self.gain, state, x, batch.cu_q, batch.row_slot, out, spec.n_heads,
                            spec.head_dim, spec.eps, raw=raw)
        return out

    def output_projection(self):
        return self.proj_weight, None

    def mix(self, h, batch, cache: LayerCache, out, accumulate: bool) -> None:
        """The mixer's output written into (or added to) fp32 ``out``."""
        linear(self.read(h, batch, cache), self.proj_weight, None, out, accumulate=accumulate)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        self.mix(h, batch, cache, residual, True)


register_mixer("decayed_memory", DecayedMemory)
