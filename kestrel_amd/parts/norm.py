"""LayerNorm with gain and optional shift, and the root-mean-square norm with gain; statistics in fp32."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from .base import Norm, register_norm
from .specs import NormSpec, ParamSpec


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * weight + bias`` over the last axis (biased variance).

    Reference: ``kestrel/models/moondream/layers.py:40-44`` (the kernel is called without
    eps; the modules are ``nn.LayerNorm(dim)``, ``text.py:311,359``).
    """

    replays_every_step = True

    def __init__(self, spec: NormSpec) -> None:
        super().__init__(spec)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        out = {"weight": ParamSpec((self.spec.dim,), "vector", "gain")}
        if self.spec.bias:
            out["bias"] = ParamSpec((self.spec.dim,), "vector", "shift")
        return out

    def bind(self, tensors, dtype, device) -> None:
        # Gains and shifts are read as fp32 by the kernel whatever they are stored in.
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()
        self.bias = tensors["bias"].to(device=device, dtype=torch.float32).contiguous() if self.spec.bias else None

    def forward(self, x, out, rows=None) -> None:
        core.layernorm(x, self.weight, self.bias, self.spec.eps, out, rows)

    def layernorm_operands(self):
        return self.weight, self.bias, float(self.spec.eps)


class RMSNorm(Norm):
    """``x / sqrt(mean(x^2) + eps) * (offset + weight)`` over the last axis: no mean is taken off, no shift is added;
    ``spec.offset`` is 0 for a weight used as stored and 1 for one stored around zero (added once, in fp32, when the
    weights are bound). It offers no ``layernorm_operands`` (it is no LayerNorm), but
    ``rms_operands``: the weight-streaming linears of a few rows take it into their launch as they take a LayerNorm."""

    replays_every_step = True

    def __init__(self, spec: NormSpec) -> None:
        super().__init__(spec)
        self.weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        around_zero = float(getattr(self.spec, "offset", 0.0)) != 0.0
        return {"weight": ParamSpec((self.spec.dim,), "vector", "shift" if around_zero else "gain")}

    def bind(self, tensors, dtype, device) -> None:
        self.weight = (tensors["weight"].to(device=device, dtype=torch.float32) + float(getattr(self.spec, "offset", 0.0))).contiguous()

    def forward(self, x, out, rows=None) -> None:
        core.rmsnorm(x, self.weight, self.spec.eps, out, rows)

    def add_normed(self, y, x, rounded=None) -> None:
        """``x += norm(y)`` for fp32 rows ``y`` into the fp32 stream ``x`` (a norm that stands behind a sublayer); ``rounded``:
        the new rows of the stream are left there too, in that tensor's type."""
        core.branches_sum(x, y, self.weight, 1.0, eps=float(self.spec.eps), rounded=rounded)

    def rms_operands(self):
        """``(weight fp32 [dim], eps)`` of ``x / sqrt(mean(x^2) + eps) * weight``."""
        return self.weight, float(self.spec.eps)


register_norm("layernorm", LayerNorm)
register_norm("rmsnorm", RMSNorm)
