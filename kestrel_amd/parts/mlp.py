"""Dense feed-forwards: two linears around an activation, plain or gated."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops.linear import ACT_GATED, activation_code, linear, linear_gated, pair_rows
from .base import FeedForward, register_feed_forward
from .specs import ClampedGatedFeedForwardSpec, DenseFeedForwardSpec, GatedFeedForwardSpec, ParamSpec


class DenseFeedForward(FeedForward):
    """``fc2(act(fc1(h)))`` with biases; the activation runs in the first linear's epilogue.

    Reference: ``kestrel/models/moondream/layers.py:64-121`` (``fc1``, ``F.gelu`` with the
    tanh approximation ``layers.py:30-31``, ``fc2``).
    """

    replays_every_step = True

    def __init__(self, spec: DenseFeedForwardSpec) -> None:
        super().__init__(spec)
        self.act = activation_code(spec.activation)
        self.fc1_weight = self.fc1_bias = self.fc2_weight = self.fc2_bias = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"fc1.weight": ParamSpec((spec.hidden_dim, spec.dim)), "fc2.weight": ParamSpec((spec.dim, spec.hidden_dim))}
        if spec.bias:
            out["fc1.bias"] = ParamSpec((spec.hidden_dim,), "vector", "bias")
            out["fc2.bias"] = ParamSpec((spec.dim,), "vector", "bias")
        return out

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        self.fc1_weight = tensors["fc1.weight"].to(device).contiguous()
        self.fc2_weight = tensors["fc2.weight"].to(device).contiguous()
        if self.spec.bias:
            self.fc1_bias = tensors["fc1.bias"].to(device=device, dtype=torch.float32).contiguous()
            self.fc2_bias = tensors["fc2.bias"].to(device=device, dtype=torch.float32).contiguous()

    def input_projection(self):
        return self.fc1_weight, self.fc1_bias, self.spec.hidden_dim, self.act

    def output_projection(self):
        return self.fc2_weight, self.fc2_bias

    def forward(self, h, batch, residual) -> None:
        hidden = batch.workspace.get("ff.hidden", (h.shape[0], self.spec.hidden_dim), self.dtype)
        linear(h, self.fc1_weight, self.fc1_bias, hidden, act=self.act)
        linear(hidden, self.fc2_weight, self.fc2_bias, residual, accumulate=True)


class GatedFeedForward(FeedForward):
    """``down(act(gate h) * (up h))``: the rows of ``gate`` and ``up`` are laid in pairs when the weights are bound, so
    that one linear computes both and takes the product in its epilogue (``ops.linear.linear_gated``)."""

    replays_every_step = True

    def __init__(self, spec: GatedFeedForwardSpec) -> None:
        super().__init__(spec)
        self.act = activation_code(spec.activation)
        self.pairs = self.pair_bias = self.down_weight = self.down_bias = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"gate.weight": ParamSpec((spec.hidden_dim, spec.dim)), "up.weight": ParamSpec((spec.hidden_dim, spec.dim)),
               "down.weight": ParamSpec((spec.dim, spec.hidden_dim))}
        if spec.bias:
            out.update({"gate.bias": ParamSpec((spec.hidden_dim,), "vector", "bias"), "up.bias": ParamSpec((spec.hidden_dim,), "vector", "bias"),
                        "down.bias": ParamSpec((spec.dim,), "vector", "bias")})
        return out

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        self.pairs = pair_rows(tensors["gate.weight"].to(device), tensors["up.weight"].to(device))
        self.down_weight = tensors["down.weight"].to(device).contiguous()
        if self.spec.bias:
            self.pair_bias = pair_rows(tensors["gate.bias"].to(device=device, dtype=torch.float32),
                                       tensors["up.bias"].to(device=device, dtype=torch.float32))
            self.down_bias = tensors["down.bias"].to(device=device, dtype=torch.float32).contiguous()

    def input_projection(self):
        return self.pairs, self.pair_bias, self.spec.hidden_dim, self.act | ACT_GATED

    def output_projection(self):
        return self.down_weight, self.down_bias

    # Rows from which the gated linear is run as a plain linear over all paired rows (the vendor library's kernels, which
    # have no epilogue for the product of a pair) followed by a pass that takes the products: at 2,048 rows of width 2,048
    # and 5,632 pairs 100 us against the 169 of this package's tiled kernel with the product in its epilogue.
    PAIRS_APART_FROM_ROWS = 256

    def forward(self, h, batch, residual) -> None:
        n = h.shape[0]
        hidden = batch.workspace.get("ff.hidden", (n, self.spec.hidden_dim), self.dtype)
        if self.dtype == torch.bfloat16 and n >= self.PAIRS_APART_FROM_ROWS:
            from ..ops import core
            sums = batch.workspace.get("ff.pair_sums", (n, 2 * self.spec.hidden_dim), self.dtype)
            linear(h, self.pairs, self.pair_bias, sums)
            core.gated_pairs(sums, hidden, self.act)
        else:
            linear_gated(h, self.pairs, self.pair_bias, hidden, self.act)
        linear(hidden, self.down_weight, self.down_bias, residual, accumulate=True)


class ClampedGatedFeedForward(GatedFeedForward):
    """``down(g sigmoid(slope g) (u + shift))`` with ``g = min(gate h, limit)`` and ``u = clamp(up h, -limit, limit)``.

    The rows of ``gate`` and ``up`` are paired as in ``GatedFeedForward``; one plain linear computes both sums side by side
    and a pass over them takes the clamps and the product (``ops.core.clamped_pairs``): the constants are numbers of the
    layer, which the epilogues of the linear kernels (activations by code) do not carry."""

    def __init__(self, spec: ClampedGatedFeedForwardSpec) -> None:
        super().__init__(spec)
        if not spec.limit > 0:
            raise ValueError(f"the clamps of a gated feed-forward need a positive limit, got {spec.limit}")

    def input_projection(self):
        return None        # (no stage of this feed-forward is a linear with an activation by code)

    def output_projection(self):
        return None

    def from_stream(self, x, norm, batch) -> bool:
        """The feed-forward of ``norm(x)`` added into fp32 ``x`` with the norm in the prologue of the first linear's launch
        (a few bf16 rows, a root-mean-square norm); ``False``: not covered, nothing was run."""
        from ..ops import core, fast
        spec = self.spec
        rms = norm.rms_operands() if callable(getattr(norm, "rms_operands", None)) else None
        if rms is None or self.dtype != torch.bfloat16:
            return False
        n = x.shape[0]
        sums = batch.workspace.get("ff.pair_sums", (n, 2 * spec.hidden_dim), self.dtype)
        if not fast.layernorm_linear(x, rms[0], None, rms[1], self.pairs, self.pair_bias, sums, 0, centred=False):
            return False
        hidden = batch.workspace.get("ff.hidden", (n, spec.hidden_dim), self.dtype)
        core.clamped_pairs(sums, hidden, spec.limit, spec.slope, spec.shift)
        linear(hidden, self.down_weight, self.down_bias, x, accumulate=True)
        return True

    def forward(self, h, batch, residual) -> None:
        from ..ops import core
        spec = self.spec
        n = h.shape[0]
        sums = batch.workspace.get("ff.pair_sums", (n, 2 * spec.hidden_dim), self.dtype)
        hidden = batch.workspace.get("ff.hidden", (n, spec.hidden_dim), self.dtype)
        linear(h, self.pairs, self.pair_bias, sums)
        core.clamped_pairs(sums, hidden, spec.limit, spec.slope, spec.shift)
        linear(hidden, self.down_weight, self.down_bias, residual, accumulate=True)


register_feed_forward("dense", DenseFeedForward)
register_feed_forward("clamped_gated_dense", ClampedGatedFeedForward)
register_feed_forward("gated_dense", GatedFeedForward)
