"""A routed mixture of gated feed-forwards with identity experts, groups of experts and a shared expert."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import ACT_GATED, activation_code, linear, linear_gated, pair_rows
from .base import FeedForward, register_feed_forward
from .specs import ParamSpec, RoutedExpertsSpec


class RoutedExperts(FeedForward):
    """``sum over the chosen k of weight_k * expert_k(h) [+ sigmoid(shared.sg h) * shared(h)]``.

    Every expert is ``down(act(gate h) * (up h))`` without biases (tensors ``e<i>.gate.weight`` and so on). The router
    (``router.weight`` ``[n_experts + n_identity, dim]``) writes fp32 logits from fp32 sums, and the choice is made in fp32; how its scores become a choice and weights is
    ``RoutedExpertsSpec``'s text. The router's last ``n_identity`` outputs are identity experts: their output is ``h``.
    The shared expert (``shared.*``) has the experts' form and a hidden size of its own; its gate ``shared.sg.weight``
    ``[1, dim]`` rides as one more row of the router's linear.

    When the weights are bound, the experts' ``gate`` and ``up`` rows are laid in pairs and the experts stacked
    (``[E, 2 hidden, dim]``, ``[E, dim, hidden]``). A step runs: the router's linear (fp32), the choice
    (``ops.core.route``), the experts' two linears, and the weighted sum. In bf16 steps of at least
    ``PAIRS_BY_EXPERT_FROM`` pairs, the pairs are listed by expert and each expert's pairs go through the matrix cores
    together (``ops.fast.experts_feed_forward_bf16``); otherwise, and in fp32, every pair is computed by itself, its expert's
    weights streamed once for it (``ops.core.experts_linear``). Measured at 48 pairs over 62 experts, where the lists hold
    hardly more than a pair an expert: 1.28 ms a step by lists, 1.42 pair by pair. Either way a pair's result depends on
    its own row alone."""

    replays_every_step = True
    PAIRS_BY_EXPERT_FROM = 33

    def __init__(self, spec: RoutedExpertsSpec) -> None:
        super().__init__(spec)
        if spec.n_experts <= 0 or spec.top <= 0 or spec.n_identity < 0:
            raise ValueError("routed experts need experts and a positive number of choices")
        self.n_outputs = spec.n_experts + spec.n_identity
        if spec.top > self.n_outputs:
            raise ValueError(f"{spec.top} choices among {self.n_outputs} router outputs")
        if spec.n_groups:
            if self.n_outputs % spec.n_groups or not 0 < spec.keep_groups <= spec.n_groups:
                raise ValueError(f"{spec.n_groups} groups (of which {spec.keep_groups} are kept) do not divide {self.n_outputs} router outputs")
            if spec.keep_groups * (self.n_outputs // spec.n_groups) < spec.top:
                raise ValueError("the kept groups hold fewer router outputs than a token chooses")
        self.act = activation_code(spec.activation)
        self.shared = spec.shared_hidden is not None
        self.gated_shared = self.shared and bool(spec.shared_gate)
        self.pairs = self.down = self.router = self.correction = None
        self.shared_pairs = self.shared_down = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {}
        for e in range(spec.n_experts):
            out[f"e{e}.gate.weight"] = ParamSpec((spec.hidden_dim, spec.dim))
            out[f"e{e}.up.weight"] = ParamSpec((spec.hidden_dim, spec.dim))
            out[f"e{e}.down.weight"] = ParamSpec((spec.dim, spec.hidden_dim))
        out["router.weight"] = ParamSpec((self.n_outputs, spec.dim))
        out["correction"] = ParamSpec((self.n_outputs,), "vector", "bias")
        if self.shared:
            out["shared.gate.weight"] = ParamSpec((spec.shared_hidden, spec.dim))
            out["shared.up.weight"] = ParamSpec((spec.shared_hidden, spec.dim))
            out["shared.down.weight"] = ParamSpec((spec.dim, spec.shared_hidden))
            if self.gated_shared:
                out["shared.sg.weight"] = ParamSpec((1, spec.dim))
        return out

    def bind(self, tensors, dtype, device) -> None:
        spec = self.spec
        self.dtype = dtype
        self.pairs = torch.stack([pair_rows(tensors[f"e{e}.gate.weight"].to(device), tensors[f"e{e}.up.weight"].to(device))
                                  for e in range(spec.n_experts)]).contiguous()
        self.down = torch.stack([tensors[f"e{e}.down.weight"].to(device) for e in range(spec.n_experts)]).contiguous()
        # The router's rows stay in the type they are held in: products of bf16 numbers are exact in fp32 and every linear
        # kernel sums in fp32, so a bf16 run computes the router's sums in 32 bits from the rounded input, as an fp32 run does
        # from its own. The shared expert's gate rides as one more row.
        rows = [tensors["router.weight"].to(device)]
        if self.gated_shared:
            rows.append(tensors["shared.sg.weight"].to(device=device, dtype=rows[0].dtype).reshape(1, spec.dim))
        self.router = torch.cat(rows, dim=0).contiguous()
        self.correction = tensors["correction"].to(device=device, dtype=torch.float32).contiguous()
        if self.shared:
            self.shared_pairs = pair_rows(tensors["shared.gate.weight"].to(device), tensors["shared.up.weight"].to(device))
            self.shared_down = tensors["shared.down.weight"].to(device).contiguous()

    def mix(self, h, batch, out, accumulate: bool) -> None:
        """The feed-forward of ``h`` written into (or added to) fp32 ``out``."""
        spec = self.spec
        n = h.shape[0]
        ws = batch.workspace
        top, E = spec.top, spec.n_experts
        logits = ws.get("experts.logits", (n, self.router.shape[0]), torch.float32)
        linear(h, self.router, None, logits)
        chosen = ws.get("experts.chosen", (n, top), torch.int32)
        weights = ws.get("experts.weights", (n, top), torch.float32)
        core.route(logits, self.n_outputs, self.correction, top, spec.n_groups, spec.keep_groups, spec.scale, chosen, weights)
        hidden = ws.get("experts.hidden", (n * top, spec.hidden_dim), self.dtype)
        y = ws.get("experts.y", (n * top, spec.dim), torch.float32)
        done = False
        if self.dtype == torch.bfloat16 and n * top >= self.PAIRS_BY_EXPERT_FROM:
            from ..ops import fast
            done = fast.experts_feed_forward_bf16(h, self.pairs, self.down, chosen, hidden, y, self.act, ws)
        if not done:
            flat = chosen.view(-1)
            core.experts_linear(h, top, self.pairs, flat, hidden, self.act | ACT_GATED)
            core.experts_linear(hidden, 1, self.down, flat, y)
        shared_out = gate = None
        if self.shared:
            shared_hidden = ws.get("experts.shared_hidden", (n, spec.shared_hidden), self.dtype)
            if self.dtype == torch.bfloat16 and n >= 256:
                sums = ws.get("experts.shared_sums", (n, 2 * spec.shared_hidden), self.dtype)
                linear(h, self.shared_pairs, None, sums)
                core.gated_pairs(sums, shared_hidden, self.act)
            else:
                linear_gated(h, self.shared_pairs, None, shared_hidden, self.act)
            shared_out = ws.get("experts.shared_out", (n, spec.dim), torch.float32)
            linear(shared_hidden, self.shared_down, None, shared_out)
            if self.gated_shared:
                gate = logits[:, self.n_outputs]
        core.experts_combine(y, h, chosen, weights, E, shared_out, gate, out, accumulate)

    def forward(self, h, batch, residual) -> None:
        self.mix(h, batch, residual, True)


register_feed_forward("routed_experts", RoutedExperts)
