"""Junctions: transformations of the whole residual stream between runs of layers."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import linear
from .base import Junction, register_junction
from .specs import ConcatLinearSpec, ParamSpec, PassVectorSpec


class ConcatLinear(Junction):
    """``x <- W [x; x0]``: the stream and the embedding output ``x0`` side by side through one linear without bias,
    ``W`` ``[dim, 2 dim]`` with the stream's columns first.

    The two are laid side by side as rows of ``2 dim`` of the activation type: the right half is written once
    a step (``begin``), the left half at every passage; the product goes back into the fp32 stream."""

    replays_every_step = True

    def __init__(self, spec: ConcatLinearSpec) -> None:
        super().__init__(spec)
        self.weight: Optional[torch.Tensor] = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.spec.dim, 2 * self.spec.dim))}

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        self.weight = tensors["weight"].to(device).contiguous()

    def _side_by_side(self, x, batch) -> torch.Tensor:
        return batch.workspace.get("junction.concat", (x.shape[0], 2 * self.spec.dim), self.dtype)

    def begin(self, x, batch) -> None:
        core.cast_columns(x, self._side_by_side(x, batch)[:, self.spec.dim:])

    def forward(self, x, batch, passage: int = 0) -> None:
        both = self._side_by_side(x, batch)
        core.cast_columns(x, both[:, :self.spec.dim])
        linear(both, self.weight, None, x)


class PassVector(Junction):
    """``x <- x + steps[passage]``: a learned vector per passage through the junction, ``steps`` ``[passages, dim]``, added
    to every token's row of the fp32 stream."""

    replays_every_step = True

    def __init__(self, spec: PassVectorSpec) -> None:
        super().__init__(spec)
        self.steps: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        return {"steps": ParamSpec((self.spec.passages, self.spec.dim), "matrix", "normal")}

    def bind(self, tensors, dtype, device) -> None:
        self.steps = tensors["steps"].to(device).contiguous()

    def forward(self, x, batch, passage: int = 0) -> None:
        if not 0 <= passage < self.spec.passages:
            raise ValueError(f"passage {passage} through a junction of {self.spec.passages} vectors")
        core.add_vector(x, self.steps[passage])


register_junction("concat_linear", ConcatLinear)
register_junction("pass_vector", PassVector)
