"""Rotary position encoding on the first ``rotary_dim`` channels of each head."""

from __future__ import annotations

from typing import Optional

import torch

from .base import PositionEncoding, Rotation, register_position
from .specs import PositionSpec


class NeoxRotary(PositionEncoding):
    """Non-interleaved rotation: channel ``i`` pairs with ``i + rotary_dim / 2``.

    Table row ``p`` = ``[cos(p f_0), .., cos(p f_{R/2-1}), sin(p f_0), ..]`` with
    ``f_i = theta ** (-2 i / R)``, all in fp32
    (``kestrel/models/moondream/rope.py:6-32``; applied at ``text.py:123-125``).
    """

    replays_every_step = True

    def __init__(self, spec: PositionSpec) -> None:
        super().__init__(spec)
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even")
        if spec.rotary_dim and spec.max_positions <= 0:
            raise ValueError("a rotary encoding needs max_positions")
        self._table: Optional[torch.Tensor] = None

    def rotation(self, device: torch.device) -> Optional[Rotation]:
        table = self.table(device)
        return None if table is None else Rotation(table, "halves")

    def table(self, device: torch.device) -> Optional[torch.Tensor]:
        spec = self.spec
        if spec.rotary_dim == 0:
            return None
        if self._table is None or self._table.device != device:
            exponents = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float32) / float(spec.rotary_dim)
            inv_freq = 1.0 / (float(spec.theta) ** exponents)
            angles = torch.arange(spec.max_positions, dtype=torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
            self._table = torch.cat([torch.cos(angles), torch.sin(angles)], dim=-1).contiguous().to(device)
        return self._table


def rotary_frequencies(rotary_dim: int, theta: float, scaling=None):
    """``f_i = theta ** (-2 i / rotary_dim)`` for the ``rotary_dim / 2`` pairs, rescaled by wavelength where a
    ``WavelengthScaling`` is given (long wavelengths divided by its factor, short ones kept, a linear blend between),
    or all divided by the factor of a ``LinearScaling``."""
    import math

    out = []
    for i in range(rotary_dim // 2):
        f = float(theta) ** (-2.0 * i / rotary_dim)
        if scaling is not None and not hasattr(scaling, "original"):
            f = f / float(scaling.factor)
        elif scaling is not None:
            wavelength = 2.0 * math.pi / f
            if wavelength > scaling.original / scaling.low:
                f = f / scaling.factor
            elif wavelength >= scaling.original / scaling.high:
                s = (scaling.original / wavelength - scaling.low) / (scaling.high - scaling.low)
                f = (1.0 - s) * f / scaling.factor + s * f
        out.append(f)
    return out


class FrequencyRotary(PositionEncoding):
    """A rotation given by its frequencies alone: the kernels compute the angle ``place * f_i`` and its cosine and sine
    in fp32 themselves, so there is no table and no longest sequence. ``spec.pairing`` says which channels angle ``i``
    turns (``"halves"`` or ``"interleaved"``), ``spec.scaling`` rescales the frequencies (by wavelength, or all alike)."""

    replays_every_step = True

    def __init__(self, spec: PositionSpec) -> None:
        super().__init__(spec)
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even and positive")
        self._freqs: Optional[torch.Tensor] = None

    def rotation(self, device: torch.device) -> Optional[Rotation]:
        spec = self.spec
        if self._freqs is None or self._freqs.device != device:
            values = rotary_frequencies(spec.rotary_dim, spec.theta, getattr(spec, "scaling", None))
            self._freqs = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(device)
        return Rotation(None, getattr(spec, "pairing", "halves"), self._freqs)


class NoPosition(PositionEncoding):
    """Encodes nothing (a mixer whose order comes from elsewhere)."""

    replays_every_step = True


register_position("rotary_neox", NeoxRotary)
register_position("rotary", FrequencyRotary)
register_position("none", NoPosition)
