"""Architectures; each module registers itself in ``kestrel_amd.config.registry`` on import."""

from . import bogivik, bokorax, letevik, moondream, vimesun  # noqa: F401
from .decoder import DecoderModel

__all__ = ["DecoderModel"]
