"""Architectures; each module registers itself in ``kestrel_amd.config.registry`` on import."""

from . import moondream  # noqa: F401
from .decoder import DecoderModel

__all__ = ["DecoderModel"]
