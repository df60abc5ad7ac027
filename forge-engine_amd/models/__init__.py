"""The generic decoder and the architectures registered on it."""

from .decoder import DecoderModel

__all__ = ["DecoderModel"]
