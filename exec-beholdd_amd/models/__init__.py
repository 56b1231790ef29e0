"""Models: the generic decoder and the architectures registered on it."""

from .decoder import DecoderModel, build_decoder
from . import qwen3

__all__ = ["DecoderModel", "build_decoder", "qwen3"]
