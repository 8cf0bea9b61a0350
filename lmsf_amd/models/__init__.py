"""Architectures. Importing this package registers the built-in ones."""
from . import llama  # noqa: F401  (registration)
from .decoder import DecoderModel

__all__ = ["DecoderModel"]
