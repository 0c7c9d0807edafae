"""The decoder that is built from a ModelSpec, and the built-in architectures: importing this package registers
them (an architecture module registers itself when it is imported; one from outside the package does the same
with ``config.registry.register_architecture``)."""
from . import llama  # noqa: F401
from .decoder import DecoderModel

__all__ = ["DecoderModel"]
