"""Architectures the engine ships; importing this package registers them."""
from . import dafidra, llama  # noqa: F401
