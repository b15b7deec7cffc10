"""Architectures the engine ships; importing this package registers them."""
from . import dafidra, llama, rorevik  # noqa: F401
