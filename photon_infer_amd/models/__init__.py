"""Architectures the engine ships; importing this package registers them."""
from . import dafidra, dokanex, llama, muretar, rorevik  # noqa: F401
