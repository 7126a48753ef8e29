"""Architectures the engine ships; importing this package registers them."""
from . import llama  # noqa: F401
