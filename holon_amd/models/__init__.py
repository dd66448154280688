"""Architectures. Importing this package registers them by their config.json name."""
from . import dopirax, nevodra, qwen3, relanex, tolurax

__all__ = ["dopirax", "nevodra", "qwen3", "relanex", "tolurax"]
