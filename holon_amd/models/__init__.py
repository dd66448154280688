"""Architectures. Importing this package registers them by their config.json name."""
from . import nevodra, qwen3, relanex, tolurax

__all__ = ["nevodra", "qwen3", "relanex", "tolurax"]
