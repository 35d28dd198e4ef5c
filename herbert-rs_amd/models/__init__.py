"""Architectures: each module turns its typed configuration into a ModelSpec and registers itself."""
from . import modasun, qwen3, vipalorn

__all__ = ["modasun", "qwen3", "vipalorn"]
