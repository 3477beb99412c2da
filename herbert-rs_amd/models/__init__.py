"""Architectures: each module turns its typed configuration into a ModelSpec and registers itself."""
from . import mefatar, modasun, qwen3, vipalorn

__all__ = ["mefatar", "modasun", "qwen3", "vipalorn"]
