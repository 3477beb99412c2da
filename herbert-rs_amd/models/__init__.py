"""Architectures: each module turns its typed configuration into a ModelSpec and registers itself."""
from . import bozasun, mefatar, modasun, qwen3, vipalorn

__all__ = ["bozasun", "mefatar", "modasun", "qwen3", "vipalorn"]
