"""Typed configurations and the architecture registry."""
from .base import read_config_json
from .registry import (Architecture, ChatFormat, load_config, register_architecture,
                       registered_architectures, resolve_architecture)
from .qwen3 import Qwen3Config
from .vipalorn import VipalornConfig
from .modasun import ModasunConfig
from .mefatar import MefatarConfig
from .bozasun import BozasunConfig

__all__ = ["Architecture", "BozasunConfig", "ChatFormat", "MefatarConfig", "ModasunConfig", "Qwen3Config", "VipalornConfig", "load_config", "read_config_json",
           "register_architecture", "registered_architectures", "resolve_architecture"]
