from .base import ConfigError, KeyReader, read_json
from .bubetar import BubetarConfig
from .kezolix import KezolixConfig
from .nebanex import NebanexConfig
from .pekasun import PekasunConfig
from .qwen2 import Qwen2Config
from .registry import (
    Architecture,
    UnknownArchitectureError,
    load_model_config,
    register_architecture,
    registered_architectures,
    resolve_architecture,
    unregister_architecture,
)

__all__ = [
    "Architecture",
    "BubetarConfig",
    "ConfigError",
    "KeyReader",
    "KezolixConfig",
    "NebanexConfig",
    "PekasunConfig",
    "Qwen2Config",
    "UnknownArchitectureError",
    "load_model_config",
    "read_json",
    "register_architecture",
    "registered_architectures",
    "resolve_architecture",
    "unregister_architecture",
]
