from .engine import EngineConfig, canonical_dtype
from .errors import ConfigError
from .model import config_value, read_config_json
from .registry import (
    Architecture,
    architecture_name,
    get_architecture,
    register_architecture,
    resolve,
    supported_architectures,
)

__all__ = [
    "EngineConfig", "canonical_dtype", "ConfigError", "config_value", "read_config_json", "Architecture",
    "architecture_name", "get_architecture", "register_architecture", "resolve", "supported_architectures",
]
