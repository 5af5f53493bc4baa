from .diporax import DiporaxConfig
from .engine import ModelConfig, ServerConfig, parse_overrides
from .kavuvik import KavuvikConfig
from .model import Llama3RopeScaling, LlamaConfig
from .registry import (
    ARCHITECTURES,
    Architecture,
    ConfigError,
    get_architecture,
    parse_config,
    read_config,
    register_architecture,
)
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec
from .vepitar import VepitarConfig
from .zabunex import ZabunexConfig

__all__ = [
    "ARCHITECTURES",
    "Architecture",
    "ConfigError",
    "DiporaxConfig",
    "KavuvikConfig",
    "LayerRun",
    "LayerSpec",
    "Llama3RopeScaling",
    "LlamaConfig",
    "ModelConfig",
    "ModelSpec",
    "PartSpec",
    "ServerConfig",
    "VepitarConfig",
    "ZabunexConfig",
    "get_architecture",
    "parse_config",
    "parse_overrides",
    "read_config",
    "register_architecture",
]
