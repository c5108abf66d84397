from .engine import ModelConfig, ServerConfig, parse_overrides
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

__all__ = [
    "ARCHITECTURES",
    "Architecture",
    "ConfigError",
    "LayerRun",
    "LayerSpec",
    "Llama3RopeScaling",
    "LlamaConfig",
    "ModelConfig",
    "ModelSpec",
    "PartSpec",
    "ServerConfig",
    "get_architecture",
    "parse_config",
    "parse_overrides",
    "read_config",
    "register_architecture",
]
