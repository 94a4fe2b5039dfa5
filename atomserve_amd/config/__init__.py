from atomserve_amd.config.engine_config import EngineConfig
from atomserve_amd.config.model_config import ConfigError, Qwen3Config
from atomserve_amd.config.registry import (
    Architecture,
    architecture_for,
    load_model_config,
    register_architecture,
    supported_architectures,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "EngineConfig",
    "Qwen3Config",
    "architecture_for",
    "load_model_config",
    "register_architecture",
    "supported_architectures",
]
