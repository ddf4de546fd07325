from wllm_amd.config.gemma import GemmaConfig
from wllm_amd.config.registry import (
    ArchitectureEntry,
    ConfigError,
    read_config_json,
    register_architecture,
    registered_architectures,
    resolve_architecture,
)

__all__ = [
    "ArchitectureEntry",
    "ConfigError",
    "GemmaConfig",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
    "resolve_architecture",
]
