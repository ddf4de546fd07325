"""Reading config.json and the one registry from an architecture's name to its model.  The typed
configuration of an architecture lives with the architecture (`wllm_amd/architectures`)."""
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
    "read_config_json",
    "register_architecture",
    "registered_architectures",
    "resolve_architecture",
]
