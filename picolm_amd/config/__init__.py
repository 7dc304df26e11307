from .llama import ConfigError, LlamaConfig, RopeScaling
from .registry import (Architecture, architecture_name, import_architecture_modules, known_architectures, read_config_json,
                       register_architecture, resolve, unregister_architecture)

__all__ = [
    "ConfigError", "LlamaConfig", "RopeScaling", "Architecture", "architecture_name", "import_architecture_modules",
    "known_architectures", "read_config_json", "register_architecture", "resolve",
    "unregister_architecture",
]
