from .base import ConfigError, ModelConfig, read_config_json
from .llama import LlamaConfig
from .nusilix import NusilixConfig, NusilixLayer
from .ribovik import RibovikConfig, RibovikLayer, RibovikMlp, RotaryScaling
from .natenex import NatenexConfig, NatenexLayer
from .lugetar import LugetarConfig, LugetarLayer
from .registry import (Architecture, register_architecture, unregister_architecture,
                       registered_architectures, resolve_architecture, config_from_dict,
                       load_config)

__all__ = [
    "ConfigError", "ModelConfig", "read_config_json", "LlamaConfig", "NusilixConfig", "NusilixLayer", "RibovikConfig", "RibovikLayer", "RibovikMlp", "RotaryScaling", "NatenexConfig", "NatenexLayer", "LugetarConfig", "LugetarLayer", "Architecture",
    "register_architecture", "unregister_architecture", "registered_architectures",
    "resolve_architecture", "config_from_dict", "load_config",
]
