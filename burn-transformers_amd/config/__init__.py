from .base import ConfigError, UnsupportedArchitecture, read_config_json
from .gpt2 import GPT2Config
from .registry import Family, register_family, resolve_family, supported_names, unregister_family

__all__ = ["ConfigError", "UnsupportedArchitecture", "read_config_json", "GPT2Config", "Family",
           "register_family", "resolve_family", "supported_names", "unregister_family"]
