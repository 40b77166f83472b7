from .base import ConfigError, UnsupportedArchitecture, read_config_json
from .gavasun import GavasunConfig
from .gpt2 import GPT2Config
from .kodatar import KodatarConfig
from .rotutar import RotutarConfig
from .salopel import SalopelConfig
from .registry import Family, register_family, resolve_family, supported_names, unregister_family

__all__ = ["ConfigError", "UnsupportedArchitecture", "read_config_json", "GavasunConfig", "GPT2Config", "KodatarConfig", "RotutarConfig", "SalopelConfig", "Family",
           "register_family", "resolve_family", "supported_names", "unregister_family"]
