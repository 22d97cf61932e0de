from .base import ConfigError, ModelConfig, read_config_json
from .dizizen import DizizenConfig
from .gimozen import GimozenConfig
from .gpt2 import GPT2Config
from .ketolix import KetolixConfig
from .perezen import PerezenConfig
from .registry import (
    Architecture,
    architecture_name,
    config_from_dict,
    get_architecture,
    load_config,
    register_architecture,
    registered_architectures,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "DizizenConfig",
    "GimozenConfig",
    "GPT2Config",
    "KetolixConfig",
    "ModelConfig",
    "PerezenConfig",
    "architecture_name",
    "config_from_dict",
    "get_architecture",
    "load_config",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
]
