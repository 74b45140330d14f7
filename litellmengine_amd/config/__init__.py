from .model_config import ConfigError, Qwen3Config, read_config_json, FULL_ATTENTION, SLIDING_ATTENTION
from .visadra_config import VisadraConfig
from .kezasun_config import KezasunConfig
from .malilorn_config import MalilornConfig
from .birelix_config import BirelixConfig
from .registry import (
    Architecture,
    architecture_of,
    get_architecture,
    load_config,
    register_architecture,
    registered_architectures,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "Qwen3Config",
    "VisadraConfig",
    "KezasunConfig",
    "MalilornConfig",
    "BirelixConfig",
    "FULL_ATTENTION",
    "SLIDING_ATTENTION",
    "architecture_of",
    "get_architecture",
    "load_config",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
]
