from .model_config import ConfigError, LlamaConfig, RopeScaling, read_config_json
from .feduzen_config import FeduzenConfig
from .mogisun_config import MogisunConfig
from .famepel_config import FamepelConfig
from .tadinex_config import TadinexConfig
from .engine_config import EngineConfig, resolve_dtype
from .registry import (
    Architecture, UnknownArchitecture, architecture_name, architecture_of, get_architecture,
    known_architectures, register_architecture, unregister_architecture,
)
from .presets import PRESETS, preset

__all__ = [
    "ConfigError", "FamepelConfig", "FeduzenConfig", "LlamaConfig", "MogisunConfig", "RopeScaling", "TadinexConfig", "read_config_json",
    "EngineConfig", "resolve_dtype",
    "Architecture", "UnknownArchitecture", "architecture_name", "architecture_of", "get_architecture",
    "known_architectures", "register_architecture", "unregister_architecture",
    "PRESETS", "preset",
]
