from .base import ConfigError
from .gufasun import GufasunConfig
from .qwen3 import Qwen3Config
from .sovutar import SovutarConfig
from .registry import (Architecture, detect_architecture, known_architectures, load_model_config,
                       register_architecture)

__all__ = ["ConfigError", "Qwen3Config", "GufasunConfig", "SovutarConfig", "Architecture", "detect_architecture",
           "known_architectures", "load_model_config", "register_architecture"]
