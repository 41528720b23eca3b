from .base import ConfigError
from .gufasun import GufasunConfig
from .qwen3 import Qwen3Config
from .retudra import RetudraConfig
from .sovutar import SovutarConfig
from .tazitar import TazitarConfig
from .registry import (Architecture, detect_architecture, known_architectures, load_model_config,
                       register_architecture)

__all__ = ["ConfigError", "Qwen3Config", "GufasunConfig", "SovutarConfig", "TazitarConfig", "RetudraConfig", "Architecture", "detect_architecture",
           "known_architectures", "load_model_config", "register_architecture"]
