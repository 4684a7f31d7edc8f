"""An inference engine for the Qwen2.5 dense decoder on one AMD MI355X (gfx950)."""

from . import models  # noqa: F401  registers the architectures
from . import parts   # noqa: F401  registers the built-in parts
from .config import (ConfigError, EngineConfig, known_architectures, read_config, read_config_dict,
                     register_architecture)
from .weights import WeightsError, write_model_folder

__all__ = ["ConfigError", "EngineConfig", "WeightsError", "known_architectures", "read_config",
           "read_config_dict", "register_architecture", "write_model_folder"]
