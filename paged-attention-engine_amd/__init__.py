"""An inference engine for the Qwen2.5 dense decoder on one AMD MI355X (gfx950)."""

from . import models  # noqa: F401  registers the architectures
from . import parts   # noqa: F401  registers the built-in parts
from .cache import BlockAllocator, CacheManager
from .config import (ConfigError, EngineConfig, known_architectures, read_config, read_config_dict,
                     register_architecture)
from .engine.executor import ModelExecutor
from .engine.llm import Engine, GenerationResult
from .engine.model import Model, expected_tensors, load_model, random_model
from .engine.scheduler import (Event, EventKind, Request, Scheduler, Sequence, SequenceStatus, StepResult,
                               is_admissible)
from .engine.step import StepEntry, StepRunner
from .weights import RandomWeights, WeightsError, load_weights, write_model_folder

__all__ = ["BlockAllocator", "CacheManager", "ConfigError", "Engine", "EngineConfig", "Event", "EventKind",
           "GenerationResult", "Model", "ModelExecutor", "Request", "Scheduler", "Sequence", "SequenceStatus",
           "StepEntry", "StepResult", "StepRunner", "WeightsError", "expected_tensors", "is_admissible",
           "known_architectures", "load_model", "load_weights", "random_model", "read_config", "read_config_dict",
           "register_architecture", "write_model_folder", "RandomWeights"]
