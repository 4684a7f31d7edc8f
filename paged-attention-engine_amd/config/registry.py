"""One registry from an architecture's name to the code that reads its config.

The reference constructs its only model class directly (README.md:33-34,
engine/model.py:164); a registry is this engine's own addition so that the model
class is chosen by `architectures[0]` of config.json everywhere.
"""

from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict, Mapping

from .model_config import ConfigError, ModelPlan

# name -> callable(config.json dict) -> typed config object with a .plan() method
_ARCHITECTURES: Dict[str, Callable[[Mapping[str, Any]], Any]] = {}


def register_architecture(name: str, config_reader: Callable[[Mapping[str, Any]], Any]) -> None:
    """`config_reader(dict)` returns an object with `.plan() -> ModelPlan` and
    `.to_json_dict() -> dict` (the config.json it would be read from)."""
    _ARCHITECTURES[name] = config_reader


def known_architectures():
    return tuple(sorted(_ARCHITECTURES))


def read_config_dict(cfg: Mapping[str, Any]):
    archs = cfg.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)):
        raise ConfigError("config.json lacks the key 'architectures'")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture '{name}'; known: {', '.join(known_architectures()) or '(none)'}")
    return _ARCHITECTURES[name](cfg)


def read_config(model_dir: str):
    """Typed config of the model folder `model_dir` (reads its config.json)."""
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as handle:
            cfg = json.load(handle)
    except FileNotFoundError as err:
        raise ConfigError(f"{path}: no such file") from err
    except json.JSONDecodeError as err:
        raise ConfigError(f"{path}: not JSON ({err})") from err
    return read_config_dict(cfg)


def plan_of(model_dir_or_dict) -> ModelPlan:
    cfg = read_config(model_dir_or_dict) if isinstance(model_dir_or_dict, str) else read_config_dict(model_dir_or_dict)
    return cfg.plan()
