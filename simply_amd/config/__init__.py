"""Configuration: typed per-architecture configs, the architecture-neutral
`ModelSpec`, serving knobs, and `load_config` that picks the config class by
`config.json`'s architecture name."""
from __future__ import annotations

import json
import os
from typing import Any, Mapping

from ..registry import ARCHITECTURES
from .engine import EngineConfig, parse_dtype
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .gemma2 import ConfigError, Gemma2Config


def architecture_name(d: Mapping[str, Any]) -> str:
    archs = d.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)):
        raise ConfigError('config.json: key "architectures" is missing or empty; known: '
                          + ", ".join(ARCHITECTURES.keys()))
    return str(archs[0])


def config_from_dict(d: Mapping[str, Any]):
    """Typed configuration of the architecture that `d` names."""
    return ARCHITECTURES.get(architecture_name(d)).from_dict(d)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path}: no config.json in the model folder")
    with open(path) as f:
        return config_from_dict(json.load(f))


__all__ = ["EngineConfig", "parse_dtype", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry",
           "ConfigError", "Gemma2Config", "architecture_name", "config_from_dict", "load_config"]
