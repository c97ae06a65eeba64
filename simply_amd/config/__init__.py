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
from .zenuzen import ZenuzenConfig
from .nemidra import NemidraConfig
from .tabupel import TabupelConfig
from .rudutar import RudutarConfig


def architecture_name(d: Mapping[str, Any]) -> str:
    archs = d.get("architectures")
    if not archs and isinstance(d.get("architecture"), str):   # (some folders name one architecture, as a string)
        return d["architecture"]
    if not archs or not isinstance(archs, (list, tuple)):
        raise ConfigError('config.json: key "architectures" is missing or empty; known: '
                          + ", ".join(ARCHITECTURES.keys()))
    return str(archs[0])


def config_from_dict(d: Mapping[str, Any], complete: bool = True):
    """Typed configuration of the architecture that `d` names.  complete False: sizes that the architecture reads
    from the tensors' shapes may still be open (`resolve_shapes` closes them)."""
    cls = ARCHITECTURES.get(architecture_name(d))
    if not complete and hasattr(cls, "from_dict_open"):
        return cls.from_dict_open(d)
    return cls.from_dict(d)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path}: no config.json in the model folder")
    with open(path) as f:
        config = config_from_dict(json.load(f), complete=False)
    if hasattr(config, "resolve_shapes"):
        # sizes that the configuration leaves to the tensors' shapes
        from ..weights.loader import stored_shapes

        config = config.resolve_shapes(stored_shapes(model_dir))
    return config


__all__ = ["EngineConfig", "parse_dtype", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry",
           "ConfigError", "Gemma2Config", "ZenuzenConfig", "NemidraConfig", "TabupelConfig", "RudutarConfig", "architecture_name", "config_from_dict", "load_config"]
