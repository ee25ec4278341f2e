"""One registry from an architecture's name to its configuration class.

config.json's ``architectures[0]`` (or, where it is absent, ``model_type``) names the
architecture, as the reference decides it (src/safetensors.rs:437-463); the class found here
reads the rest of config.json and describes the model.  Another architecture is added with
`register_architecture`, from anywhere: the engine's files need no change.
"""
from __future__ import annotations

from typing import Any, Dict, Type

from .base import ConfigError, ModelConfig, read_config_json

_ARCHITECTURES: Dict[str, Type[ModelConfig]] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_class: Type[ModelConfig], model_type: str = "") -> None:
    """Make `name` (as in config.json's ``architectures``) known; `model_type` is the
    ``model_type`` value that also selects it."""
    _ARCHITECTURES[name] = config_class
    if model_type:
        _MODEL_TYPES[model_type] = name


def known_architectures():
    return sorted(_ARCHITECTURES)


def architecture_of(cfg: Dict[str, Any]) -> str:
    """`model_type` decides if it is a known one; else `architectures[0]`."""
    mt = cfg.get("model_type") or ""
    archs = cfg.get("architectures") or []
    hf = archs[0] if isinstance(archs, list) and archs and isinstance(archs[0], str) else ""
    if isinstance(mt, str) and mt in _MODEL_TYPES:
        return _MODEL_TYPES[mt]
    if hf in _ARCHITECTURES:
        return hf
    shown = mt if mt else hf
    raise ConfigError(
        f"model_type '{shown}' is not supported ({', '.join(known_architectures()) or 'none registered'})")


def config_from_dict(cfg: Dict[str, Any]) -> ModelConfig:
    return _ARCHITECTURES[architecture_of(cfg)].from_dict(cfg)


def config_from_dir(model_dir: str) -> ModelConfig:
    return config_from_dict(read_config_json(model_dir))
