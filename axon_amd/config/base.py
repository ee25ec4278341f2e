"""Typed reading of config.json and the description of a model as data.

An architecture's configuration class reads its own config.json keys into typed fields and
turns them into a `ModelSpec`: which parts each layer is made of, with their sizes and
constants as parameters, and the order in which layers run.  Nothing below the
configuration knows which model it belongs to.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json the engine refuses, with the key and value that are wrong."""


# --------------------------------------------------------------------------- typed getters

_MISSING = object()


def get_whole(cfg: Dict[str, Any], key: str, default: Any = _MISSING, *, minimum: int = 1) -> Optional[int]:
    """A whole number >= minimum.  The reference refuses anything else with
    "config.json k = v is not a whole number" (src/safetensors.rs:466-504)."""
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(f"config.json is missing {key}")
        return default
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) > 0xFFFFFFFF:
        raise ConfigError(f"config.json {key} = {v!r} is not a whole number")
    v = int(v)
    if v < minimum:
        raise ConfigError(f"config.json {key} = {v} must be at least {minimum}")
    return v


def get_number(cfg: Dict[str, Any], key: str, default: Any = _MISSING, *, positive: bool = True) -> Optional[float]:
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(f"config.json is missing {key}")
        return default
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != v or v in (float("inf"), float("-inf")):
        raise ConfigError(f"config.json {key} = {v!r} is not a number")
    if positive and not v > 0:
        raise ConfigError(f"config.json {key} = {v} must be above 0")
    return float(v)


def get_flag(cfg: Dict[str, Any], key: str, default: bool) -> bool:
    v = cfg.get(key, None)
    if v is None:
        return default
    if not isinstance(v, bool):
        raise ConfigError(f"config.json {key} = {v!r} is not true or false")
    return v


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path) as f:
            cfg = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{model_dir} has no config.json") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not JSON: {e}") from None
    if not isinstance(cfg, dict):
        raise ConfigError("config.json is not a JSON object")
    if os.path.isfile(os.path.join(model_dir, "hf_quant_config.json")):
        # src/safetensors.rs:1444-1449: a quantized export names itself in a file of its own
        raise ConfigError("quantized checkpoint (hf_quant_config.json): quantized weights are not supported")
    return cfg


# --------------------------------------------------------------------------- a model as data

@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: the name it is registered under and its parameters."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, json.dumps(self.params, sort_keys=True, default=str)))


@dataclass(frozen=True)
class LayerSpec:
    """A layer: how its parts are arranged (`block`), and the parts.  `prefix` is where its
    tensors live in the checkpoint ("model.layers.3.")."""
    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norm: PartSpec
    prefix: str


@dataclass(frozen=True)
class Run:
    """One entry of the execution order: run `layer` with the cache `cache`.  Two runs may name
    the same layer (its weights are used twice); a run whose `cache` is another run's, with
    `writes_cache` false, reads what that run wrote and stores nothing of its own."""
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    """Everything the builder needs: embedding, layers, their order, final norm, head."""
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    order: List[Run]
    final_norm: PartSpec
    head: PartSpec
    max_positions: int


class ModelConfig:
    """What an architecture's configuration must offer (see `Qwen2Config` for one):

    * ``architecture``: the name config.json's ``architectures[0]`` carries;
    * ``from_dict(cfg)``: the typed reading, refusing what it cannot run;
    * ``to_dict()``: back to config.json keys (the random-weights mode writes it);
    * ``model_spec()``: the model as data;
    * ``tensor_shapes()``: every checkpoint tensor's name and shape (the loader's check and
      the random-weights mode both come from it).
    """
    architecture: str = ""

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError

    # ---- what a checkpoint of this architecture may look like (hooks; the defaults fit most)
    def vocab_tensor(self) -> Optional[str]:
        """If config.json may lack the vocabulary's size: the tensor whose first dimension is it
        (the loader then calls `with_vocab`).  None: the configuration always knows it."""
        return None

    def with_vocab(self, vocab_size: int) -> "ModelConfig":
        raise NotImplementedError

    def ignores_tensor(self, name: str) -> bool:
        """Tensors a checkpoint may hold that the model does not read (tables that are
        recomputed, say): they are neither unexpected nor loaded."""
        return False

    def model_spec(self) -> ModelSpec:
        raise NotImplementedError
