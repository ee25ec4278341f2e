"""From a model folder (or a configuration and a seed) to a loaded model on the device."""
from __future__ import annotations

from typing import Optional

import torch

from ..config import ModelConfig, config_from_dict, read_config_json
from ..models import DecoderModel, build_model_description
from ..weights import Checkpoint, CheckpointSource, RandomSource, WeightStore, check_tensors
from .runtime import Runtime


def read_model_config(model_dir: str, checkpoint: Optional[Checkpoint] = None) -> ModelConfig:
    """config.json through the registry.  A configuration that does not know its vocabulary yet
    names the tensor that does (`ModelConfig.vocab_tensor`)."""
    config = config_from_dict(read_config_json(model_dir))
    name = config.vocab_tensor()
    if name is not None:
        ck = checkpoint or Checkpoint(model_dir)
        if name not in ck:
            from ..weights import WeightError
            raise WeightError([name], [], [])
        config = config.with_vocab(ck.shape(name)[0])
    return config


def load_model(model_dir: str, rt: Runtime) -> DecoderModel:
    ck = Checkpoint(model_dir)
    config = read_model_config(model_dir, ck)
    model = build_model_description(config)
    source = CheckpointSource(ck)
    check_tensors(model.tensors(), source, config.ignores_tensor)
    model.load(WeightStore(source, rt.device, rt.dtype), rt)
    _release_staging(rt)
    return model


def random_model(config: ModelConfig, rt: Runtime, seed: int = 0, std: float = 0.02) -> DecoderModel:
    """A model whose weights are drawn on the device (nothing is written)."""
    model = build_model_description(config)
    storage = torch.bfloat16 if rt.dtype == torch.bfloat16 else torch.float32
    source = RandomSource(model.tensors(), seed, std=std, storage=storage)
    model.load(WeightStore(source, rt.device, rt.dtype), rt)
    _release_staging(rt)
    return model


def _release_staging(rt: Runtime) -> None:
    """The row-major copies that were repacked are gone; give their memory back to the device,
    so that the cache pool, which is sized from what is free, can have it."""
    if rt.device is not None and torch.cuda.is_available():
        torch.cuda.synchronize(rt.device)
        torch.cuda.empty_cache()
