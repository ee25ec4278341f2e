"""Random weights from a configuration and a seed.

Every tensor is drawn from its own generator, seeded by (seed, tensor name): matrices and
biases N(0, std), gains 1 + N(0, gain_std), integer tables uniform.  `write_random_model`
writes a model folder (config.json, model.safetensors) that the engine, and anything else
that reads safetensors, loads like a real checkpoint.  `RandomSource` draws the same kind of
tensors straight on a device, for sizes too large to write out.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable, List

import torch

from ..parts.base import TensorDecl
from .safetensors_io import write_safetensors

STORAGE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def _seed_of(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") & ((1 << 63) - 1)


def draw(decl: TensorDecl, seed: int, std: float, gain_std: float, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed(_seed_of(seed, decl.name))
    if decl.role == "table":
        return torch.randint(0, 1 << 15, decl.shape, generator=g, device=device, dtype=torch.int32)
    t = torch.randn(decl.shape, generator=g, device=device, dtype=torch.float32)
    return t.mul_(gain_std).add_(1.0) if decl.role == "gain" else t.mul_(std)


def required(decls: Iterable[TensorDecl], include_optional: bool) -> List[TensorDecl]:
    seen, out = set(), []
    for d in decls:
        if d.name in seen or (d.optional and not include_optional):
            continue
        seen.add(d.name)
        out.append(d)
    return out


def write_random_model(config, out_dir: str, seed: int = 0, std: float = 0.02, gain_std: float = 0.1,
                       storage: str = "float32", optional: str = "bias") -> str:
    """Write `out_dir/config.json` and `out_dir/model.safetensors` for `config` (a ModelConfig).
    `optional`: which optional tensors are written: "bias" (optional biases yes, an optional
    head no), "all" or "none"."""
    from ..models import build_model_description
    decls = build_model_description(config).tensors()
    keep = []
    for d in required(decls, include_optional=True):
        if d.optional and (optional == "none" or (optional == "bias" and d.role != "bias")):
            continue
        keep.append(d)
    os.makedirs(out_dir, exist_ok=True)
    dt = STORAGE[storage]
    tensors = []
    for d in keep:
        t = draw(d, seed, std, gain_std)
        tensors.append((d.name, t if d.role == "table" else t.to(dt)))
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors, {"format": "pt"})
    cfg = config.to_dict()
    cfg["torch_dtype"] = storage
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)
    return out_dir


class RandomSource:
    """Tensors drawn on `device` when asked for: the same interface as a checkpoint."""

    def __init__(self, decls: Iterable[TensorDecl], seed: int, std: float = 0.02, gain_std: float = 0.1,
                 storage: torch.dtype = torch.bfloat16, optional: str = "bias"):
        self.decls: Dict[str, TensorDecl] = {}
        for d in required(decls, include_optional=True):
            if d.optional and (optional == "none" or (optional == "bias" and d.role != "bias")):
                continue
            self.decls[d.name] = d
        self.seed, self.std, self.gain_std, self.storage = seed, std, gain_std, storage

    def names(self):
        return list(self.decls)

    def __contains__(self, name):
        return name in self.decls

    def shape(self, name):
        return self.decls[name].shape

    def dtype(self, name):
        return torch.int32 if self.decls[name].role == "table" else self.storage

    def tensor(self, name, device="cpu"):
        d = self.decls[name]
        t = draw(d, self.seed, self.std, self.gain_std, device=device)
        return t if d.role == "table" else t.to(self.storage)
