"""Weights by tensor name, checked against what the model's parts declare.

`check_tensors` compares the declared tensors with a checkpoint and raises ONE error that
lists every missing tensor, every unexpected one and every wrong shape or unusable dtype
(the reference checks the same things up front: src/model.rs:1491-1541, 1581-1607;
src/safetensors.rs:1553-1558; what the architecture says it does not read is skipped, as
`*.rotary_emb.inv_freq` is there: src/safetensors.rs:1157-1159).

`WeightStore` hands tensors to the parts on the device.  Storage rule: a matrix is kept in the
compute dtype (bfloat16 for serving; float32 for the 32-bit path, where a bfloat16 checkpoint
is widened exactly); a vector (gain, bias) keeps 32-bit storage if it was stored so and
bfloat16 otherwise, except on the 32-bit path where everything is float32; integer tables
are int32.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence

import torch

from ..parts.base import TensorDecl

FLOAT_DTYPES = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
INT_DTYPES = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


class WeightError(ValueError):
    """What is wrong with a checkpoint, all of it at once."""

    def __init__(self, missing: Sequence[str], unexpected: Sequence[str], wrong: Sequence[str]):
        self.missing, self.unexpected, self.wrong = list(missing), list(unexpected), list(wrong)
        lines = ["the checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong:
            lines.append(f"  wrong shape or dtype ({len(self.wrong)}): " + "; ".join(self.wrong))
        super().__init__("\n".join(lines))


def check_tensors(decls: Iterable[TensorDecl], source, ignored=None) -> None:
    """`source` offers names(), shape(name), dtype(name); `ignored(name)` says which of its
    tensors the architecture knows and does not read (`ModelConfig.ignores_tensor`)."""
    decls = list(decls)
    declared: Dict[str, TensorDecl] = {}
    for d in decls:
        declared.setdefault(d.name, d)
    have = [n for n in source.names() if not (ignored is not None and ignored(n))]
    have_set = set(have)
    missing = [d.name for d in declared.values() if not d.optional and d.name not in have_set]
    unexpected = sorted(n for n in have if n not in declared)
    wrong = []
    for name, d in declared.items():
        if name not in have_set:
            continue
        shape, dt = tuple(source.shape(name)), source.dtype(name)
        if shape != tuple(d.shape):
            wrong.append(f"{name} has shape {list(shape)}, the model needs {list(d.shape)}")
        elif d.role == "table" and dt not in INT_DTYPES:
            wrong.append(f"{name} is {dt}, an integer table is needed")
        elif d.role != "table" and dt not in FLOAT_DTYPES:
            wrong.append(f"{name} is {dt}, a floating-point tensor is needed")
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong)


class WeightStore:
    """Tensors for the parts, on `device`, in the storage the rule above gives them."""

    def __init__(self, source, device, dtype: torch.dtype):
        self.source = source
        self.device = device
        self.dtype = dtype
        self._matrices: Dict[str, torch.Tensor] = {}

    def has(self, name: str) -> bool:
        return name in self.source

    def matrix(self, name: str, optional: bool = False) -> Optional[torch.Tensor]:
        if name in self._matrices:      # a tied head shares the embedding's storage
            return self._matrices[name]
        if not self.has(name):
            if optional:
                return None
            raise KeyError(f"missing tensor {name}")
        t = self.source.tensor(name, self.device).to(device=self.device, dtype=self.dtype).contiguous()
        self._matrices[name] = t
        return t

    def forget(self, name: str) -> None:
        """Drop the store's reference to a matrix (its user keeps another form of it)."""
        self._matrices.pop(name, None)

    def fused_matrix(self, names: List[str]) -> torch.Tensor:
        """The named [rows_i, K] matrices stacked into one [sum rows_i, K]."""
        shapes = [tuple(self.source.shape(n)) for n in names]
        out = torch.empty((sum(s[0] for s in shapes), shapes[0][1]), dtype=self.dtype, device=self.device)
        at = 0
        for n, s in zip(names, shapes):
            out[at:at + s[0]].copy_(self.source.tensor(n, self.device))
            at += s[0]
        return out

    def vector(self, name: str, optional: bool = False) -> Optional[torch.Tensor]:
        if not self.has(name):
            if optional:
                return None
            raise KeyError(f"missing tensor {name}")
        t = self.source.tensor(name, self.device)
        if self.dtype == torch.float32 or t.dtype in (torch.float32, torch.float64):
            want = torch.float32
        else:
            want = torch.bfloat16
        return t.to(device=self.device, dtype=want).contiguous()

    def table(self, name: str) -> torch.Tensor:
        return self.source.tensor(name, self.device).to(device=self.device, dtype=torch.int32).contiguous()


class CheckpointSource:
    """A model folder's tensors (see `safetensors_io.Checkpoint`)."""

    def __init__(self, checkpoint):
        self.ck = checkpoint

    def names(self):
        return self.ck.names()

    def __contains__(self, name):
        return name in self.ck

    def shape(self, name):
        return self.ck.shape(name)

    def dtype(self, name):
        return self.ck.dtype(name)

    def tensor(self, name, device=None):
        return self.ck.tensor(name)
