"""What every part is handed at run time: the device, the compute dtype and the kernels."""
from __future__ import annotations

import torch

from ..config.engine import dtype_name
from ..kernels import kernels


class Runtime:
    def __init__(self, dtype: str = "bfloat16", device: str = "cuda:0"):
        self.dtype_name = dtype_name(dtype)
        self.dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[self.dtype_name]
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible: the engine runs on an AMD GPU through its HIP kernels and has "
                               "no other path")
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.k = kernels(self.dtype_name)
        self.elem_size = 2 if self.dtype_name == "bfloat16" else 4


class Workspace:
    """Temporary tensors of a step.  Memory comes from the caching allocator, which hands a
    freed block to the next request of its size without touching the device, so a layer's
    temporaries are reused by the next layer; under graph capture they come from the graph's
    own pool and keep their addresses."""

    def __init__(self, device):
        self.device = device

    def take(self, shape, dtype) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype, device=self.device)
