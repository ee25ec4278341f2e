"""RMSNorm: rows of the 32-bit residual stream, normalised into the compute dtype.

out = (x * 1/sqrt(mean(x^2) + eps)) * gain (src/model.rs:3888-3898).  Parameters: `size`,
`eps`, `tensor` (the gain's name under the part's prefix).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .base import FollowingNorm, Norm, PrecedingNorm, TensorDecl, register_norm


class RMSNorm(Norm):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.name = prefix + params.get("tensor", "weight")
        self.gain = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.size,), "gain")]

    def load(self, store, rt) -> None:
        self.gain = store.vector(self.name)

    def forward(self, ctx, x, out=None, rows: Optional["torch.Tensor"] = None):
        """x: float32 [T, size]; `rows` picks rows of x (the wanted positions before the head)."""
        n = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = ctx.ws.take((n, self.size), ctx.rt.dtype)
        return ctx.rt.k.rmsnorm(x, self.gain, self.eps, out, rows)

    def following(self, ctx, n_rows: int) -> Optional[FollowingNorm]:
        """The product before the norm writes the finished rows (where its kernel offers it)."""
        return FollowingNorm(self.gain, self.eps, ctx.ws.take((n_rows, self.size), ctx.rt.dtype))

    def preceding(self, ctx, x) -> Optional[PrecedingNorm]:
        """The product after the norm reads the float32 rows and norms them on the way (where its
        kernel offers it)."""
        return PrecedingNorm(self, x)


register_norm("rmsnorm", RMSNorm)
