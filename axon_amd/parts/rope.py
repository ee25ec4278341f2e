"""Rotary position encoding (rotate-half): the frequencies, and the table of a step.

freq_i = theta^(-2i / rotary_dim) in float64 (src/model.rs:638-657); the table of a step is
(sin, cos)(pos * freq_i) computed in float64 on the device and rounded once to float32
(src/model.rs:2612-2621), shared by every layer whose encoding has the same parameters.
Parameters: `head_dim`, `rotary_dim` (the leading dims that rotate; the whole head here),
`theta`.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from .base import PositionEncoding, register_position


class RotaryEncoding(PositionEncoding):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        self.theta = float(params["theta"])
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ConfigError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self.key = None
        self._freqs = None

    def frequencies(self) -> torch.Tensor:
        n = self.rotary_dim // 2
        return torch.tensor([self.theta ** (-2.0 * i / self.rotary_dim) for i in range(n)], dtype=torch.float64)

    def load(self, store, rt) -> None:
        f = self.frequencies()
        # encodings with the same frequencies share one table per step; a subclass that
        # changes the frequencies gets a table of its own
        self.key = ("rotary", tuple(f.tolist()))
        self._freqs = f.to(rt.device)

    def tables(self, ctx) -> torch.Tensor:
        """float32 [T, rotary_dim / 2, 2] for the positions of this step (made once per step)."""
        t = ctx.shared.get(self.key)
        if t is None:
            t = ctx.ws.take((ctx.n_tokens, self.rotary_dim // 2, 2), torch.float32)
            ctx.rt.k.rope_table(ctx.positions, self._freqs, t)
            ctx.shared[self.key] = t
        return t


register_position("rope", RotaryEncoding)
