"""Sampling settings, the random stream, and picks for the rows of a step.

Names and meanings of the settings are the reference's flags (src/sample.rs:101-190,
src/cli.rs:219-230): `temperature` (--temp; 0 = greedy: the highest logit, no penalty, no
other setting applies), `top_k` (40; 0 = off), `top_p` (0.9; 1 = off), `min_p` (0 = off),
`repeat_penalty` (1.1; 1 = off), `repeat_last_n` (64; 0 = off), `seed`.  They apply in the
order penalty -> top-k -> top-p -> min-p -> temperature -> draw, one draw per decided token.

Greedy rows are picked by the device's argmax; sampled rows get their penalty and top-k on the
device (k up to 1024) and only k candidates travel to the host, where the native sampler
finishes; a row with top-k off travels whole.
"""
from __future__ import annotations

import ctypes
import os
import time
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import host_lib

DEVICE_TOPK_MAX = 1024


@dataclass
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 40
    top_p: float = 0.9
    min_p: float = 0.0
    repeat_penalty: float = 1.1
    repeat_last_n: int = 64
    seed: Optional[int] = None

    def __post_init__(self):
        if not 0.0 <= self.temperature <= 100.0:
            raise ValueError(f"--temp needs a number from 0 to 100, got '{self.temperature}'")
        if self.top_k < 0 or self.repeat_last_n < 0:
            raise ValueError("--top-k and --repeat-last-n need whole numbers")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError(f"--top-p needs a number from 0 to 1, got '{self.top_p}'")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError(f"--min-p needs a number from 0 to 1, got '{self.min_p}'")
        if not 0.0 < self.repeat_penalty <= 100.0:
            raise ValueError("--repeat-penalty must be above 0 (1 = off)")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0


def random_seed() -> int:
    """A seed from the clock and the process id (src/sample.rs:192-200)."""
    return (time.time_ns() ^ (os.getpid() << 32)) & ((1 << 64) - 1)


class Rng:
    """xoshiro256** seeded through splitmix64 (src/sample.rs:212-242)."""

    def __init__(self, seed: int):
        self._lib = host_lib()
        self.state = (ctypes.c_uint64 * 4)()
        self._lib.axh_rng_seed(ctypes.c_uint64(seed & ((1 << 64) - 1)), self.state)

    def next_u64(self) -> int:
        return self._lib.axh_rng_next_u64(self.state)

    def f64(self) -> float:
        return self._lib.axh_rng_next_f64(self.state)


class Sampler:
    """One generation stream: its settings and its random numbers."""

    def __init__(self, params: SamplingParams):
        self.params = params
        self.seed = params.seed if params.seed is not None else random_seed()
        self.rng = Rng(self.seed)
        self._lib = host_lib()

    def recent(self, history: Sequence[int]) -> List[int]:
        n = self.params.repeat_last_n
        if n == 0 or self.params.repeat_penalty == 1.0:
            return []
        return list(history[-n:])

    def pick_keys(self, keys: torch.Tensor) -> int:
        """From the device's k candidate keys (a CPU int64 tensor)."""
        p = self.params
        return self._lib.axh_sample_pick_keys(ctypes.c_void_p(keys.data_ptr()), keys.numel(), p.temperature, p.top_p,
                                              p.min_p, self.rng.f64())

    def pick_row(self, logits: torch.Tensor, history: Sequence[int]) -> int:
        """From a whole row held by the host (a CPU float32 tensor)."""
        p = self.params
        rec = self.recent(history)
        arr = (ctypes.c_int * max(len(rec), 1))(*rec)
        return self._lib.axh_sample_pick_row(ctypes.c_void_p(logits.data_ptr()), logits.numel(), arr, len(rec),
                                             p.repeat_penalty, p.top_k, p.temperature, p.top_p, p.min_p, self.rng.f64())


def argmax_row(logits: torch.Tensor) -> int:
    """The greedy pick of a host row: of equal maxima the last, NaN never."""
    logits = logits.contiguous()
    return host_lib().axh_argmax_row(ctypes.c_void_p(logits.data_ptr()), logits.numel())


def pick_rows(rt, logits: torch.Tensor, samplers: Sequence[Optional[Sampler]],
              histories: Sequence[Sequence[int]]) -> List[int]:
    """The next token of every row of `logits` (device, float32 [rows, vocab]).  `samplers[r]`
    is None for a greedy row; `histories[r]` is the row's tokens so far, the one the logits
    follow included.  Sampled rows' logits are penalised in place."""
    rows, vocab = logits.shape
    picks: List[Optional[int]] = [None] * rows
    greedy = [r for r in range(rows) if samplers[r] is None or samplers[r].params.greedy]
    device_rows = [r for r in range(rows) if r not in greedy and 1 <= samplers[r].params.top_k <= DEVICE_TOPK_MAX]
    host_rows = [r for r in range(rows) if r not in greedy and r not in device_rows]
    dev = logits.device
    if greedy:
        if len(greedy) == rows:
            out = torch.empty(rows, dtype=torch.int32, device=dev)
            rt.k.argmax(logits, out)
            for r, v in enumerate(out.tolist()):
                picks[r] = v
        else:
            sel = logits[torch.tensor(greedy, device=dev)]
            out = torch.empty(len(greedy), dtype=torch.int32, device=dev)
            rt.k.argmax(sel, out)
            for r, v in zip(greedy, out.tolist()):
                picks[r] = v
    if device_rows:
        n = len(device_rows)
        recents = [samplers[r].recent(histories[r]) for r in device_rows]
        width = max(1, max(len(x) for x in recents))
        ks = [min(samplers[r].params.top_k, vocab) for r in device_rows]
        # one copy to the device: the recent tokens, how many, k, and the penalties' bits
        flat = np.zeros(n * width + 3 * n, dtype=np.int32)
        rec = flat[:n * width].reshape(n, width)
        for i, x in enumerate(recents):
            rec[i, :len(x)] = x
        flat[n * width:n * width + n] = [len(x) for x in recents]
        flat[n * width + n:n * width + 2 * n] = ks
        flat[n * width + 2 * n:].view(np.float32)[:] = [samplers[r].params.repeat_penalty for r in device_rows]
        on = torch.from_numpy(flat).to(dev)
        sel = logits if n == rows else logits[torch.tensor(device_rows, device=dev)].contiguous()
        cands = torch.empty((n, max(ks)), dtype=torch.int64, device=dev)      # a row's first k places are written
        rt.k.topk(sel, on[:n * width].view(n, width), on[n * width:n * width + n], on[n * width + 2 * n:].view(torch.float32),
                  on[n * width + n:n * width + 2 * n], cands, k_max=max(ks))
        host = cands.cpu()
        for i, r in enumerate(device_rows):
            picks[r] = samplers[r].pick_keys(host[i, :ks[i]].contiguous())
    for r in host_rows:
        picks[r] = samplers[r].pick_row(logits[r].cpu().contiguous(), histories[r])
    return picks
