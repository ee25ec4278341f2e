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


class _Pinned:
    """Pinned host buffers that are used again: a ring per (purpose, dtype, size class), so that a
    buffer is written again only long after the copy that read it has run."""

    def __init__(self):
        self.rings = {}

    def take(self, purpose: str, numel: int, dtype) -> torch.Tensor:
        size = 1 << max(6, (max(numel, 1) - 1).bit_length())
        ring = self.rings.setdefault((purpose, dtype, size), {"at": 0, "bufs": []})
        if len(ring["bufs"]) < 8:
            ring["bufs"].append(torch.empty(size, dtype=dtype).pin_memory())
            return ring["bufs"][-1][:numel]
        ring["at"] = (ring["at"] + 1) % 8
        return ring["bufs"][ring["at"]][:numel]


_PINNED = _Pinned()


class PendingRowPicks:
    """The picks of a step's rows, decided in two halves: what runs on the device is queued when
    this is made (penalty and top-k, the copy of the candidates), `finish()` waits for it and
    lets the native sampler draw.  Between the two the host is free to prepare the next step."""

    def __init__(self, rt, logits: torch.Tensor, samplers: Sequence[Optional[Sampler]], histories: Sequence[Sequence[int]]):
        rows, vocab = logits.shape
        self.samplers, self.histories, self.logits = samplers, histories, logits
        self.picks: List[Optional[int]] = [None] * rows
        self.greedy = [r for r in range(rows) if samplers[r] is None or samplers[r].params.greedy]
        self.device_rows = [r for r in range(rows) if r not in self.greedy and 1 <= samplers[r].params.top_k <= DEVICE_TOPK_MAX]
        self.host_rows = [r for r in range(rows) if r not in self.greedy and r not in self.device_rows]
        self.greedy_out = self.keys_host = self.event = None
        dev = logits.device
        if self.greedy:
            sel = logits if len(self.greedy) == rows else logits[torch.tensor(self.greedy, device=dev)]
            self.greedy_out = torch.empty(len(self.greedy), dtype=torch.int32, device=dev)
            rt.k.argmax(sel, self.greedy_out)
        if self.device_rows:
            n = len(self.device_rows)
            recents = [samplers[r].recent(histories[r]) for r in self.device_rows]
            width = max(1, max(len(x) for x in recents))
            self.ks = [min(samplers[r].params.top_k, vocab) for r in self.device_rows]
            # one copy to the device, through pinned memory (it does not wait for the step that is
            # running): the recent tokens, how many, k, and the penalties' bits
            staged = _PINNED.take("topk in", n * width + 3 * n, torch.int32)
            flat = staged.numpy()
            flat[:] = 0
            rec = flat[:n * width].reshape(n, width)
            for i, x in enumerate(recents):
                rec[i, :len(x)] = x
            flat[n * width:n * width + n] = [len(x) for x in recents]
            flat[n * width + n:n * width + 2 * n] = self.ks
            flat[n * width + 2 * n:].view(np.float32)[:] = [samplers[r].params.repeat_penalty for r in self.device_rows]
            on = staged.to(dev, non_blocking=True)
            sel = logits if n == rows else logits[torch.tensor(self.device_rows, device=dev)].contiguous()
            self.k_stride = max(self.ks)
            cands = torch.empty((n, self.k_stride), dtype=torch.int64, device=dev)      # a row's first k places are written
            rt.k.topk(sel, on[:n * width].view(n, width), on[n * width:n * width + n], on[n * width + 2 * n:].view(torch.float32),
                      on[n * width + n:n * width + 2 * n], cands, k_max=self.k_stride)
            self.keys_host = _PINNED.take("topk out", n * self.k_stride, torch.int64)
            self.keys_host.copy_(cands.view(-1), non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record()

    def finish(self) -> List[int]:
        picks = self.picks
        if self.greedy:
            for r, v in zip(self.greedy, self.greedy_out.tolist()):
                picks[r] = v
        if self.device_rows:
            n = len(self.device_rows)
            self.event.synchronize()
            # every row's pick in one call of the native sampler, each from its own stream
            ss = [self.samplers[r] for r in self.device_rows]
            params = np.array([[s.params.temperature, s.params.top_p, s.params.min_p] for s in ss], dtype=np.float32).T.copy()
            ks = np.array(self.ks, dtype=np.int32)
            states = (ctypes.c_void_p * n)(*[ctypes.addressof(s.rng.state) for s in ss])
            out = np.empty(n, dtype=np.int32)
            host_lib().axh_sample_pick_keys_rows(
                ctypes.c_void_p(self.keys_host.data_ptr()), self.k_stride, n, ctypes.c_void_p(ks.ctypes.data),
                ctypes.c_void_p(params[0].ctypes.data), ctypes.c_void_p(params[1].ctypes.data),
                ctypes.c_void_p(params[2].ctypes.data), states, ctypes.c_void_p(out.ctypes.data))
            for r, v in zip(self.device_rows, out.tolist()):
                picks[r] = v
        for r in self.host_rows:
            picks[r] = self.samplers[r].pick_row(self.logits[r].cpu().contiguous(), self.histories[r])
        return picks


def pick_rows(rt, logits: torch.Tensor, samplers: Sequence[Optional[Sampler]],
              histories: Sequence[Sequence[int]]) -> List[int]:
    """The next token of every row of `logits` (device, float32 [rows, vocab]).  `samplers[r]`
    is None for a greedy row; `histories[r]` is the row's tokens so far, the one the logits
    follow included.  Sampled rows' logits are penalised in place."""
    return PendingRowPicks(rt, logits, samplers, histories).finish()
