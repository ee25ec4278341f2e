"""The scheduler above the step function: admission, portions under a token budget, decoding,
finishing, and what happens when pages run out.

The decisions are made natively (`csrc/host/scheduler.cpp`); this class feeds it the free
pages, turns its plan into step entries and reports back what ran.  The policy in short:
first come first served; decoding requests first, then prompt portions, oldest first, under
`max_batch_tokens`; a request that cannot get a page takes the pages of the youngest request
younger than itself, which is later fed again from its first token and continues with the
same tokens; a request that could not fit the pool alone is refused when it is added.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_long
from dataclasses import dataclass
from typing import List, Sequence, Tuple

from ..cache.manager import host_lib


class SchedulerError(RuntimeError):
    pass


@dataclass
class Planned:
    id: int
    start: int
    count: int
    wants_logits: bool


class Scheduler:
    def __init__(self, n_pages: Sequence[int], page_size: Sequence[int], window: Sequence[int],
                 max_batch_tokens: int, max_seqs: int, max_seq_len: int):
        self.lib = host_lib()
        n = len(n_pages)
        self.n_groups = n
        arr = lambda v: (c_int * max(n, 1))(*v)
        self._h = self.lib.axh_sched_create(n, arr(n_pages), arr(page_size), arr(window), max_batch_tokens, max_seqs,
                                            max_seq_len)
        if not self._h:
            raise SchedulerError("bad scheduler settings")
        self.cap = max(max_seqs, 1) * 2 + 8
        self._ids = (ctypes.c_int64 * self.cap)()
        self._starts = (c_long * self.cap)()
        self._counts = (c_long * self.cap)()
        self._wants = (c_int * self.cap)()
        self._pre = (ctypes.c_int64 * self.cap)()

    @classmethod
    def for_cache(cls, cache, max_batch_tokens: int) -> "Scheduler":
        plans = cache.plans
        return cls([p.n_pages for p in plans], [p.page_size for p in plans], [p.spec.window for p in plans],
                   max_batch_tokens, cache.max_seqs, cache.max_seq_len)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                self.lib.axh_sched_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def _error(self) -> str:
        return self.lib.axh_sched_error(self._h).decode()

    def add(self, rid: int, prompt_len: int, max_new: int) -> None:
        if self.lib.axh_sched_add(self._h, rid, prompt_len, max_new) != 0:
            raise SchedulerError(self._error())

    def plan(self, free_pages: Sequence[int]) -> Tuple[List[Planned], List[int]]:
        """The next step's entries, and the requests that must give up their pages first."""
        free = (c_long * max(self.n_groups, 1))(*free_pages)
        n_pre = c_int(0)
        n = self.lib.axh_sched_plan(self._h, free, self._ids, self._starts, self._counts, self._wants, self.cap,
                                    self._pre, ctypes.byref(n_pre))
        if n < 0:
            raise SchedulerError(self._error())
        entries = [Planned(self._ids[i], self._starts[i], self._counts[i], bool(self._wants[i])) for i in range(n)]
        return entries, [self._pre[i] for i in range(n_pre.value)]

    def commit(self, rid: int, n_run: int, appended: bool, finished: bool) -> None:
        if self.lib.axh_sched_commit(self._h, rid, n_run, int(appended), int(finished)) != 0:
            raise SchedulerError(self._error())

    def remove(self, rid: int) -> int:
        return self.lib.axh_sched_remove(self._h, rid)

    def counts(self) -> Tuple[int, int, int]:
        """(waiting, running, preemptions so far)."""
        w, r, p = c_long(0), c_long(0), c_long(0)
        self.lib.axh_sched_counts(self._h, ctypes.byref(w), ctypes.byref(r), ctypes.byref(p))
        return w.value, r.value, p.value

    def progress(self, rid: int):
        """(tokens in the cache, tokens the request consists of, running?) or None."""
        c, t, s = c_long(0), c_long(0), c_int(0)
        if self.lib.axh_sched_progress(self._h, rid, ctypes.byref(c), ctypes.byref(t), ctypes.byref(s)) != 0:
            return None
        return c.value, t.value, bool(s.value)
