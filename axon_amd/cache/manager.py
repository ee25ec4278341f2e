"""The cache manager: paged storage per cache group, block tables, and per-request state.

Host decisions (which page, which slot) are made by the native allocator
(`csrc/host/cache.cpp`); this class owns the device memory they index:

* per group, one tensor [layers, entries, pages, heads, page_size, head_dim] in the compute
  dtype (for attention: entries = keys and values), so a page holds `page_size` positions of
  every layer of its group, and one int32 block table [max_seqs, max_pages_per_seq];
* per run with state, one float32 arena [max_seqs, elems], zeroed when a request opens.

A request is `open()`ed into a slot, `reserve()`s pages as it grows (all groups or nothing),
is `trim()`med after each step (windowed groups give back pages the window has passed) and
`close()`d at its end.  Block table rows that changed are uploaded before a step by
`sync_tables()`.  With `device=None` nothing is allocated on a device: the bookkeeping alone,
for tests and planning.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_long, c_void_p
from dataclasses import dataclass
from typing import List, Sequence, Tuple

import torch

from ..kernels import build
from ..parts.base import CacheSpec


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A reservation that did not fit; nothing was taken.  `short` pages were missing."""

    def __init__(self, short: int, msg: str):
        super().__init__(msg)
        self.short = short


_HOST = None


def host_lib():
    """The native host runtime (cache manager and scheduler), loaded once."""
    global _HOST
    if _HOST is None:
        lib = ctypes.CDLL(build.build_host())
        IP, LP, I64P = POINTER(c_int), POINTER(c_long), POINTER(ctypes.c_int64)
        sig = {
            "axh_cache_create": (c_void_p, [c_int, IP, IP, IP, c_int, c_int, c_long]),
            "axh_cache_destroy": (None, [c_void_p]),
            "axh_cache_error": (c_char_p, [c_void_p]),
            "axh_cache_open": (c_int, [c_void_p]),
            "axh_cache_close": (c_int, [c_void_p, c_int]),
            "axh_cache_reserve": (c_int, [c_void_p, c_int, c_long]),
            "axh_cache_reserve_many": (c_int, [c_void_p, c_int, IP, LP]),
            "axh_cache_trim": (c_int, [c_void_p, c_int, c_long]),
            "axh_cache_row": (c_int, [c_void_p, c_int, c_int, c_void_p, c_int]),
            "axh_cache_free_pages": (c_int, [c_void_p, c_int]),
            "axh_cache_free_slots": (c_int, [c_void_p]),
            "axh_cache_pages_of": (c_int, [c_void_p, c_int, c_int]),
            "axh_cache_length": (c_long, [c_void_p, c_int]),
            "axh_cache_check": (c_int, [c_void_p]),
            "axh_sched_create": (c_void_p, [c_int, IP, IP, IP, c_int, c_int, c_long]),
            "axh_sched_destroy": (None, [c_void_p]),
            "axh_sched_error": (c_char_p, [c_void_p]),
            "axh_sched_add": (c_int, [c_void_p, ctypes.c_int64, c_long, c_long]),
            "axh_sched_plan": (c_int, [c_void_p, LP, I64P, LP, LP, IP, c_int, I64P, IP]),
            "axh_sched_commit": (c_int, [c_void_p, ctypes.c_int64, c_long, c_int, c_int]),
            "axh_sched_remove": (c_int, [c_void_p, ctypes.c_int64]),
            "axh_sched_counts": (None, [c_void_p, LP, LP, LP]),
            "axh_sched_progress": (c_int, [c_void_p, ctypes.c_int64, LP, LP, IP]),
            "axh_rng_seed": (None, [ctypes.c_uint64, c_void_p]),
            "axh_rng_next_u64": (ctypes.c_uint64, [c_void_p]),
            "axh_rng_next_f64": (ctypes.c_double, [c_void_p]),
            "axh_sample_pick_keys": (c_int, [c_void_p, c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                             ctypes.c_double]),
            "axh_sample_pick_keys_rows": (None, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                 c_void_p]),
            "axh_sample_pick_row": (c_int, [c_void_p, c_int, c_void_p, c_int, ctypes.c_float, c_int, ctypes.c_float,
                                            ctypes.c_float, ctypes.c_float, ctypes.c_double]),
            "axh_argmax_row": (c_int, [c_void_p, c_int]),
            "axh_step_layout": (c_long, [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_long,
                                         c_void_p, c_long, c_void_p, IP, c_char_p, c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _HOST = lib
    return _HOST


@dataclass
class GroupPlan:
    """A cache group before memory is given to it: the need of its layers, how many layers
    (runs that store) it has, and its geometry."""
    spec: CacheSpec
    n_layers: int
    page_size: int
    n_pages: int

    def bytes_per_page(self, elem_size: int) -> int:
        """`elem_size`: of the compute dtype, which a group that names no dtype of its own stores."""
        if self.spec.dtype is not None:
            elem_size = torch.empty((), dtype=getattr(torch, self.spec.dtype)).element_size()
        return self.n_layers * self.spec.entries * self.spec.heads * self.page_size * self.spec.head_dim * elem_size


class CacheGroup:
    """One group's device memory and block table."""

    def __init__(self, plan: GroupPlan, max_seqs: int, max_pages_per_seq: int, device, dtype):
        self.plan = plan
        self.page_size = plan.page_size
        self.n_pages = plan.n_pages
        self.window = plan.spec.window
        self.storage = None
        self.block_table = None
        self.host_table = torch.zeros((max_seqs, max_pages_per_seq), dtype=torch.int32)
        if device is not None:
            s = plan.spec
            self.storage = torch.zeros((plan.n_layers, s.entries, plan.n_pages, s.heads, plan.page_size, s.head_dim),
                                       dtype=dtype if s.dtype is None else getattr(torch, s.dtype), device=device)
            self.block_table = torch.zeros((max_seqs, max_pages_per_seq), dtype=torch.int32, device=device)
            # staging of changed rows on their way to the device (CacheManager.sync_tables): max_seqs rows
            # and, in a last row, the slots they belong to
            shape = (max_seqs + 1, max(max_pages_per_seq, max_seqs))
            self.stages = [torch.zeros(shape, dtype=torch.int32).pin_memory() for _ in range(4)]
            self.stage_events = [None] * 4
            self.stage_at = 0
            self.stage_device = torch.zeros(shape, dtype=torch.int32, device=device)

    def layer(self, index: int) -> Tuple[torch.Tensor, ...]:
        """The arrays of one layer of the group: for attention (keys, values), each
        [pages, heads, page_size, head_dim]."""
        return tuple(self.storage[index, e] for e in range(self.plan.spec.entries))


class CacheManager:
    def __init__(self, groups: Sequence[GroupPlan], state_elems: Sequence[int], max_seqs: int, max_seq_len: int,
                 device=None, dtype=torch.float32, shuffle_seed: int = -1):
        self.lib = host_lib()
        self.max_seqs = max_seqs
        self.max_seq_len = max_seq_len
        self.device = device
        min_page = min([g.page_size for g in groups], default=16)
        self.max_pages_per_seq = max(1, -(-max_seq_len // min_page))
        n = len(groups)
        arr = lambda vals: (c_int * max(n, 1))(*vals)
        self._h = self.lib.axh_cache_create(n, arr([g.n_pages for g in groups]), arr([g.page_size for g in groups]),
                                            arr([g.spec.window for g in groups]), max_seqs, self.max_pages_per_seq,
                                            shuffle_seed)
        if not self._h:
            raise CacheError(f"bad cache geometry: {[(g.n_pages, g.page_size, g.spec.window) for g in groups]}")
        self.plans = list(groups)
        self.groups = [CacheGroup(g, max_seqs, self.max_pages_per_seq, device, dtype) for g in groups]
        # a state arena per run with state: `state_elems` holds sizes, or (size, dtype name) pairs
        sized = [(e, "float32") if isinstance(e, int) else (int(e[0]), str(e[1])) for e in state_elems]
        self.states = [torch.zeros((max_seqs, max(e, 1)), dtype=getattr(torch, dt), device=device) if device is not None
                       else None for e, dt in sized]
        self._dirty: set = set()

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                self.lib.axh_cache_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def _error(self) -> str:
        return self.lib.axh_cache_error(self._h).decode()

    # ------------------------------------------------------------------ requests
    def group(self, index: int) -> CacheGroup:
        return self.groups[index]

    def state(self, index: int) -> torch.Tensor:
        return self.states[index]

    def open(self) -> int:
        slot = self.lib.axh_cache_open(self._h)
        if slot < 0:
            raise CacheError(self._error())
        for s in self.states:
            if s is not None:
                s[slot].zero_()
        return slot

    def close(self, slot: int) -> int:
        freed = self.lib.axh_cache_close(self._h, slot)
        if freed < 0:
            raise CacheError(self._error())
        self._dirty.discard(slot)
        return freed

    def reserve(self, slot: int, n_tokens: int) -> None:
        """Pages for positions [0, n_tokens) in every group, or OutOfPages and nothing taken."""
        if n_tokens > self.max_seq_len:
            raise CacheError(f"{n_tokens} positions exceed the {self.max_seq_len} a request may reach")
        held = [self.lib.axh_cache_pages_of(self._h, g, slot) for g in range(len(self.groups))]
        rc = self.lib.axh_cache_reserve(self._h, slot, n_tokens)
        if rc == 0:
            # only a row that took a page has to be uploaded again
            if any(self.lib.axh_cache_pages_of(self._h, g, slot) != held[g] for g in range(len(self.groups))):
                self._dirty.add(slot)
        elif rc <= -1000000:
            raise CacheError(self._error())
        else:
            raise OutOfPages(-rc, f"the cache is full: {-rc} pages short for {n_tokens} positions of slot {slot}")

    def reserve_many(self, needs: Sequence[Tuple[int, int]]) -> None:
        """Pages for every (slot, positions) of a step, in every group: for all of them or, with
        OutOfPages, for none (what a step reserves is what all of its entries need)."""
        if not needs:
            return
        for slot, n_tokens in needs:
            if n_tokens > self.max_seq_len:
                raise CacheError(f"{n_tokens} positions exceed the {self.max_seq_len} a request may reach")
        n_groups = len(self.groups)
        held = [[self.lib.axh_cache_pages_of(self._h, g, slot) for g in range(n_groups)] for slot, _ in needs]
        slots = (c_int * len(needs))(*[s for s, _ in needs])
        tokens = (c_long * len(needs))(*[n for _, n in needs])
        rc = self.lib.axh_cache_reserve_many(self._h, len(needs), slots, tokens)
        if rc == 0:
            for (slot, _), before in zip(needs, held):
                if any(self.lib.axh_cache_pages_of(self._h, g, slot) != before[g] for g in range(n_groups)):
                    self._dirty.add(slot)
        elif rc <= -1000000:
            raise CacheError(self._error())
        else:
            raise OutOfPages(-rc, f"the cache is full: {-rc} pages short for the {len(needs)} requests of the step")

    def trim(self, slot: int, n_cached: int) -> int:
        freed = self.lib.axh_cache_trim(self._h, slot, n_cached)
        if freed < 0:
            raise CacheError(f"trim: slot {slot} is not open")
        return freed

    # ------------------------------------------------------------------ tables
    def row(self, group: int, slot: int) -> List[int]:
        buf = (c_int * self.max_pages_per_seq)()
        n = self.lib.axh_cache_row(self._h, group, slot, buf, self.max_pages_per_seq)
        if n < 0:
            raise CacheError(f"no block table row for group {group}, slot {slot}")
        return list(buf[:n])

    def sync_tables(self) -> None:
        """Upload the rows that changed since the last call, in stream order before the kernels
        that read them: one staged copy and one scatter per group."""
        if not self._dirty:
            return
        slots = sorted(self._dirty)
        n = len(slots)
        for gi, g in enumerate(self.groups):
            if g.block_table is None:
                rows = torch.zeros((n, self.max_pages_per_seq), dtype=torch.int32)
            else:
                # Through pinned memory, without waiting for the device: the rows as they are now go into
                # one of a ring of staging buffers (with the slots they belong to in the buffer's last
                # row), one copy brings them over and a scatter puts them in place, in stream order.
                # A staging buffer is written again only after the copy that read it has run.
                at = g.stage_at = (g.stage_at + 1) % len(g.stages)
                if g.stage_events[at] is not None:
                    g.stage_events[at].synchronize()
                stage = g.stages[at]
                rows = stage[:n, :self.max_pages_per_seq]
                rows.zero_()
                stage[self.max_seqs, :n] = torch.tensor(slots, dtype=torch.int32)
            for i, slot in enumerate(slots):
                got = self.lib.axh_cache_row(self._h, gi, slot, c_void_p(rows[i].data_ptr()), self.max_pages_per_seq)
                if got < 0:
                    raise CacheError(f"no block table row for group {gi}, slot {slot}")
            g.host_table[slots] = rows
            if g.block_table is not None:
                g.stage_device[:n].copy_(stage[:n], non_blocking=True)
                g.stage_device[self.max_seqs].copy_(stage[self.max_seqs], non_blocking=True)
                event = g.stage_events[at] or torch.cuda.Event()
                event.record()
                g.stage_events[at] = event
                g.block_table.index_copy_(0, g.stage_device[self.max_seqs, :n].long(),
                                          g.stage_device[:n, :self.max_pages_per_seq])
        self._dirty.clear()

    # ------------------------------------------------------------------ accounting
    def free_pages(self, group: int = 0) -> int:
        return self.lib.axh_cache_free_pages(self._h, group)

    def free_slots(self) -> int:
        return self.lib.axh_cache_free_slots(self._h)

    def pages_of(self, group: int, slot: int) -> int:
        return self.lib.axh_cache_pages_of(self._h, group, slot)

    def length(self, slot: int) -> int:
        return self.lib.axh_cache_length(self._h, slot)

    def check(self) -> None:
        """Raise if a page or slot is lost, held twice or free and held at once."""
        if self.lib.axh_cache_check(self._h) != 0:
            raise CacheError("cache invariant broken: " + self._error())
