"""The step function: one batch of (request, its next tokens) through the model, from the cache.

`Engine.step(entries, end)` takes, for each request in the step, the tokens that follow what
the cache already holds for it (a portion of a prompt, or one decoded token; cut anywhere)
and the places among them whose logits are wanted.  All entries run as ONE batch: the tokens
are laid side by side, every part sees them once, and attention reads each request's earlier
positions from its pages.  It returns float32 logits [wanted, vocab] in the order of the
entries and of their `want` lists.  Requests named in `end` give back what they hold after
the step.

Everything is validated before any work starts, and pages are reserved for all entries or
for none (the reference refuses a bad step before it runs anything: src/cuda/qwen2/slots.rs:393-438).
The reference runs prompt portions and decode rows as two passes of one scheduler step
(src/serve/engine.rs:2413-2417); here they are one pass.
"""
from __future__ import annotations

import ctypes
from collections import ChainMap
from dataclasses import dataclass
from typing import Dict, Hashable, Iterable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, host_lib
from ..config.engine import EngineConfig
from ..models.decoder import DecoderModel
from .runtime import Runtime, Workspace


class StepError(ValueError):
    """A step that was refused before anything ran."""


@dataclass
class StepEntry:
    id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class Span:
    """One entry as the parts see it: its slot, where its tokens lie in the batch, and the
    position of its first token."""
    slot: int
    q_start: int
    q_len: int
    start_pos: int


@dataclass
class LiveRequest:
    slot: int
    n_cached: int = 0


class StepContext:
    """What the parts are given for one step."""

    def __init__(self, rt: Runtime, cache: CacheManager, ws: Workspace, meta: torch.Tensor, n_tokens: int,
                 spans: List[Span]):
        self.rt = rt
        self.cache = cache
        self.ws = ws
        self.n_tokens = n_tokens
        self.tokens = meta[0, :n_tokens]
        self.positions = meta[1, :n_tokens]
        self.seq_rows = meta[2, :n_tokens]
        self.spans = spans
        self.shared: Dict = {}       # per-step values shared by parts with equal parameters
        # a step of single tokens that may be replayed from a graph: the index list 0..T-1 on the
        # device, and what the mixers said about the step's shape (see Mixer.decode_shape)
        self.decode_only = False
        self.decode_index: Optional[torch.Tensor] = None
        self.decode_shapes: Dict = {}
        self.decode_inputs: Dict = {}       # what the mixers asked to have on the device (Mixer.decode_input)
        self.decode_scratch: Dict = {}      # workspaces that stay in place (Mixer.decode_scratch)

    def no_rotation(self) -> torch.Tensor:
        return torch.empty((self.n_tokens, 0, 2), dtype=torch.float32, device=self.rt.device)


class PendingPicks:
    """The greedy picks of a decoding step on their way to the host: the copy was queued behind
    the step, `tolist` waits for it alone (later steps may already be running).  The staging
    buffer is one of a ring of four: read it before three further decoding steps are queued."""

    def __init__(self, buffer: torch.Tensor, event, n: int):
        self._buffer, self._event, self._n = buffer, event, n
        self._values: Optional[List[int]] = None

    def tolist(self) -> List[int]:
        if self._values is None:
            self._event.synchronize()
            self._values = self._buffer[:self._n].tolist()
        return self._values


class Engine:
    def __init__(self, model: DecoderModel, rt: Runtime, cfg: EngineConfig):
        self.model = model
        self.rt = rt
        self.cfg = cfg
        self.max_seq_len = cfg.max_seq_len or model.max_positions
        for b in model.blocks:
            limit = b.mixer.max_context()
            if limit is not None and self.max_seq_len > limit:
                raise StepError(f"max_seq_len {self.max_seq_len}: a mixer of this model takes contexts of up to {limit}")
        self.ws = Workspace(rt.device)
        plans = model.group_plans(cfg.page_size, self._pool_size)
        self.cache = CacheManager(plans, model.cache_plan.state_elems, cfg.max_seqs, self.max_seq_len, rt.device,
                                  rt.dtype, cfg.shuffle_pages_seed)
        self.live: Dict[Hashable, LiveRequest] = {}
        self.has_window = any(p.spec.window > 0 for p in plans)
        self.steps = 0
        # Decoding steps replayed from HIP graphs: static inputs and outputs, graphs per shape.  The
        # step is cut into segments: the runs whose parts are graph_safe are captured, together
        # with as much of the embedding, the final norm, the head and the pick as is; a part that
        # is not (it branches on host values or keeps state) runs launch by launch between two
        # graphs, once a step.
        n_runs = len(model.order)
        safe = [model.run_is_graph_safe(i) for i in range(n_runs)]
        self._ends_safe = model.ends_are_graph_safe()
        self._segments = []                 # (captured?, first run, end run)
        for i, ok in enumerate(safe):
            if self._segments and self._segments[-1][0] == ok:
                self._segments[-1] = (ok, self._segments[-1][1], i + 1)
            else:
                self._segments.append((ok, i, i + 1))
        self.graphs_ok = cfg.use_graphs and self._ends_safe and any(safe)
        self._graphs: Dict = {}
        self._graph_pool = None
        self._shape_mixers = []         # one mixer for each distinct thing a decoding step's shape depends on
        seen = set()
        for b in model.blocks:
            pair = b.mixer.decode_shape([0])
            if pair is not None and pair[0] not in seen:
                seen.add(pair[0])
                self._shape_mixers.append(b.mixer)
        # what mixers want on the device in a decoding step (Mixer.decode_input): a buffer that stays
        # where it is, and its staging ring
        self._input_mixers, self._inputs, self._input_hosts = [], {}, {}
        seen = set()
        for b in model.blocks:
            asked = b.mixer.decode_input([0])
            if asked is not None and asked[0] not in seen:
                seen.add(asked[0])
                cap = max(1, b.mixer.decode_input_capacity(cfg.max_seqs, self.max_seq_len))
                self._input_mixers.append(b.mixer)
                self._inputs[asked[0]] = torch.full((cap,), -1, dtype=torch.int32, device=rt.device)
                self._input_hosts[asked[0]] = [torch.full((cap,), -1, dtype=torch.int32).pin_memory() for _ in range(4)]
        # workspaces mixers want in decoding steps (Mixer.decode_scratch): one per name, sized for the
        # most requests and the longest context, allocated at the first decoding step
        self._scratch_sizes: Dict = {}
        for b in model.blocks:
            asked = b.mixer.decode_scratch(cfg.max_seqs, self.max_seq_len)
            if asked is not None:
                self._scratch_sizes[asked[0]] = max(self._scratch_sizes.get(asked[0], 0), int(asked[1]))
        self._scratch: Optional[Dict] = None
        self._meta = torch.zeros((3, cfg.max_seqs), dtype=torch.int32, device=rt.device)
        # staging in pinned memory, a ring: a step's inputs and picks travel while the host
        # prepares the next step
        self._meta_hosts = [torch.zeros((3, cfg.max_seqs), dtype=torch.int32).pin_memory() for _ in range(4)]
        self._pick_hosts = [torch.zeros(cfg.max_seqs, dtype=torch.int32).pin_memory() for _ in range(4)]
        self._ring_events = [None] * 4
        self._ring_at = 0
        self._last_decode: Optional[List[Hashable]] = None      # the requests of the last decoding step, in order
        self._pending: Optional[PendingPicks] = None
        self._prepared = None             # a decoding step that is ready but for its tokens (prepare_continue)
        self._index = torch.arange(cfg.max_seqs, dtype=torch.int32, device=rt.device)
        self._logits = None
        self._picks = torch.zeros(cfg.max_seqs, dtype=torch.int32, device=rt.device)
        self.last_picks: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ sizing
    def _pool_size(self, spec, n_layers: int, page_size: int) -> int:
        cfg = self.cfg
        if cfg.num_pages > 0:
            return cfg.num_pages
        if cfg.max_cache_tokens > 0:
            return max(1, -(-cfg.max_cache_tokens // page_size))
        # from the memory that is free now: every group gets an equal share of the fraction
        free, _ = torch.cuda.mem_get_info(self.rt.device)
        n_groups = max(1, len(self.model.cache_plan.group_specs))
        elem = self.rt.elem_size if spec.dtype is None else torch.empty((), dtype=getattr(torch, spec.dtype)).element_size()
        per_page = n_layers * spec.entries * spec.heads * page_size * spec.head_dim * elem
        pages = int(free * cfg.memory_fraction / n_groups) // max(per_page, 1)
        cap = cfg.max_seqs * -(-self.max_seq_len // page_size)
        return max(1, min(pages, cap))

    # ------------------------------------------------------------------ requests
    def n_cached(self, rid: Hashable) -> int:
        return self.live[rid].n_cached if rid in self.live else 0

    def release(self, rid: Hashable) -> None:
        """Give back the pages, the slot and the state of a request."""
        req = self.live.pop(rid, None)
        if req is not None:
            self.cache.close(req.slot)
            if self._last_decode is not None and rid in self._last_decode:
                self._last_decode = None

    def release_all(self) -> None:
        for rid in list(self.live):
            self.release(rid)

    # ------------------------------------------------------------------ the step
    def _layout(self, entries: Sequence[StepEntry]):
        """The entries of a step checked and their tokens laid side by side, by the native host
        library in one call (csrc/host/step.cpp): (meta int32 [3, T]: token ids, positions and
        slots of the step's tokens; the rows whose logits are wanted).  Every request of the step
        has its slot by now.  A refused step raises StepError and has written nothing."""
        n = len(entries)
        try:
            flat = [np.asarray(e.tokens, dtype=np.int64).reshape(-1) for e in entries]
            wants = [np.asarray(e.want, dtype=np.int64).reshape(-1) for e in entries]
        except (TypeError, ValueError, OverflowError) as err:
            raise StepError(f"a step's tokens and wanted places are whole numbers: {err}") from None
        counts = np.array([len(t) for t in flat], dtype=np.int64)
        want_counts = np.array([len(w) for w in wants], dtype=np.int64)
        tokens = np.concatenate(flat) if n else np.zeros(0, dtype=np.int64)
        want = np.concatenate(wants) if n else np.zeros(0, dtype=np.int64)
        slots = np.array([self.live[e.id].slot for e in entries], dtype=np.int32)
        cached = np.array([self.live[e.id].n_cached for e in entries], dtype=np.int64)
        T = int(counts.sum())
        meta = np.empty((3, max(T, 1)), dtype=np.int32)
        want_rows = np.empty(max(len(want), 1), dtype=np.int32)
        refused, message = ctypes.c_int(-1), ctypes.create_string_buffer(200)
        ptr = lambda a: ctypes.c_void_p(a.ctypes.data)
        rc = host_lib().axh_step_layout(n, ptr(slots), ptr(cached), ptr(counts), ptr(tokens), ptr(want), ptr(want_counts),
                                        self.model.vocab_size, self.max_seq_len, ptr(meta), meta.shape[1], ptr(want_rows),
                                        ctypes.byref(refused), message, len(message))
        if rc < 0:
            who = f"request {entries[refused.value].id!r}: " if refused.value >= 0 else ""
            raise StepError(who + message.value.decode())
        return meta[:, :T], want_rows[:len(want)], counts

    def step(self, entries: Sequence[StepEntry], end: Iterable[Hashable] = ()) -> Optional[torch.Tensor]:
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        seen = set()
        for e in entries:
            if e.id in seen:
                raise StepError(f"request {e.id!r} appears twice in one step")
            seen.add(e.id)
        new = sum(1 for e in entries if e.id not in self.live)
        if new > self.cache.free_slots():
            raise StepError(f"{len(self.live) + new} live requests, at most {self.cfg.max_seqs}")
        # Everything is checked, and pages are taken for every entry or for none, before anything
        # runs: a step that is refused or does not fit leaves the cache as it was.
        opened = []
        try:
            for e in entries:
                if e.id not in self.live:
                    self.live[e.id] = LiveRequest(self.cache.open())
                    opened.append(e.id)
            meta, want_rows, counts = self._layout(entries)
            self.cache.reserve_many([(self.live[e.id].slot, self.live[e.id].n_cached + int(n)) for e, n in zip(entries, counts)])
        except Exception:
            for rid in opened:
                self.release(rid)
            raise

        logits = None
        self.last_picks = None
        self._last_decode = None
        self._pending = None
        self._prepared = None
        if entries:
            spans, at = [], 0
            for e, n in zip(entries, counts):
                req = self.live[e.id]
                spans.append(Span(req.slot, at, int(n), req.n_cached))
                at += int(n)
            T = at
            self.cache.sync_tables()
            if T == len(entries) and len(want_rows) == T and T <= self.cfg.max_seqs:
                logits = self._decode_step(meta[0].tolist(), meta[1].tolist(), meta[2].tolist(), spans)
                self._last_decode = [e.id for e in entries]
            else:
                on_device = torch.from_numpy(np.ascontiguousarray(meta)).to(self.rt.device)
                ctx = StepContext(self.rt, self.cache, self.ws, on_device, T, spans)
                x = self.model.forward(ctx)
                if len(want_rows):
                    sel = torch.from_numpy(want_rows.copy()).to(self.rt.device)
                    logits = self.model.logits(ctx, x, sel)
            for e, n in zip(entries, counts):
                req = self.live[e.id]
                req.n_cached += int(n)
                if self.has_window:
                    self.cache.trim(req.slot, req.n_cached)
            self.steps += 1
        for rid in end:
            self.release(rid)
        return logits

    def profile(self, entries: Sequence[StepEntry], end: Iterable[Hashable] = ()):
        """One step launched kernel by kernel (no graph) with an event after every launch:
        ([{name, ms, launches, bytes}] in first-launch order, total ms), as the reference's
        profile of a step (src/cuda/qwen2.rs:3338-3397).  `bytes`: the weight matrices those
        launches read.  The events between the kernels also keep them from overlapping, so this
        is each kernel alone; the step itself is a real one (the cache moves on)."""
        events = []

        def mark(name, nbytes):
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            events.append((name, ev, nbytes))

        graphs, self.graphs_ok = self.graphs_ok, False
        self.rt.k.set_launch_hook(mark)
        try:
            mark("start", 0)
            self.step(entries, end)
        finally:
            self.rt.k.set_launch_hook(None)
            self.graphs_ok = graphs
        torch.cuda.synchronize()
        rows: Dict[str, dict] = {}
        for (_, before, _), (name, after, nbytes) in zip(events, events[1:]):
            row = rows.setdefault(name, dict(name=name, ms=0.0, launches=0, bytes=0))
            row["ms"] += before.elapsed_time(after)
            row["launches"] += 1
            row["bytes"] += nbytes
        return list(rows.values()), events[0][1].elapsed_time(events[-1][1])

    def step_from_picks(self, ids: Sequence[Hashable]) -> torch.Tensor:
        """One more decoding step for exactly the requests of the last decoding step, in its
        order: each takes as its token the greedy pick that step made for it.  The pick is taken
        on the device, so the host need not have read it yet: it can queue this step and read
        the previous step's picks (`picks_async`) while this one runs.  Returns the logits as
        `step` does."""
        self.prepare_continue(ids)
        return self.run_prepared(None)

    def prepare_continue(self, ids: Sequence[Hashable]) -> None:
        """Everything of one more decoding step of the last decoding step's requests (the same
        ones, in the same order) that does not depend on their next tokens: pages, block tables,
        positions, what the mixers want on the device.  The host can do this while the device
        still runs the step before and the tokens are not decided yet; `run_prepared(tokens)`
        then starts the step.  Raises (and leaves everything as it was) if it cannot be done:
        OutOfPages, a request at its longest."""
        ids = list(ids)
        if self._last_decode is None or ids != self._last_decode:
            raise StepError("a decoding step is continued by the same requests in the same order")
        reqs = [self.live[rid] for rid in ids]
        for rid, req in zip(ids, reqs):
            if req.n_cached + 1 > self.max_seq_len:
                raise StepError(f"request {rid!r} would reach {req.n_cached + 1} positions, at most {self.max_seq_len}")
        self.cache.reserve_many([(req.slot, req.n_cached + 1) for req in reqs])      # OutOfPages: nothing taken, nothing run
        positions = [req.n_cached for req in reqs]
        rows = [req.slot for req in reqs]
        spans = [Span(req.slot, i, 1, req.n_cached) for i, req in enumerate(reqs)]
        self.cache.sync_tables()
        self._prepared = (ids, reqs, self._decode_prepare(positions, rows, spans))

    def run_prepared(self, tokens: Optional[Sequence[int]]) -> torch.Tensor:
        """Start the step that `prepare_continue` prepared, with these tokens (one a request, in
        order), or with the greedy picks of the step before, taken on the device, if None."""
        if self._prepared is None:
            raise StepError("run_prepared follows prepare_continue")
        ids, reqs, prepared = self._prepared
        self._prepared = None
        if tokens is not None:
            tokens = [int(t) for t in tokens]
            if len(tokens) != len(ids) or any(not 0 <= t < self.model.vocab_size for t in tokens):
                raise StepError(f"run_prepared: {len(ids)} requests need a token of the vocabulary each")
        logits = self._decode_launch(prepared, tokens)
        for req in reqs:
            req.n_cached += 1
            if self.has_window:
                self.cache.trim(req.slot, req.n_cached)
        self.steps += 1
        return logits

    def drop_prepared(self) -> None:
        """Forget a prepared step that will not run (the pages it reserved stay with their
        requests, which use them at their next token or give them back at their end)."""
        self._prepared = None

    def picks_async(self) -> Optional[PendingPicks]:
        """The last decoding step's greedy picks as a copy that is under way (None after any
        other step)."""
        return self._pending

    # ------------------------------------------------------------------ decoding steps
    def _decode_context(self, T: int, spans: List[Span], shapes: Dict, inputs: Dict) -> StepContext:
        ctx = StepContext(self.rt, self.cache, self.ws, self._meta, T, spans)
        ctx.decode_only = True
        ctx.decode_index = self._index[:T]
        ctx.decode_shapes = shapes
        ctx.decode_inputs = inputs
        ctx.decode_scratch = self._scratch
        return ctx

    def _decode_forward(self, T: int, spans: List[Span], shapes: Dict, inputs: Dict):
        """A step of T single tokens whose tokens, positions and slots are in `self._meta`,
        launch by launch.  Logits go to the static buffer, greedy picks beside them."""
        ctx = self._decode_context(T, spans, shapes, inputs)
        x = self.model.forward(ctx)
        logits = self.model.logits(ctx, x, ctx.decode_index, out=self._logits[:T])
        self.rt.k.argmax(logits, self._picks[:T])
        return logits

    def _segment(self, ctx: StepContext, x: torch.Tensor, index: int) -> None:
        """Segment `index` of a decoding step on the residual stream x, in place: its runs, with
        the embedding before the first run and the final norm, the head and the pick behind the
        last (logits into the static buffer)."""
        _, first, end = self._segments[index]
        if first == 0:
            self.model.embed(ctx, out=x)
        self.model.forward_runs(ctx, x, first, end)
        if end == len(self.model.order):
            logits = self.model.logits(ctx, x, ctx.decode_index, out=self._logits[:ctx.n_tokens])
            self.rt.k.argmax(logits, self._picks[:ctx.n_tokens])

    def _decode_graphs(self, key, T: int, spans: List[Span], shapes: Dict, inputs: Dict) -> torch.Tensor:
        """Replay (at the first step of a shape: set up and capture) the step's segments.  What
        the parts share within a step (`ctx.shared`: tables, plans) is kept from the captured
        segments, whose graphs refresh it at every replay; what a segment that runs launch by
        launch adds is the step's own and is dropped after it."""
        entry = self._graphs.get(key)
        if entry is None:
            entry = self._graphs[key] = dict(
                x=torch.empty((T, self.model.hidden_size), dtype=torch.float32, device=self.rt.device), shared={},
                graphs=[None] * len(self._segments))
        x = entry["x"]

        def context(shared):
            ctx = self._decode_context(T, spans, shapes, inputs)
            ctx.shared = shared
            return ctx

        of_step = ChainMap({}, entry["shared"])
        for index, (captured, _, _) in enumerate(self._segments):
            if not captured:
                self._segment(context(of_step), x, index)
                continue
            if entry["graphs"][index] is None:
                # Once without capture, on a copy of the stream: kernels set themselves up at their
                # first launch, and a captured segment writes the same cache rows however often it
                # runs.  Then the capture itself, which runs nothing; the replay below is the step.
                self._segment(context(ChainMap({}, entry["shared"])), x.clone(), index)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                if self._graph_pool is None:
                    self._graph_pool = torch.cuda.graph_pool_handle()
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    self._segment(context(entry["shared"]), x, index)
                entry["graphs"][index] = graph
            entry["graphs"][index].replay()
        return self._logits[:T]

    def _decode_step(self, tokens, positions, rows, spans) -> torch.Tensor:
        """Every entry brings one token and wants its logits.  Inputs are copied into static
        device buffers; with graphs on, the launches of this (number of tokens, shape) are
        captured once and replayed afterwards.  Returns a view of a static logits buffer, valid
        until the next decoding step; `last_picks` holds the greedy pick of each row."""
        return self._decode_launch(self._decode_prepare(positions, rows, spans), tokens)

    def _decode_prepare(self, positions, rows, spans):
        """What a step of single tokens needs beside the tokens: positions and slots on their way
        to the device, the step's shape, the values the mixers asked for."""
        T = len(positions)
        if self._scratch is None:
            self._scratch = {name: torch.empty(n, dtype=torch.float32, device=self.rt.device)
                             for name, n in self._scratch_sizes.items()}
        if self._logits is None:
            self._logits = torch.empty((self.cfg.max_seqs, self.model.vocab_size), dtype=torch.float32,
                                       device=self.rt.device)
        # inputs through a ring of pinned buffers, without waiting: a buffer is written again only
        # after the copies that read or wrote it have run
        at = self._ring_at = (self._ring_at + 1) % len(self._meta_hosts)
        if self._ring_events[at] is not None:
            self._ring_events[at].synchronize()
        host = self._meta_hosts[at]
        host[1:, :T] = torch.tensor([positions, rows], dtype=torch.int32)
        self._meta[1:].copy_(host[1:], non_blocking=True)
        shapes = {}
        for mixer in self._shape_mixers:
            name, value = mixer.decode_shape(positions)
            shapes[name] = value
        inputs = {}
        for mixer in self._input_mixers:
            name, values = mixer.decode_input(positions)
            n = len(values)
            if n > self._inputs[name].numel():
                raise StepError(f"{name}: {n} values for the device, room for {self._inputs[name].numel()}")
            staged = self._input_hosts[name][at]
            staged[:n] = torch.as_tensor(values, dtype=torch.int32)
            self._inputs[name][:n].copy_(staged[:n], non_blocking=True)
            inputs[name] = self._inputs[name][:n]
            shapes[("values of", name)] = n          # a graph reads exactly this many
        return T, at, spans, shapes, inputs

    def _decode_launch(self, prepared, tokens) -> torch.Tensor:
        T, at, spans, shapes, inputs = prepared
        host = self._meta_hosts[at]
        if tokens is None:
            # the tokens are the previous step's picks, already on the device
            self._meta[0, :T].copy_(self._picks[:T])
        else:
            host[0, :T] = torch.tensor(tokens, dtype=torch.int32)
            self._meta[0].copy_(host[0], non_blocking=True)
        if not self.graphs_ok:
            logits = self._decode_forward(T, spans, shapes, inputs)
        else:
            logits = self._decode_graphs((T, tuple(sorted(shapes.items(), key=repr))), T, spans, shapes, inputs)
        self.last_picks = self._picks[:T]
        # the picks start their way to the host behind the step
        self._pick_hosts[at][:T].copy_(self._picks[:T], non_blocking=True)
        event = self._ring_events[at] or torch.cuda.Event()
        event.record()
        self._ring_events[at] = event
        self._pending = PendingPicks(self._pick_hosts[at], event, T)
        return logits
