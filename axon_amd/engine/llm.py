"""The Python entry point: `axon_amd.load(model).generate(token_ids, ...)`.

In the manner of the reference's library root (src/lib.rs:19-35, 112-127: `load`, then a
backend, then `generate` with greedy or sampled options, src/generate.rs:29-114), with token
ids in and token ids out: there is no tokenizer here.  Any number of prompts may be given;
they are batched continuously by the scheduler.
"""
from __future__ import annotations

import json
import os
import sys
import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..config import EngineConfig, ModelConfig, config_from_dict
from ..cache.manager import OutOfPages
from ..sampling import PendingRowPicks, Sampler, SamplingParams
from .loading import load_model, random_model
from .runtime import Runtime
from .scheduler import Scheduler
from .step import Engine, StepEntry, StepError


@dataclass
class GenStats:
    """What a `generate` call did (the reference's GenStats, src/generate.rs:29-45, reduced to
    what this engine has): steps run, tokens fed as prompt, tokens decided, time."""
    steps: int = 0
    prompt_tokens: int = 0
    decided: int = 0
    preemptions: int = 0
    seconds: float = 0.0
    prompt_seconds: float = 0.0     # steps that fed prompt tokens
    decode_seconds: float = 0.0     # steps that only decoded
    decode_steps: int = 0
    decode_tokens: int = 0


@dataclass
class _Request:
    tokens: List[int]
    prompt_len: int
    max_new: int
    sampler: Optional[Sampler]
    out: List[int] = field(default_factory=list)
    done: bool = False
    stopped: bool = False        # it picked a stop token (learnt a step late when decoding runs ahead)


class StepTrace:
    """AXON_STEP_TRACE=FILE: one JSON line per scheduler step appended to FILE, a measurement aid
    that changes no output (the reference's AXON_SERVE_TRACE, src/serve/engine.rs:682-773,
    2011-2034): `t_ms` since the trace opened, the step's wall `ms` (the device is waited for, so
    running ahead is off while tracing), its prompt portions (`feeds`, `fed` tokens), its
    decoding rows (`rows`, their mean `depth` in positions; null without any), then the requests
    `waiting` and `running` and the `preempted` ones of this step."""

    def __init__(self, path: str):
        self.out = open(path, "a", buffering=1)
        self.t0 = time.time()

    @classmethod
    def from_env(cls) -> Optional["StepTrace"]:
        path = os.environ.get("AXON_STEP_TRACE", "")
        if not path:
            return None
        try:
            trace = cls(path)
        except OSError as e:
            print(f"axon: AXON_STEP_TRACE {path}: {e}", file=sys.stderr)
            return None
        print(f"axon: step trace to {path}", file=sys.stderr)
        return trace

    def line(self, started: float, ms: float, plan, waiting: int, running: int, preempted: int) -> None:
        feeds = [p for p in plan if p.count > 1 or p.start == 0]
        rows = [p for p in plan if p.count == 1 and p.start > 0]
        depth = round(sum(p.start for p in rows) / len(rows), 1) if rows else None
        self.out.write(json.dumps({"t_ms": round((started - self.t0) * 1e3, 3), "ms": round(ms, 3), "feeds": len(feeds),
                                   "fed": sum(p.count for p in feeds), "rows": len(rows), "depth": depth,
                                   "waiting": waiting, "running": running, "preempted": preempted}) + "\n")


class LLM:
    def __init__(self, model, rt: Runtime, cfg: EngineConfig):
        self.model = model
        self.rt = rt
        self.cfg = cfg
        self.engine = Engine(model, rt, cfg)
        self.last_stats = GenStats()
        self._next_id = 0

    @property
    def config(self) -> ModelConfig:
        return self.model.config

    # ------------------------------------------------------------------ generation
    def generate(self, prompts: Union[Sequence[int], Sequence[Sequence[int]]], max_new_tokens: int = 32,
                 temperature: float = 0.0, top_k: int = 40, top_p: float = 0.9, min_p: float = 0.0,
                 repeat_penalty: float = 1.1, repeat_last_n: int = 64, seed: Optional[int] = None,
                 stop: Sequence[int] = (), sampling: Optional[SamplingParams] = None) -> List[List[int]]:
        """New tokens for every prompt (lists of token ids).  `temperature` 0 is greedy: the
        highest logit, and no other sampling setting applies.  With a temperature, request i
        draws from the stream seeded `seed + i`.  A token in `stop` ends its request and is not
        returned (src/generate.rs:169-171)."""
        single = len(prompts) > 0 and isinstance(prompts[0], int)
        batch = [list(prompts)] if single else [list(p) for p in prompts]
        params = sampling or SamplingParams(temperature, top_k, top_p, min_p, repeat_penalty, repeat_last_n, seed)
        sched = Scheduler.for_cache(self.engine.cache, self.cfg.max_batch_tokens)
        reqs: Dict[int, _Request] = {}
        order = []
        for i, p in enumerate(batch):
            if not p:
                raise ValueError("a prompt needs at least one token")
            rid = self._next_id
            self._next_id += 1
            sampler = None
            if not params.greedy:
                base = params.seed if params.seed is not None else None
                sampler = Sampler(SamplingParams(params.temperature, params.top_k, params.top_p, params.min_p,
                                                 params.repeat_penalty, params.repeat_last_n,
                                                 None if base is None else base + i))
            reqs[rid] = _Request(p, len(p), max_new_tokens, sampler)
            order.append(rid)
            if max_new_tokens <= 0:
                reqs[rid].done = True
            else:
                sched.add(rid, len(p), max_new_tokens)
        stats = GenStats()
        t0 = time.time()
        stop = set(int(s) for s in stop)
        cache = self.engine.cache
        n_groups = len(cache.groups)
        # Greedy decoding runs one step ahead of the host: a step takes its tokens from the picks
        # of the step before on the device (Engine.step_from_picks), and the picks are read a step
        # late, while the next step runs.  Until they are read the requests' lists hold None in
        # their place.  That a request has reached its length is known without the token; that it
        # picked a stop token is learnt a step late: the token is taken back, the request ends,
        # and the row that the step ahead ran for it is dropped unread.
        trace = StepTrace.from_env()
        ahead_ok = trace is None
        behind = None            # (picks on their way, the requests they belong to)
        # Sampled tokens are drawn on the host, so a step cannot start before the one before it has
        # ended.  What it can do is have everything but its tokens ready by then: while the device
        # runs a decoding step whose rows will all decode again, the next step is prepared
        # (Engine.prepare_continue: pages, tables, positions), and once the tokens are drawn it
        # only takes them and starts.  If the next plan is another after all (a request drew a stop
        # token, one was admitted) the prepared step is dropped.
        prepared = None          # the requests of a step that is ready but for its tokens
        # The clocks of `GenStats`.  Steps are queued ahead of the device, so a step's own time is not
        # known on the host; what is known is when the host had to wait.  Everything between two
        # marks is charged to the kind of step (decoding only, or feeding prompts) that was being
        # prepared, waits for earlier steps included, and the device is waited for where the kind
        # changes and at the end: the two clocks add up to the wall time, and tokens divided by
        # their clock can never beat a synchronised measurement of the same steps.
        clock = {"mark": time.time(), "kind": None}

        def charge(decoding: bool) -> None:
            now = time.time()
            if decoding:
                stats.decode_seconds += now - clock["mark"]
            else:
                stats.prompt_seconds += now - clock["mark"]
            clock["mark"] = now

        def settle(behind) -> List[int]:
            """Fill in the picks that were on their way; the requests that picked a stop token."""
            picks, ids = behind
            stopped = []
            for rid, tok in zip(ids, picks.tolist()):
                r = reqs[rid]
                if r.stopped:                        # a row that ran ahead of its request's end
                    continue
                at = len(r.tokens) - 1
                while r.tokens[at] is not None:      # the one place that is still open
                    at -= 1
                if int(tok) in stop:
                    del r.tokens[at:], r.out[at - r.prompt_len:]
                    r.stopped = True
                    stopped.append(rid)
                    continue
                r.tokens[at] = int(tok)
                r.out[at - r.prompt_len] = int(tok)
            return stopped

        try:
            while any(not r.done for r in reqs.values()):
                plan, preempted = sched.plan([cache.free_pages(g) for g in range(n_groups)])
                feed = (behind is not None and not preempted and [p.id for p in plan] == behind[1]
                        and all(p.count == 1 and p.wants_logits for p in plan))
                take_prepared = (prepared is not None and not preempted and [p.id for p in plan] == prepared
                                 and all(p.count == 1 and p.wants_logits for p in plan))
                if prepared is not None and not take_prepared:
                    self.engine.drop_prepared()
                prepared = None
                stopped = []
                if behind is not None and not feed:
                    stopped = settle(behind)
                    behind = None
                for rid in preempted:
                    self.engine.release(rid)
                    stats.preemptions += 1
                if stopped:
                    # learnt before the step was launched: those requests leave it
                    for rid in stopped:
                        if not reqs[rid].done:
                            reqs[rid].done = True
                            sched.remove(rid)
                            self.engine.release(rid)
                    plan = [p for p in plan if not reqs[p.id].stopped]
                    stopped = []
                    if not plan:
                        continue
                if not plan:
                    raise RuntimeError("the scheduler has requests but planned nothing: the cache pool is too small")
                decoding = all(p.count == 1 and p.start > 0 for p in plan)
                if clock["kind"] is not None and clock["kind"] != decoding:
                    torch.cuda.synchronize()         # the steps of the other kind have run: their time is theirs
                    charge(clock["kind"])
                clock["kind"] = decoding
                t_step = time.time()
                if feed:
                    logits = self.engine.step_from_picks([p.id for p in plan])
                    stopped = settle(behind)     # the step before: read while this one runs
                    behind = None
                elif take_prepared:
                    logits = self.engine.run_prepared([reqs[p.id].tokens[p.start] for p in plan])
                else:
                    entries = [StepEntry(p.id, reqs[p.id].tokens[p.start:p.start + p.count],
                                         [p.count - 1] if p.wants_logits else []) for p in plan]
                    logits = self.engine.step(entries)
                stats.steps += 1
                wanted = [p for p in plan if p.wants_logits]
                greedy_step = bool(wanted) and all(reqs[p.id].sampler is None for p in wanted)
                picks = []
                late = None
                if wanted:
                    if greedy_step and ahead_ok and len(wanted) == len(plan) and self.engine.picks_async() is not None:
                        late = self.engine.picks_async()        # read after the next step is queued
                    elif greedy_step and self.engine.last_picks is not None:
                        picks = self.engine.last_picks.tolist()     # a decoding step picked greedily already
                    else:
                        on_their_way = PendingRowPicks(self.rt, logits, [reqs[p.id].sampler for p in wanted],
                                                       [reqs[p.id].tokens for p in wanted])
                        # the device is busy with the step and the candidates: time to prepare the next step
                        if (ahead_ok and len(wanted) == len(plan) and all(p.count == 1 for p in plan)
                                and all(len(reqs[p.id].out) + 1 < reqs[p.id].max_new for p in plan)
                                and sched.counts()[0] == 0
                                and all(cache.free_pages(g) >= 2 * len(plan) + 2 for g in range(n_groups))):
                            try:
                                self.engine.prepare_continue([p.id for p in plan])
                                prepared = [p.id for p in plan]
                            except (OutOfPages, StepError):
                                prepared = None
                        picks = on_their_way.finish()
                at = 0
                for p in plan:
                    r = reqs[p.id]
                    appended = finished = False
                    if r.stopped:                    # this step ran a row for it in vain
                        at += 1
                        finished = not r.done
                    elif p.wants_logits:
                        tok = None if late is not None else int(picks[at])
                        at += 1
                        stats.decided += 1
                        if tok is not None and tok in stop:
                            finished = True
                        else:
                            r.tokens.append(tok)
                            r.out.append(tok)
                            appended = True
                            finished = len(r.out) >= r.max_new
                    else:
                        stats.prompt_tokens += p.count
                    sched.commit(p.id, p.count, appended, finished)
                    if finished:
                        r.done = True
                        self.engine.release(p.id)
                if late is not None:
                    behind = (late, [p.id for p in plan])
                if trace is not None:
                    torch.cuda.synchronize()
                    waiting, running, _ = sched.counts()
                    trace.line(t_step, (time.time() - t_step) * 1e3, plan, waiting, running, len(preempted))
                charge(decoding)
                if decoding:
                    stats.decode_steps += 1
                    stats.decode_tokens += len(plan)
                else:
                    stats.prompt_tokens += sum(p.count for p in plan if p.wants_logits and p.count > 1)
            if behind is not None:
                settle(behind)
                behind = None
            if clock["kind"] is not None:
                torch.cuda.synchronize()
                charge(clock["kind"])
        finally:
            self.engine.drop_prepared()
            for rid in order:
                self.engine.release(rid)
        stats.seconds = time.time() - t0
        self.last_stats = stats
        outs = [reqs[rid].out for rid in order]
        return outs

    # ------------------------------------------------------------------ logits
    def logits(self, token_ids: Sequence[int], all_positions: bool = False) -> torch.Tensor:
        """float32 logits after `token_ids`: at the last position [vocab], or at every position
        [len, vocab], as a tensor of the caller's own.  The cache is left as it was."""
        ids = list(token_ids)
        rid = ("logits", self._next_id)
        self._next_id += 1
        want = list(range(len(ids))) if all_positions else [len(ids) - 1]
        out = self.engine.step([StepEntry(rid, ids, want)], end=[rid]).clone()     # a one-token step returns a view
        return out if all_positions else out[0]


def load(model: Union[str, dict, ModelConfig], dtype: str = "bfloat16", *, random_seed: Optional[int] = None,
         init_std: float = 0.02, device: str = "cuda:0", page_size: int = 64, num_pages: int = 0,
         max_cache_tokens: int = 0, memory_fraction: float = 0.85, max_seqs: int = 64, max_batch_tokens: int = 2048,
         max_seq_len: int = 0, use_graphs: bool = True) -> LLM:
    """A model folder (config.json + safetensors), or a configuration (a dict of config.json
    keys or a ModelConfig) with `random_seed` for random weights, to a ready `LLM`."""
    rt = Runtime(dtype, device)
    if isinstance(model, str):
        m = load_model(model, rt)
    else:
        config = config_from_dict(model) if isinstance(model, dict) else model
        if random_seed is None:
            raise ValueError("a configuration without a model folder needs random_seed")
        m = random_model(config, rt, random_seed, init_std)
    cfg = EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_cache_tokens=max_cache_tokens,
                       memory_fraction=memory_fraction, max_seqs=max_seqs, max_batch_tokens=max_batch_tokens,
                       max_seq_len=max_seq_len, use_graphs=use_graphs)
    return LLM(m, rt, cfg)
