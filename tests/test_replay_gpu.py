"""Trace replay through bin/trace_run, as a user drives it: the same requests whole, with the
last 32 tokens decoded one by one, in portions of changing size down to two tokens, mixed
with other requests in a pool so small that pages are used again, and given up half way and fed
again from their first token; float32 and bfloat16; all compared with the plain implementation,
and with each other bit for bit (src/lm.rs:272-278: a row's result is what it is alone, whatever
else is in the step)."""
import numpy as np
import pytest
import torch

from helpers import TINY, TraceBuilder, prompts_for, run_trace, tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [1, 5, 17, 33, 70, 100], "B": [2, 9, 70, 41, 130, 64], "C": [3, 66, 129], "D": [4, 70, 300, 131],
           "E": [2, 129, 64, 520]}


def oracle(model_dir, prompts):
    cfg, w = P.load_plain(model_dir)
    return [P.forward_logits(cfg, w, p).float().numpy() for p in prompts]


def first_life(rid):
    """The request a row belongs to: a request fed again after it was given up carries a mark."""
    return rid.rstrip("~")


def check(rows, refs, ids, dtype):
    worst = 0.0
    for (rid, pos), got in rows.items():
        rid = first_life(rid)
        ref = refs[ids.index(rid)][pos]
        tol = tolerance(dtype, torch.from_numpy(refs[ids.index(rid)]))
        err = float(np.abs(got - ref).max())
        assert err <= tol, f"request {rid} position {pos}: |diff| {err} > {tol}"
        worst = max(worst, err)
    return worst


def whole(prompts):
    tb = TraceBuilder()
    for i, p in enumerate(prompts):
        tb.step([(f"r{i}", p, list(range(len(p))))], end=[f"r{i}"])
    return tb


def last_32_one_by_one(prompts):
    tb = TraceBuilder()
    for i, p in enumerate(prompts):
        head = max(len(p) - 32, 1)
        tb.step([(f"r{i}", p[:head], [head - 1])])
        for t in range(head, len(p)):
            tb.step([(f"r{i}", [p[t]], [0])], end=[f"r{i}"] if t == len(p) - 1 else [])
        if head == len(p):
            tb.step([], end=[f"r{i}"])
    return tb


def changing_portions(prompts, sizes=(7, 2, 16, 3, 2, 33, 1, 5, 64, 2)):
    tb = TraceBuilder()
    for i, p in enumerate(prompts):
        at, k = 0, i
        while at < len(p):
            n = min(sizes[k % len(sizes)], len(p) - at)
            tb.step([(f"r{i}", p[at:at + n], list(range(n)))], end=[f"r{i}"] if at + n == len(p) else [])
            at, k = at + n, k + 1
    return tb


def mixed(prompts, seed=0, live_at_most=4):
    """Up to four live requests: portions of some beside single tokens of others; a request
    may sit out a step; finished requests give their pages to the ones that start later."""
    rng = np.random.default_rng(seed)
    tb = TraceBuilder()
    waiting = list(range(len(prompts)))
    live = {}
    while waiting or live:
        while waiting and len(live) < live_at_most:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for i in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                         # left out of this step
            p, at = prompts[i], live[i]
            decode = at >= max(len(p) - 32, 1) or rng.random() < 0.3
            n = 1 if decode else int(min(rng.choice([2, 3, 7, 16, 29]), len(p) - at))
            entries.append((f"r{i}", p[at:at + n], list(range(n)) if rng.random() < 0.8 else [n - 1]))
            live[i] = at + n
            if live[i] == len(p):
                end.append(f"r{i}")
                del live[i]
        if entries:
            tb.step(entries, end)
    return tb


def given_up_and_fed_again(prompts, seed=0, live_at_most=3):
    """What a scheduler does when pages run out (src/serve/engine.rs:2244-2276): a request that
    has been fed part of its prompt and has decoded a few tokens is ended, its pages go to the
    others, and later it is fed again from its first token (here under its name with a mark), in
    other portions, up to its end.  Both lives' rows must be those of the whole request."""
    rng = np.random.default_rng(seed)
    tb = TraceBuilder()
    waiting = [(i, f"r{i}") for i in range(len(prompts))]
    live = {}
    while waiting or live:
        while waiting and len(live) < live_at_most:
            i, rid = waiting.pop(0)
            live[rid] = (i, 0)
        entries, end = [], []
        for rid in list(live):
            i, at = live[rid]
            p = prompts[i]
            n = int(min(rng.choice([1, 1, 2, 5, 16, 40]), len(p) - at))
            entries.append((rid, p[at:at + n], list(range(n))))
            at += n
            live[rid] = (i, at)
            if at == len(p):
                end.append(rid)
                del live[rid]
            elif not rid.endswith("~") and at >= len(p) // 2:
                end.append(rid)                                  # given up half way ...
                del live[rid]
                waiting.append((i, rid + "~"))                   # ... and back in the queue, from token 0
        tb.step(entries, end)
    return tb


def max_tokens_for(tb, prompts_by_id):
    """The most tokens live requests hold at any time, each rounded up to 64."""
    live, most = {}, 0
    for s in tb.steps:
        for e in s["entries"]:
            live[e["id"]] = live.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // 64) * 64 for n in live.values()))
        for rid in s["end"]:
            live.pop(rid, None)
    return most


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_schedule_matches_the_plain_implementation(name, dtype, model_dirs, tmp_path):
    model_dir = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    prompts = prompts_for(name, LENGTHS[name], seed=3)
    ids = [f"r{i}" for i in range(len(prompts))]
    refs = oracle(model_dir, prompts)
    page = ["--page-size", str(TINY[name]["page_size"])]
    results = {}
    for label, tb in (("whole", whole(prompts)), ("last32", last_32_one_by_one(prompts)),
                      ("portions", changing_portions(prompts)), ("mixed", mixed(prompts, seed=len(name))),
                      ("refed", given_up_and_fed_again(prompts, seed=len(name)))):
        budget = max_tokens_for(tb, None)
        # the mixed schedule with pages handed out in a shuffled order, and its decoding steps from graphs
        more = ["--shuffle-pages", "5", "--graphs"] if label == "mixed" else []
        out = run_trace(model_dir, dtype, tb.steps, str(tmp_path / label), budget, extra=page + more)
        rows = tb.collect(out)
        check(rows, refs, ids, dtype)
        results[label] = rows
    # every position was asked for in the whole and portions schedules
    assert len(results["whole"]) == sum(len(p) for p in prompts) == len(results["portions"])
    # beyond the tolerance: however the tokens were cut and whatever shared their steps, the logits
    # are the same bits, in float32 and in bfloat16
    for label in ("last32", "portions", "mixed", "refed"):
        for (rid, pos), row in results[label].items():
            assert np.array_equal(row, results["whole"][(first_life(rid), pos)]), (label, rid, pos)


def test_a_step_that_wants_nothing_writes_nothing_and_requests_can_pause(model_dirs, tmp_path):
    model_dir = model_dirs("A")
    p, q = prompts_for("A", [20, 12], seed=9)
    tb = TraceBuilder()
    tb.step([("a", p[:10], [])])                                  # nothing wanted: no file
    tb.step([("b", q[:12], [11])])                                # "a" is left out of this step
    tb.step([("a", p[10:], [9])], end=["a", "b"])
    out = run_trace(model_dir, "float32", tb.steps, str(tmp_path / "o"), 128, extra=["--page-size", "8"])
    assert sorted(out) == [1, 2]
    rows = tb.collect(out)
    refs = oracle(model_dir, [p, q])
    check(rows, refs, ["a", "b"], "float32")
