"""Random schedules through Engine.step against the same requests run whole and alone, bit for
bit (src/lm.rs:272-278: a row's result is what it is alone, whatever else is in the step): up to
four live requests, portions of random size beside single tokens, requests that sit a step out,
requests given up half way and fed again from their first token, a pool of pages so small that
pages are used again (handed out in a shuffled order or not), decoding steps from graphs or not;
the five tiny configurations, float32 and bfloat16, their own page size or another."""
import numpy as np
import pytest
import torch

from axon_amd.engine import StepEntry
from helpers import TINY, engine_for

pytestmark = pytest.mark.gpu


def pages_of(n, page):
    return -(-n // page)


def run_schedule(seed, name, dtype, model_dir):
    rng = np.random.default_rng(seed)
    cfg = TINY[name]["config"]
    page = int(rng.choice([8, 16, 32, 64])) if rng.random() < 0.5 else TINY[name]["page_size"]
    n_req = int(rng.integers(3, 8))
    lens = [int(rng.integers(1, min(cfg["max_position_embeddings"], 330))) for _ in range(n_req)]
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in lens]
    # every request whole and alone
    eng = engine_for(model_dir, dtype, page, num_pages=max(pages_of(n, page) for n in lens) + 2)
    whole = [eng.step([StepEntry(("w", i), p, list(range(len(p))))], end=[("w", i)]).cpu().clone()
             for i, p in enumerate(prompts)]
    eng.cache.check()
    # the schedule: room for the four longest requests and one page more
    pool = sum(sorted((pages_of(n, page) for n in lens), reverse=True)[:4]) + 1
    eng = engine_for(model_dir, dtype, page, num_pages=pool, use_graphs=bool(rng.random() < 0.5),
                     shuffle_pages_seed=int(seed) if rng.random() < 0.5 else -1)
    waiting = [(i, 0) for i in range(n_req)]          # (request, which life)
    live = {}                                         # id -> [request, tokens fed]
    steps = rows = 0
    while waiting or live:
        steps += 1
        assert steps < 5000, "the schedule does not end"
        while waiting and len(live) < 4:
            i, life = waiting[0]
            held = sum(pages_of(max(at, 1), page) for _, at in live.values())
            if live and held + pages_of(lens[i], page) > pool:
                break                                              # no room yet for its whole length
            waiting.pop(0)
            live[(i, life)] = [i, 0]
        entries, ends = [], []
        for rid in list(live):
            i, at = live[rid]
            if len(live) > 1 and rng.random() < 0.15:
                continue                                           # sits this step out
            left = lens[i] - at
            n = 1 if (rng.random() < 0.4 or left <= 3) else int(min(rng.choice([2, 3, 7, 16, 29, 64, 130]), left))
            if pages_of(at + n, page) - pages_of(at, page) > pool - sum(pages_of(a, page) for _, a in live.values()):
                continue                                           # no page for these tokens in this step
            want = list(range(n)) if rng.random() < 0.7 else [n - 1]
            entries.append((rid, StepEntry(rid, prompts[i][at:at + n], want), at))
            live[rid][1] = at + n
            if at + n == lens[i]:
                ends.append(rid)
            elif rid[1] == 0 and at + n >= lens[i] // 2 and rng.random() < 0.1:
                ends.append(rid)                                   # given up; fed again later from its first token
                waiting.append((i, 1))
        if not entries:
            rid = max(live, key=lambda r: live[r][1])              # nobody can move: the largest makes room
            eng.step([], end=[rid])
            i, _ = live.pop(rid)
            waiting.append((i, rid[1] + 1))
            continue
        out = eng.step([e for _, e, _ in entries], end=ends).cpu()
        row = 0
        for rid, e, at in entries:
            for w in e.want:
                assert torch.equal(out[row], whole[rid[0]][at + w]), (seed, name, dtype, page, rid, at + w)
                row += 1
        rows += row
        for rid in ends:
            live.pop(rid, None)
    eng.cache.check()
    return rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_random_schedules_give_the_bits_of_a_request_alone(name, dtype, model_dirs):
    model_dir = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    rows = sum(run_schedule(100 * ord(name) + seed, name, dtype, model_dir) for seed in range(12))
    assert rows > 1000
