"""The native host sampler against the plain one and the reference's own vectors."""
import math
import random

import pytest
import torch

from axon_amd.sampling import Rng, Sampler, SamplingParams, argmax_row
from plain import qwen2_plain as P


def test_rng_matches_the_plain_stream():
    for seed in (0, 1, 42, 2 ** 63 + 5):
        a, b = Rng(seed), P.PlainRng(seed)
        assert [a.next_u64() for _ in range(20)] == [b.next_u64() for _ in range(20)]
        assert [a.f64() for _ in range(5)] == [b.f64() for _ in range(5)]


def test_argmax_row_rules():
    inf, nan = float("inf"), float("nan")
    for row in ([-inf] * 5, [1.0, 3.0, 3.0, 2.0], [nan, 1.0, nan], [nan, nan, nan], [-1.0, 0.0, -0.0],
                [0.0, -0.0, -1.0], [5.0], [-3.0, -3.0]):
        assert argmax_row(torch.tensor(row, dtype=torch.float32)) == P.argmax_last(row), row


def params(**kw):
    base = dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, repeat_last_n=0, seed=0)
    base.update(kw)
    return SamplingParams(**base)


class FixedU(Sampler):
    """A sampler whose next uniform number is given (the pick is a function of u)."""

    def __init__(self, p, u):
        super().__init__(p)
        self.u = u
        self.rng = self

    def f64(self):
        return self.u


def test_reference_vectors_through_the_native_sampler():
    l = torch.tensor([math.log(0.5), math.log(0.3), math.log(0.2)], dtype=torch.float32)
    for u, i in [(0.0, 0), (0.499, 0), (0.501, 1), (0.799, 1), (0.801, 2), (0.9999, 2)]:      # src/sample.rs:1138-1148
        assert FixedU(params(), u).pick_row(l, []) == i
    assert FixedU(params(top_p=0.49), 0.99).pick_row(l, []) == 0
    assert FixedU(params(top_p=0.51), 0.99).pick_row(l, []) == 1
    assert FixedU(params(min_p=0.61), 0.99).pick_row(l, []) == 0
    assert FixedU(params(min_p=0.41), 0.99).pick_row(l, []) == 1
    assert FixedU(params(top_k=2, top_p=0.6), 0.99).pick_row(l, []) == 0
    inf, nan = float("inf"), float("nan")
    assert FixedU(params(), 0.9999).pick_row(torch.tensor([-inf, 2.0, nan]), []) == 1
    assert FixedU(params(), 0.5).pick_row(torch.tensor([-inf] * 3), []) == 2
    assert FixedU(params(), 0.5).pick_row(torch.tensor([nan] * 3), []) == 2
    # the penalty changes the order: 3.0 / 1.1 < 2.8 (src/sample.rs:1051-1059)
    s = FixedU(params(repeat_penalty=1.1, repeat_last_n=64, top_k=1), 0.0)
    assert s.pick_row(torch.tensor([3.0, 2.8]), [0]) == 1


@pytest.mark.parametrize("seed", range(4))
def test_random_rows_match_the_plain_sampler(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(40):
        n = rng.choice([5, 64, 300])
        logits = (torch.randn(n, generator=g) * rng.choice([0.5, 3.0])).float()
        if rng.random() < 0.3:
            logits[rng.randrange(n)] = logits[rng.randrange(n)]                     # a tie
        hist = [rng.randrange(n) for _ in range(rng.randint(1, 30))]
        kw = dict(temperature=rng.choice([0.3, 0.8, 1.5]), top_k=rng.choice([0, 1, 7, 40]),
                  top_p=rng.choice([1.0, 0.9, 0.5]), min_p=rng.choice([0.0, 0.05, 0.3]),
                  repeat_penalty=rng.choice([1.0, 1.1, 2.0]), repeat_last_n=rng.choice([0, 4, 64]))
        u = rng.random()
        got = FixedU(SamplingParams(seed=0, **kw), u).pick_row(logits.clone(), hist)
        pen = P.penalize(logits.tolist(), hist, kw["repeat_last_n"], kw["repeat_penalty"])
        pen = [float(torch.tensor(v, dtype=torch.float32)) for v in pen]                # 32-bit, as the engine's rows
        want = P.pick(P.candidates(pen, kw["top_k"]), kw["temperature"], kw["top_p"], kw["min_p"], u)
        assert got == want, kw


def test_settings_are_checked():
    for bad in (dict(temperature=-1.0), dict(temperature=101.0), dict(top_p=1.5), dict(min_p=-0.1),
                dict(repeat_penalty=0.0), dict(top_k=-1)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    assert SamplingParams().greedy and not SamplingParams(temperature=0.8).greedy
    d = SamplingParams(temperature=0.8)
    assert (d.top_k, d.top_p, d.min_p, d.repeat_penalty, d.repeat_last_n) == (40, 0.9, 0.0, 1.1, 64)   # src/sample.rs:179-190
