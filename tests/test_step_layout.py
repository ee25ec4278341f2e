"""The native layout of a step (csrc/host/step.cpp): entries checked and their tokens laid side by
side in one call.  Against the obvious loops, for random steps, and every refusal."""
import ctypes
import random

import numpy as np

from axon_amd.cache.manager import host_lib


def layout(entries, vocab=1000, max_len=500, stride=None):
    """entries: (slot, positions held, tokens, wanted places)."""
    flat = [np.asarray(t, dtype=np.int64) for _, _, t, _ in entries]
    wants = [np.asarray(w, dtype=np.int64) for *_, w in entries]
    counts = np.array([len(t) for t in flat], dtype=np.int64)
    want_counts = np.array([len(w) for w in wants], dtype=np.int64)
    tokens = np.concatenate(flat) if flat else np.zeros(0, np.int64)
    want = np.concatenate(wants) if wants else np.zeros(0, np.int64)
    slots = np.array([s for s, *_ in entries], dtype=np.int32)
    cached = np.array([c for _, c, *_ in entries], dtype=np.int64)
    total = int(counts.sum())
    stride = stride or max(total, 1)
    meta = np.full((3, stride), -7, dtype=np.int32)
    rows = np.full(max(len(want), 1), -7, dtype=np.int32)
    refused, message = ctypes.c_int(-1), ctypes.create_string_buffer(200)
    p = lambda a: ctypes.c_void_p(a.ctypes.data)
    rc = host_lib().axh_step_layout(len(entries), p(slots), p(cached), p(counts), p(tokens), p(want), p(want_counts), vocab,
                                    max_len, p(meta), stride, p(rows), ctypes.byref(refused), message, 200)
    return rc, refused.value, message.value.decode(), meta, rows


def test_random_steps_are_laid_out_as_the_plain_loops_do():
    rng = random.Random(3)
    for _ in range(200):
        entries = []
        for _e in range(rng.randrange(1, 6)):
            n = rng.choice([1, 1, 2, 7, 40])
            held = rng.randrange(0, 300)
            want = sorted(rng.sample(range(n), rng.randrange(0, n + 1)))
            entries.append((rng.randrange(0, 16), held, [rng.randrange(1000) for _ in range(n)], want))
        rc, refused, message, meta, rows = layout(entries)
        tokens, positions, slots, wanted, at = [], [], [], [], 0
        for slot, held, toks, want in entries:
            tokens += toks
            positions += list(range(held, held + len(toks)))
            slots += [slot] * len(toks)
            wanted += [at + w for w in want]
            at += len(toks)
        assert rc == at and refused == -1 and message == ""
        assert meta.tolist() == [tokens, positions, slots] and rows[:len(wanted)].tolist() == wanted


def test_a_refused_step_names_the_entry_and_writes_nothing():
    good = (2, 10, [5, 6, 7], [2])
    for bad, code, text in [((1, 0, [], []), -1, "brings no tokens"),
                            ((1, 0, [5, 1000], [0]), -2, "token 1000 is outside the vocabulary of 1000"),
                            ((1, 0, [5, -1], [0]), -2, "token -1 is outside"),
                            ((1, 0, [5, 6], [2]), -3, "wanted place 2 is outside its 2 tokens"),
                            ((1, 0, [5, 6], [-1]), -3, "wanted place -1"),
                            ((1, 499, [5, 6], [0]), -4, "would reach 501 positions, at most 500")]:
        rc, refused, message, meta, rows = layout([good, bad])
        assert (rc, refused) == (code, 1) and text in message
        assert (meta == -7).all() and (rows == -7).all()
    rc, refused, message, meta, _ = layout([good, good], stride=5)
    assert rc == -5 and refused == -1 and "6 tokens, room for 5" in message and (meta == -7).all()
