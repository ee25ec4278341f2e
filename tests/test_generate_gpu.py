"""Generation through the Python entry point and the command line against the plain
implementation: greedy, sampled with a seed, under page pressure (requests give way and come
back), long decoding, and the first tokens of a sequence."""
import os
import subprocess
import sys

import pytest
import torch

import axon_amd
from helpers import ROOT, TINY, prompts_for, tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_greedy_generation_matches_the_plain_loop(name, dtype, model_dirs):
    d = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    cfg, w = P.load_plain(d)
    prompts = prompts_for(name, {"A": [1, 5, 17, 33], "B": [2, 9, 70, 41, 3, 25], "E": [3, 140, 66]}[name], seed=1)
    n_new = {"A": 16, "B": 24, "E": 12}[name]
    llm = axon_amd.load(d, dtype=dtype, page_size=TINY[name]["page_size"], num_pages=64, max_seqs=4, max_batch_tokens=48)
    outs = llm.generate(prompts, max_new_tokens=n_new)
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        if dtype == "float32":
            assert o == P.greedy_generate(cfg, w, p, n_new)
        else:
            # bfloat16 may take another branch at a near tie: follow the engine's own tokens and
            # require each pick to be within tolerance of the oracle's best logit
            logits = P.forward_logits(cfg, w, p + o)
            for i, tok in enumerate(o):
                row = logits[len(p) - 1 + i]
                assert row.max() - row[tok] <= 2 * tolerance(dtype, row), (i, tok)
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 64 and not llm.engine.live


def test_sampled_generation_matches_the_plain_sampler(model_dirs):
    d = model_dirs("B")
    cfg, w = P.load_plain(d)
    prompts = prompts_for("B", [2, 30, 11], seed=2)
    llm = axon_amd.load(d, dtype="float32", page_size=16, num_pages=32, max_seqs=4)
    kw = dict(temperature=0.8, top_k=40, top_p=0.9, min_p=0.0, repeat_penalty=1.1, repeat_last_n=64)
    outs = llm.generate(prompts, max_new_tokens=24, seed=5, **kw)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert o == P.sample_generate(cfg, w, p, 24, temp=0.8, top_k=40, top_p=0.9, min_p=0.0, repeat_penalty=1.1,
                                      repeat_last_n=64, seed=5 + i)
    # the same seed gives the same tokens whatever else is in the batch
    alone = llm.generate([prompts[1]], max_new_tokens=24, seed=6, **kw)[0]
    assert alone == llm.generate(prompts, max_new_tokens=24, seed=5, **kw)[1]
    # top-k off (every token a candidate) and top-k above the device's limit run on the host
    for k in (0, 300):
        o = llm.generate([prompts[0]], max_new_tokens=8, seed=9, temperature=1.2, top_k=k, top_p=1.0, repeat_penalty=1.0)[0]
        assert o == P.sample_generate(cfg, w, prompts[0], 8, temp=1.2, top_k=k, top_p=1.0, min_p=0.0,
                                      repeat_penalty=1.0, repeat_last_n=64, seed=9)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_one_step_ahead_of_the_host(dtype, model_dirs, monkeypatch, tmp_path):
    """A step fed from the previous step's picks on the device gives the logits and tokens of a
    step fed the same tokens from the host, bit for bit; and greedy generation, which runs
    ahead, returns what generation that reads every token first returns, with stop tokens that
    end requests at their first token, in the middle, at their last token and never."""
    from axon_amd.engine import StepEntry
    d = model_dirs("B", dtype)
    prompts = prompts_for("B", [7, 30, 19], seed=11)
    ahead = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=32, max_seqs=4, max_batch_tokens=64).engine
    plain = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=32, max_seqs=4, max_batch_tokens=64).engine
    ids = ["x", "y", "z"]
    for eng in (ahead, plain):
        for rid, p in zip(ids, prompts):
            eng.step([StepEntry(rid, p[:-1], [])])
    first = [StepEntry(rid, [p[-1]], [0]) for rid, p in zip(ids, prompts)]
    ahead.step(first)
    late = ahead.picks_async()
    plain.step(first)
    toks = plain.last_picks.tolist()
    assert late.tolist() == toks
    for i in range(20):
        got = ahead.step_from_picks(ids).clone()
        behind, late = late, ahead.picks_async()
        assert behind.tolist() == toks
        want = plain.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)])
        assert torch.equal(got, want), i
        toks = plain.last_picks.tolist()
    assert late.tolist() == toks
    with pytest.raises(axon_amd.engine.StepError):
        ahead.step_from_picks(["x", "y"])                   # not the last step's requests
    ahead.release("z")
    with pytest.raises(axon_amd.engine.StepError):
        ahead.step_from_picks(ids)
    ahead.release_all()
    ahead.cache.check()

    llm = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=32, max_seqs=4, max_batch_tokens=24)
    more = prompts_for("B", [5, 40, 12, 26, 9], seed=12)
    run_ahead = llm.generate(more, max_new_tokens=21)
    steps_ahead = llm.last_stats.steps
    assert all(len(o) == 21 and None not in o for o in run_ahead)
    stops = [run_ahead[0][0], run_ahead[1][9], run_ahead[2][20], run_ahead[3][1]]
    cut = [o[:min([o.index(s) for s in stops if s in o], default=len(o))] for o in run_ahead]
    assert len(set(len(o) for o in cut)) >= 3 and any(len(o) == 0 for o in cut)
    stopped_ahead = llm.generate(more, max_new_tokens=21, stop=stops)
    assert stopped_ahead == cut
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 32 and not llm.engine.live
    monkeypatch.setenv("AXON_STEP_TRACE", str(tmp_path / "steps.jsonl"))   # tracing reads every token first
    one_by_one = llm.generate(more, max_new_tokens=21)
    assert run_ahead == one_by_one and steps_ahead == llm.last_stats.steps
    assert llm.generate(more, max_new_tokens=21, stop=stops) == cut
    assert len((tmp_path / "steps.jsonl").read_text().splitlines()) == steps_ahead + llm.last_stats.steps
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 32 and not llm.engine.live


def test_stop_tokens_end_a_request_and_are_not_returned(model_dirs):
    d = model_dirs("A")
    cfg, w = P.load_plain(d)
    p = prompts_for("A", [9], seed=4)[0]
    full = P.greedy_generate(cfg, w, p, 12)
    stop = full[5]
    want = P.greedy_generate(cfg, w, p, 12, stop=[stop])
    assert len(want) < 12
    llm = axon_amd.load(d, dtype="float32", page_size=8, num_pages=16, max_seqs=2)
    assert llm.generate(p, max_new_tokens=12, stop=[stop]) == [want]
    assert llm.generate(p, max_new_tokens=0) == [[]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_under_page_pressure_requests_give_way_and_continue_with_the_same_tokens(dtype, model_dirs):
    d = model_dirs("B", "float32" if dtype == "float32" else "bfloat16")
    cfg, w = P.load_plain(d)
    prompts = prompts_for("B", [20, 25, 18, 30, 22], seed=6)
    roomy = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=64, max_seqs=4, max_batch_tokens=32)
    want = roomy.generate(prompts, max_new_tokens=40)
    assert roomy.last_stats.preemptions == 0
    # 9 pages of 16: one request needs up to 70 tokens = 5 pages, so two cannot both finish
    tight = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=9, max_seqs=4, max_batch_tokens=32)
    got = tight.generate(prompts, max_new_tokens=40)
    assert tight.last_stats.preemptions > 0
    # a request that gave way is fed again from its first token (prompt and generated tokens) and goes
    # on with the same tokens: feeding again gives the cache the same bits, in both precisions
    assert got == want
    if dtype == "float32":
        assert got == [P.greedy_generate(cfg, w, p, 40) for p in prompts]
    tight.engine.cache.check()
    assert tight.engine.cache.free_pages() == 9
    # sampled requests keep their random stream across a preemption; a stop token ends one of them early
    s_want = roomy.generate(prompts, max_new_tokens=30, temperature=0.9, seed=3)
    s_got = tight.generate(prompts, max_new_tokens=30, temperature=0.9, seed=3)
    assert s_got == s_want
    stop = s_want[1][7]
    cut = tight.generate(prompts, max_new_tokens=30, temperature=0.9, seed=3, stop=[stop])
    for full, part in zip(s_want, cut):
        assert part == (full[:full.index(stop)] if stop in full else full)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_a_requests_tokens_do_not_depend_on_the_batch(name, dtype, model_dirs):
    """Eighteen requests of different lengths that finish one after the other, so that the
    decoding batch shrinks 18, 17, 16, ... and prompt portions share steps with decoding tokens:
    every request gets the tokens it gets when it runs alone, greedy and sampled with a seed,
    in float32 and in bfloat16 (the matrix-core kernels: head sizes 64 and 128)."""
    d = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    lengths = [3, 70, 9, 130, 17, 33, 64, 65, 2, 40, 100, 5, 21, 90, 12, 150, 7, 48]
    prompts = prompts_for(name, lengths, seed=21)
    page = TINY[name]["page_size"]
    llm = axon_amd.load(d, dtype=dtype, page_size=page, num_pages=18 * (200 // page + 2), max_seqs=18, max_batch_tokens=96)
    for kw in (dict(), dict(temperature=0.8, top_k=40, top_p=0.9, repeat_penalty=1.1, seed=100)):
        news = [4 + 2 * i for i in range(len(prompts))]
        full = llm.generate(prompts, max_new_tokens=max(news), **kw)
        for i, (p, o) in enumerate(zip(prompts, full)):
            solo_kw = dict(kw)
            if "seed" in kw:
                solo_kw["seed"] = kw["seed"] + i            # request i of a call draws from the stream seeded seed + i
            alone = llm.generate([p], max_new_tokens=news[i], **solo_kw)[0]
            assert alone == o[:news[i]], (name, dtype, i, kw)
        # other company, another token budget and so other portions: the same tokens
        llm.cfg.max_batch_tokens = 40
        some = llm.generate(prompts[3:9], max_new_tokens=10, **({**kw, "seed": kw["seed"] + 3} if "seed" in kw else kw))
        llm.cfg.max_batch_tokens = 96
        assert some == [o[:10] for o in full[3:9]]
    llm.engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_stays_on_the_oracle(dtype, model_dirs):
    """300 tokens decoded one by one after a short prompt (pages 8: dozens of page edges, five
    attention blocks), then every decode step's logits against the whole sequence at once."""
    d = model_dirs("A", "float32" if dtype == "float32" else "bfloat16")
    cfg, w = P.load_plain(d)
    p = prompts_for("A", [3], seed=8)[0]
    c = dict(TINY["A"]["config"], max_position_embeddings=512)
    import json, shutil, tempfile
    tmp = tempfile.mkdtemp()
    try:
        shutil.copy(os.path.join(d, "model.safetensors"), tmp)
        json.dump(c, open(os.path.join(tmp, "config.json"), "w"))
        llm = axon_amd.load(tmp, dtype=dtype, page_size=8, num_pages=48, max_seqs=2)
        out = llm.generate(p, max_new_tokens=300)[0]
        seq = p + out
        ref = P.forward_logits(cfg, w, seq).float()
        from axon_amd.engine import StepEntry
        eng = llm.engine
        eng.step([StepEntry("x", seq[:3], [])])
        worst = 0.0
        for t in range(3, len(seq)):
            row = eng.step([StepEntry("x", [seq[t]], [0])])[0].cpu()
            worst = max(worst, float((row - ref[t]).abs().max()))
        eng.release("x")
        assert worst <= tolerance(dtype, ref), worst
    finally:
        shutil.rmtree(tmp)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_first_tokens_of_a_sequence(dtype, model_dirs):
    """Position 0 alone, then 1, 2, 3: no earlier key, the rotation is the identity at 0."""
    d = model_dirs("B", "float32" if dtype == "float32" else "bfloat16")
    cfg, w = P.load_plain(d)
    llm = axon_amd.load(d, dtype=dtype, page_size=16, num_pages=8, max_seqs=2)
    for p in prompts_for("B", [1, 1, 2, 4], seed=10):
        ref = P.forward_logits(cfg, w, p).float()
        got = llm.logits(p, all_positions=True).cpu()
        assert (got - ref).abs().max() <= tolerance(dtype, ref)
        one = llm.logits(p).cpu()
        assert torch.equal(one, got[-1])


def test_a_step_that_does_not_fit_takes_nothing(model_dirs):
    """Two live requests and a new one in a step whose pages do not all fit: the step is refused,
    the live requests hold what they held, the new one was never opened, and the step's tokens
    fed afterwards in two steps give the logits of an undisturbed engine."""
    from axon_amd.cache import OutOfPages
    from axon_amd.engine import StepEntry
    from helpers import engine_for
    d = model_dirs("A")
    p = prompts_for("A", [25, 17, 17], seed=13)
    eng = engine_for(d, "float32", page_size=8, num_pages=6)
    eng.step([StepEntry("a", p[0][:20], []), StepEntry("b", p[1][:9], [])])            # 3 + 2 pages of 6
    cache = eng.cache
    held = lambda: (cache.free_pages(0), {r: (eng.live[r].n_cached, cache.pages_of(0, eng.live[r].slot),
                                               cache.row(0, eng.live[r].slot)) for r in eng.live})
    before = held()
    with pytest.raises(OutOfPages):                                                      # 1 + 1 + 3 pages, 1 free
        eng.step([StepEntry("a", p[0][20:], [4]), StepEntry("b", p[1][9:], [7]), StepEntry("c", p[2], [16])])
    assert held() == before and "c" not in eng.live and cache.free_slots() == 2
    cache.check()
    la = eng.step([StepEntry("a", p[0][20:], [4])], end=["a"]).clone()
    lb = eng.step([StepEntry("b", p[1][9:], [7])], end=["b"]).clone()
    lc = eng.step([StepEntry("c", p[2], [16])], end=["c"]).clone()
    fresh = engine_for(d, "float32", page_size=8, num_pages=16)
    for rid, prompt, got in (("a", p[0], la), ("b", p[1], lb), ("c", p[2], lc)):
        want = fresh.step([StepEntry(rid, prompt, [len(prompt) - 1])], end=[rid])
        assert torch.equal(got, want)
    assert cache.free_pages(0) == 6
    # a context longer than the attention kernels' list of work can name is refused when the engine is
    # built, with that reason; the longest one they take is accepted
    from axon_amd.engine.step import StepError
    from axon_amd.kernels import kernels
    limit = kernels("bfloat16").attention_decode_max_context
    with pytest.raises(StepError, match="contexts of up to"):
        engine_for(d, "bfloat16", page_size=8, num_pages=6, max_seq_len=limit + 1)
    assert engine_for(d, "bfloat16", page_size=8, num_pages=6, max_seq_len=limit).max_seq_len == limit


def test_logits_are_the_callers_own(model_dirs):
    """A one-token step answers from a buffer the next one-token step writes again: `logits`
    hands out a copy."""
    llm = axon_amd.load(model_dirs("A"), dtype="float32", page_size=8, num_pages=8, max_seqs=2)
    a = llm.logits([5])
    kept = a.clone()
    b = llm.logits([7])
    assert torch.equal(a, kept) and not torch.equal(a, b)


def test_command_line_gen_and_logits(model_dirs):
    d = model_dirs("A")
    cfg, w = P.load_plain(d)
    p = prompts_for("A", [7], seed=11)[0]
    ids = " ".join(map(str, p))
    axon = [sys.executable, os.path.join(ROOT, "bin", "axon")]
    r = subprocess.run(axon + ["gen", d, ids, "-n", "10", "--dtype", "float32", "--page-size", "8"], capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == P.greedy_generate(cfg, w, p, 10)
    assert "prompt eval: 7 tok" in r.stderr and "decode: " in r.stderr and "tok/s" in r.stderr
    r = subprocess.run(axon + ["gen", d, ids, "-n", "6", "--dtype", "float32", "--temp", "0.7", "--seed", "4"],
                       capture_output=True, text=True, timeout=300)
    assert [int(t) for t in r.stdout.split()] == P.sample_generate(
        cfg, w, p, 6, temp=0.7, top_k=40, top_p=0.9, min_p=0.0, repeat_penalty=1.1, repeat_last_n=64, seed=4)
    # several prompts in one call: a line each, the lines of the prompts run alone
    q = prompts_for("A", [12], seed=12)[0]
    r = subprocess.run(axon + ["gen", d, ids, " ".join(map(str, q)), "-n", "5", "--dtype", "float32", "--page-size", "8"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [[int(t) for t in line.split()] for line in r.stdout.splitlines()] == [
        P.greedy_generate(cfg, w, p, 5), P.greedy_generate(cfg, w, q, 5)]
    assert f"prompt eval: {len(p) + len(q)} tok" in r.stderr
    # a configuration and a seed in place of a model folder: the same seed, the same tokens
    config = os.path.join(d, "config.json")
    runs = [subprocess.run(axon + ["gen", config, ids, "-n", "6", "--random-weights", seed, "--std", "0.3", "--dtype", "float32"],
                           capture_output=True, text=True, timeout=300) for seed in ("3", "3", "4")]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr
    assert runs[0].stdout == runs[1].stdout != runs[2].stdout and len(runs[0].stdout.split()) == 6
    r = subprocess.run(axon + ["logits", d, ids, "-k", "3", "--dtype", "float32"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    ref = P.forward_logits(cfg, w, p)[-1]
    top = torch.topk(ref, 3)
    lines = [l.split() for l in r.stdout.splitlines() if "logit" in l]
    assert [int(l[0]) for l in lines] == top.indices.tolist()
    assert all(abs(float(l[2]) - v) < 1e-3 for l, v in zip(lines, top.values.tolist()))
