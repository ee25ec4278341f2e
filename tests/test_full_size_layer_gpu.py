"""One layer of the sizes the engine is measured at (width 3584, 28 query heads on 4 kv heads of
128, feed-forward 18944) and one of the next size up (width 5120, 40 heads on 8, feed-forward
13824, and the one after that with a feed-forward of 27648), with a small vocabulary, against the plain implementation: the tiny configurations of
the other tests never meet the kernels that these widths select (products that split K between
blocks, norms finished by the product before them, the prompt kernel with a group of 7 or 5,
decoding over several chunks).  A mixed schedule takes every product through each of its
classes of rows (up to 16, 64, 256, more)."""
import pytest
import torch

import axon_amd
from axon_amd.config import config_from_dict
from axon_amd.engine import StepEntry
from axon_amd.weights import write_random_model
from helpers import tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

FULL = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=1, hidden_size=3584, intermediate_size=18944,
            num_attention_heads=28, num_key_value_heads=4, head_dim=128, vocab_size=1024, max_position_embeddings=4096,
            rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)


# the layer of the next size up: another width, a group of 5 query heads, other feed-forward width
WIDER = dict(FULL, hidden_size=5120, intermediate_size=13824, num_attention_heads=40, num_key_value_heads=8,
             rms_norm_eps=1e-5)


# and the largest measured size: the same width, a feed-forward twice as wide (K 27,648 for the down projection)
WIDEST = dict(WIDER, intermediate_size=27648)


def _layer_case(tmp_path_factory, sizes, name):
    d = str(tmp_path_factory.mktemp(name))
    write_random_model(config_from_dict(sizes), d, seed=31, std=0.02, storage="bfloat16")
    cfg, w = P.load_plain(d)
    g = torch.Generator().manual_seed(2)
    prompts = {rid: torch.randint(0, sizes["vocab_size"], (n,), generator=g).tolist()
               for rid, n in (("a", 620), ("b", 150), ("c", 61))}
    oracle = {rid: P.forward_logits(cfg, w, toks) for rid, toks in prompts.items()}
    return d, prompts, oracle


@pytest.fixture(scope="module")
def full_layer(tmp_path_factory):
    return _layer_case(tmp_path_factory, FULL, "full_layer")


@pytest.fixture(scope="module")
def wider_layer(tmp_path_factory):
    return _layer_case(tmp_path_factory, WIDER, "wider_layer")


@pytest.fixture(scope="module")
def widest_layer(tmp_path_factory):
    return _layer_case(tmp_path_factory, WIDEST, "widest_layer")


@pytest.mark.parametrize("dtype,page", [("bfloat16", 16), ("bfloat16", 64), ("bfloat16", 8), ("float32", 16)])
def test_a_layer_of_the_measured_sizes_through_every_class_of_rows(dtype, page, full_layer):
    _through_every_class_of_rows(dtype, page, full_layer)


def test_a_layer_of_the_next_size_through_every_class_of_rows(wider_layer):
    _through_every_class_of_rows("bfloat16", 16, wider_layer)


def test_a_layer_of_the_largest_size_through_every_class_of_rows(widest_layer):
    _through_every_class_of_rows("bfloat16", 16, widest_layer)


def _through_every_class_of_rows(dtype, page, case):
    d, prompts, oracle = case
    n_pages = 1024 // page + 4
    llm = axon_amd.load(d, dtype=dtype, page_size=page, num_pages=n_pages, max_seqs=4, max_batch_tokens=512)
    eng = llm.engine
    fed = {rid: 0 for rid in prompts}
    worst = 0.0
    seen = {}

    def step(parts, end=()):
        """parts: (request, tokens to feed, wanted places among them)"""
        nonlocal worst
        entries, where = [], []
        for rid, n, want in parts:
            at = fed[rid]
            entries.append(StepEntry(rid, prompts[rid][at:at + n], want))
            where += [(rid, at + w) for w in want]
            fed[rid] = at + n
        logits = eng.step(entries, end=end)
        if where:
            got = logits.cpu().double()
            for row, (rid, pos) in zip(logits.cpu(), where):
                seen[(rid, pos)] = row.clone()
            for row, (rid, pos) in zip(got, where):
                ref = oracle[rid][pos]
                err = float((row - ref).abs().max())
                assert err <= tolerance(dtype, ref), (rid, pos, err)
                worst = max(worst, err / tolerance(dtype, ref))

    step([("a", 300, [0, 150, 299])])                              # a prompt portion of more than 256 rows
    step([("a", 130, [129]), ("b", 70, [3, 69])])                  # 200 rows: two portions
    step([("a", 150, [149]), ("b", 2, [1]), ("c", 40, [39])])      # 192 rows, a portion of two tokens
    step([("a", 1, [0]), ("b", 30, [29]), ("c", 19, [18])])        # 50 rows: a decoded token beside portions
    step([("a", 1, [0]), ("b", 40, [0, 39]), ("c", 1, [0])])       # 42 rows
    for _ in range(8):                                             # single tokens: the short-step kernels, graphs
        step([("a", 1, [0]), ("b", 1, [0])])
    step([("c", 1, [0])], end=["c"])
    step([("a", 22, list(range(22)))])                             # 22 rows of one request, all wanted
    for _ in range(8):
        step([("a", 1, [0])])                                      # over 600 positions: three chunks
    assert fed == {"a": 620, "b": 150, "c": 61}
    eng.release_all()
    # every row again with its request alone and whole in one step: the same bits, in both precisions
    for rid in prompts:
        places = sorted(pos for r, pos in seen if r == rid)
        alone = eng.step([StepEntry(rid + "!", prompts[rid], places)], end=[rid + "!"]).cpu()
        for row, pos in zip(alone, places):
            assert torch.equal(row, seen[(rid, pos)]), (rid, pos)
    eng.cache.check()
    assert eng.cache.free_pages() == n_pages
