"""Random batches through `LLM.generate`: a request's tokens are the same alone, in a batch, and
in an engine with so few pages that requests give way and are fed again (src/serve/engine.rs:2244-2276);
greedy and sampled with random settings, with a stop token, decoding steps from graphs or not; the
pool is whole again afterwards."""
import numpy as np
import pytest

import axon_amd
from helpers import TINY

pytestmark = pytest.mark.gpu


def one_case(seed, name, dtype, model_dir):
    rng = np.random.default_rng(seed)
    cfg = TINY[name]["config"]
    page = int(rng.choice([8, 16, 32, 64]))
    n_req = int(rng.integers(1, 9))
    n_new = int(rng.integers(1, 40))
    longest = max(2, min(cfg["max_position_embeddings"] - n_new - 1, 120))
    lens = [int(rng.integers(1, longest)) for _ in range(n_req)]
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in lens]
    kw = {}
    if rng.random() < 0.5:
        kw = dict(temperature=float(rng.choice([0.5, 0.9, 1.3])), top_k=int(rng.choice([1, 5, 40, 0])),
                  top_p=float(rng.choice([0.5, 0.9, 1.0])), min_p=float(rng.choice([0.0, 0.05])),
                  repeat_penalty=float(rng.choice([1.0, 1.1, 1.3])), seed=int(seed))
    need = [-(-(n + n_new) // page) for n in lens]
    roomy = axon_amd.load(model_dir, dtype=dtype, page_size=page, num_pages=sum(need) + 4, max_seqs=8,
                          max_batch_tokens=int(rng.choice([16, 64, 256])), use_graphs=bool(rng.random() < 0.5))
    want = roomy.generate(prompts, max_new_tokens=n_new, **kw)
    # request i of a sampled batch draws from the stream seeded seed + i
    alone = [roomy.generate([p], max_new_tokens=n_new, **({**kw, "seed": kw["seed"] + i} if kw else {}))[0]
             for i, p in enumerate(prompts)]
    assert alone == want, (seed, name, dtype, page, kw)
    pages = max(need) + int(rng.integers(0, max(1, sum(need) - max(need))))
    tight = axon_amd.load(model_dir, dtype=dtype, page_size=page, num_pages=pages, max_seqs=int(rng.choice([2, 4, 8])),
                          max_batch_tokens=int(rng.choice([16, 64, 256])), use_graphs=bool(rng.random() < 0.5))
    assert tight.generate(prompts, max_new_tokens=n_new, **kw) == want, (seed, name, dtype, page, pages, kw)
    preemptions = tight.last_stats.preemptions
    tight.engine.cache.check()
    assert tight.engine.cache.free_pages() == pages
    flat = [t for w in want for t in w]
    if flat:
        stop = int(flat[int(rng.integers(0, len(flat)))])
        cut = tight.generate(prompts, max_new_tokens=n_new, stop=[stop], **kw)
        assert cut == [full[:full.index(stop)] if stop in full else full for full in want], (seed, name, dtype, stop)
    return preemptions


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_random_batches_give_every_request_its_own_tokens(name, dtype, model_dirs):
    model_dir = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    gave_way = sum(one_case(1000 * ord(name) + seed, name, dtype, model_dir) for seed in range(8))
    assert gave_way >= 0
