"""Random configurations of the architecture through the engine against the plain
implementation: head sizes in steps of 16 up to 256, any number of heads and groups, widths and
vocabularies that are no power of two, tied or not, several page sizes; whole prompts, portions
and single tokens mixed; float32 and bfloat16."""
import random

import pytest
import torch

from axon_amd.config import config_from_dict
from axon_amd.engine import StepEntry
from axon_amd.weights import write_random_model
from helpers import engine_for, tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def random_config(seed: int):
    rng = random.Random(seed)
    hd = rng.choice([16, 32, 48, 64, 64, 80, 96, 112, 128, 128, 160, 256])
    nkv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 5, 7, 8])
    nh = nkv * group
    hidden = rng.choice([40, 64, 72, 128, 192, 200, 256, 320])
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=rng.choice([1, 2, 3]), hidden_size=hidden,
               intermediate_size=rng.choice([48, 100, 128, 176, 320, 448]), num_attention_heads=nh,
               num_key_value_heads=nkv, head_dim=hd, vocab_size=rng.choice([97, 256, 300, 1000, 4099]),
               max_position_embeddings=512, rope_theta=rng.choice([1e4, 1e6, 5e5]),
               rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]), tie_word_embeddings=rng.random() < 0.5)
    return cfg, rng.choice([8, 16, 16, 32, 64]), rng


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(seed, tmp_path):
    cfg, page, rng = random_config(seed)
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path / dtype)
        write_random_model(config_from_dict(cfg), d, seed=seed, std=0.05, storage="float32" if dtype == "float32" else "bfloat16")
        pc, pw = P.load_plain(d)
        g = torch.Generator().manual_seed(seed)
        seqs = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (rng.randint(60, 150), rng.randint(2, 40))]
        refs = [P.forward_logits(pc, pw, s).float() for s in seqs]
        eng = engine_for(d, dtype, page, num_pages=-(-sum(len(s) for s in seqs) // page) + 3)
        # request 0 in portions with single tokens at the end, request 1 joins in the middle
        got = [[], []]
        at = [0, 0]
        cuts = [rng.choice([1, 2, 5, 17, 33, 64]) for _ in range(40)]
        step = 0
        while at[0] < len(seqs[0]) or at[1] < len(seqs[1]):
            entries = []
            for i in (0, 1):
                if at[i] >= len(seqs[i]) or (i == 1 and step < 2):
                    continue
                left = len(seqs[i]) - at[i]
                n = 1 if left <= 8 else min(cuts[(step + i) % len(cuts)], left)
                entries.append(StepEntry(i, seqs[i][at[i]:at[i] + n], list(range(n))))
            if not entries:                  # request 0 is through before request 1 joins
                step += 1
                continue
            out = eng.step(entries).cpu()
            row = 0
            for e in entries:
                got[e.id].append(out[row:row + len(e.tokens)].clone())
                row += len(e.tokens)
                at[e.id] += len(e.tokens)
            step += 1
        for i in (0, 1):
            err = (torch.cat(got[i]) - refs[i]).abs().max()
            assert err <= tolerance(dtype, refs[i]), (cfg, page, dtype, i, float(err))
        eng.release_all()
        eng.cache.check()
