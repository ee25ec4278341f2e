"""Shared by the tests: the tiny configurations, model folders, prompts, tolerances, schedules."""
import json
import os
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Two tiny configurations of the architecture that differ in every size and option: head
# counts and groups, head size, widths that are no power of two, layers, vocabulary, theta, eps,
# tied or not, and (with it) the std of the weights and the page size they are run with.
TINY = {
    "A": dict(config=dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=64,
                          intermediate_size=176, num_attention_heads=4, num_key_value_heads=2, vocab_size=256,
                          max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-6,
                          tie_word_embeddings=True, hidden_act="silu", use_sliding_window=False),
              std=0.02, page_size=8, seed=11),
    "B": dict(config=dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=3, hidden_size=96,
                          intermediate_size=256, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
                          vocab_size=320, max_position_embeddings=256, rope_theta=1000000.0, rms_norm_eps=1e-5,
                          tie_word_embeddings=False),
              std=0.05, page_size=16, seed=23),
    # a third one with a head size above 64 that is no power of two, a width that is no
    # multiple of 16 products' K step, and a vocabulary that is no multiple of anything
    "C": dict(config=dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=120,
                          intermediate_size=200, num_attention_heads=6, num_key_value_heads=3, head_dim=80,
                          vocab_size=509, max_position_embeddings=512, rope_theta=50000.0, rms_norm_eps=1e-3,
                          tie_word_embeddings=False),
              std=0.04, page_size=32, seed=5),
    # head sizes 64 and 128, widths that are multiples of 64, a group of 7 query heads on one kv
    # head (q width != hidden width): the shapes the matrix-core kernels of the bfloat16 path take
    "D": dict(config=dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=192,
                          intermediate_size=320, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
                          vocab_size=300, max_position_embeddings=1024, rope_theta=10000.0, rms_norm_eps=1e-6,
                          tie_word_embeddings=True),
              std=0.05, page_size=64, seed=7),
    "E": dict(config=dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=256,
                          intermediate_size=384, num_attention_heads=7, num_key_value_heads=1, head_dim=128,
                          vocab_size=401, max_position_embeddings=2048, rope_theta=1000000.0, rms_norm_eps=1e-5,
                          tie_word_embeddings=False),
              std=0.05, page_size=8, seed=9),
}


def make_model_dir(path: str, name: str, storage: str = "float32") -> str:
    from axon_amd.config import config_from_dict
    from axon_amd.weights import write_random_model
    t = TINY[name]
    write_random_model(config_from_dict(t["config"]), path, seed=t["seed"], std=t["std"], storage=storage)
    return path


def prompts_for(name: str, lengths, seed: int = 0):
    g = torch.Generator().manual_seed(seed)
    v = TINY[name]["config"]["vocab_size"]
    return [torch.randint(0, v, (n,), generator=g).tolist() for n in lengths]


def tolerance(dtype: str, ref: torch.Tensor) -> float:
    """The allowed max |difference| of logits: float32 within rounding of a float64 oracle;
    bfloat16 (8 bits of mantissa in every stored activation) within 1 % of the range the logits
    span, three times what grading bfloat16 against float32 observes on these configurations
    (tests/test_invariance_gpu.py: at most 0.31 % of the range)."""
    if dtype == "float32":
        return 2e-5 * max(1.0, float(ref.abs().max()))
    return 1e-2 * max(float(ref.max() - ref.min()), 1e-3)


def engine_for(model_dir: str, dtype: str, page_size: int, num_pages: int, max_seqs: int = 4, **kw):
    from axon_amd.config import EngineConfig
    from axon_amd.engine import Engine, Runtime
    from axon_amd.engine.loading import load_model
    rt = Runtime(dtype)
    model = load_model(model_dir, rt)
    kw.setdefault("use_graphs", False)
    return Engine(model, rt, EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs, **kw))


# --------------------------------------------------------------------------- trace replay

def run_trace(model_dir: str, dtype: str, steps, out_dir: str, max_tokens: int, extra=()):
    """Drive bin/trace_run as a user would: steps on stdin, one at a time, each sent only after
    the `done` line of the one before.  Returns {step: float32 array [wanted, vocab]}."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out",
           out_dir, "--max-tokens", str(max_tokens), *extra]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for s in steps:
            p.stdin.write(json.dumps(s) + "\n")
            p.stdin.flush()
            line = p.stdout.readline().strip()
            assert line == f"done {s['step']}", f"trace_run answered {line!r} to step {s['step']}"
        p.stdin.close()
        assert p.wait(timeout=120) == 0
    finally:
        if p.poll() is None:
            p.kill()
    with open(os.path.join(model_dir, "config.json")) as f:
        vocab = json.load(f)["vocab_size"]
    out = {}
    for s in steps:
        path = os.path.join(out_dir, f"{s['step']}.f32")
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        if wanted:
            out[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not os.path.exists(path)
    return out


class TraceBuilder:
    """Builds the steps of a schedule and remembers which (request, position) each wanted row
    is, so the rows can be compared with a whole-sequence oracle."""

    def __init__(self):
        self.steps = []
        self.where = []       # per step: list of (request, position)
        self.fed = {}

    def step(self, entries, end=()):
        recs, where = [], []
        for rid, tokens, want in entries:
            start = self.fed.get(rid, 0)
            recs.append({"id": rid, "tokens": list(tokens), "want": list(want)})
            where += [(rid, start + w) for w in want]
            self.fed[rid] = start + len(tokens)
        for rid in end:
            self.fed.pop(rid, None)
        self.steps.append({"step": len(self.steps), "entries": recs, "end": list(end)})
        self.where.append(where)

    def collect(self, outputs):
        """{(request, position): logits row} from run_trace's result."""
        rows = {}
        for s, where in zip(self.steps, self.where):
            for i, key in enumerate(where):
                rows[key] = outputs[s["step"]][i]
        return rows
