"""The command line, in the manner of the reference's `axon` (src/cli.rs:35-68, 856-1248):

    axon gen MODEL "IDS" ["IDS" ...] [-n N] [--ctx N] [--dtype T] [sampling flags]   generate (greedy unless --temp > 0)
    axon logits MODEL "IDS" [-k K] [--all N]                             top-K next-token logits after the prompt
    axon info MODEL                                                      print a summary and exit
    axon random-weights CONFIG.json OUT [--seed S] [--std F]             write a model folder with random weights

MODEL is a folder with config.json and model.safetensors; with `--random-weights SEED` it is a
config.json (or a folder holding one) and the weights are drawn from the seed, nothing is read or
written.  `gen` takes any number of prompts and batches them; a line of ids is printed for each.

There is no tokenizer here: a prompt is a list of token ids ("5 17 3" or "5,17,3"), and what
`gen` prints is token ids.  Sampling flags have the reference's names, defaults and order
(src/sample.rs:101-190): --repeat-penalty (1.1), --repeat-last-n (64), --top-k (40), --top-p
(0.9), --min-p (0), --temp (gen: 0 = greedy), --seed.  A usage error prints one line and
`try 'axon --help'`, and exits with 2 (src/cli.rs:311-317).
"""
from __future__ import annotations

import argparse
import json
import math
import sys
from typing import List, Optional


class _Parser(argparse.ArgumentParser):
    def error(self, message):
        print(f"axon: {message}\ntry 'axon --help'", file=sys.stderr)
        raise SystemExit(2)


def _refuse(message: str) -> "NoReturn":
    print(f"axon: {message}\ntry 'axon --help'", file=sys.stderr)
    raise SystemExit(2)


def parse_ids(text: str) -> List[int]:
    parts = text.replace(",", " ").split()
    if not parts:
        _refuse("the prompt has no token ids")
    try:
        ids = [int(p) for p in parts]
    except ValueError:
        _refuse(f"the prompt must be token ids separated by spaces or commas, got '{text}'")
    if any(i < 0 for i in ids):
        _refuse("token ids cannot be negative")
    return ids


def _engine_flags(p: argparse.ArgumentParser) -> None:
    p.add_argument("--dtype", default="bfloat16", help="bfloat16 (default) or float32: true 32-bit everywhere")
    p.add_argument("--ctx", type=int, default=0, help="positions a request may reach (default: the model's)")
    p.add_argument("--page-size", type=int, default=64, help="positions in one cache page (default 64: a block of the attention kernels)")
    p.add_argument("--num-pages", type=int, default=0, help="pages in the cache pool (default: what the request needs)")
    p.add_argument("--device", default="cuda:0", help="the GPU to run on (default cuda:0)")
    p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                   help="MODEL is a config.json: run it with random weights drawn from this seed")
    p.add_argument("--std", type=float, default=0.02, help="with --random-weights: their standard deviation (default 0.02)")
    p.add_argument("--verbose", action="store_true", help="print what was loaded and the settings in use")


def _sampling_flags(p: argparse.ArgumentParser) -> None:
    g = p.add_argument_group("sampling flags (applied in this order)")
    g.add_argument("--repeat-penalty", type=float, default=None,
                   help="divide (multiply, if negative) the logits of tokens among the last N by P (default 1.1; 1 = off)")
    g.add_argument("--repeat-last-n", type=int, default=None,
                   help="how many tokens back the penalty looks, prompt included (default 64; 0 = off)")
    g.add_argument("--top-k", type=int, default=None, help="keep the K most likely tokens (default 40; 0 = off)")
    g.add_argument("--top-p", type=float, default=None,
                   help="then the fewest whose probability adds up to P (default 0.9; 1 = off)")
    g.add_argument("--min-p", type=float, default=None,
                   help="then those at least P times as likely as the top one (default 0 = off)")
    g.add_argument("--temp", type=float, default=None,
                   help="then divide the logits by T and draw (default 0 = greedy: the highest logit, no penalty, "
                        "no other flag applies)")
    g.add_argument("--seed", type=int, default=None, help="the random seed (default: a new one each run, printed)")


def build_parser() -> argparse.ArgumentParser:
    ap = _Parser(prog="axon", description="A small inference engine for AMD MI355X: token ids in, token ids out.")
    sub = ap.add_subparsers(dest="command")
    g = sub.add_parser("gen", help="generate (greedy unless --temp > 0)")
    g.add_argument("model")
    g.add_argument("prompt", nargs="+", help='token ids, e.g. "5 17 3"; several prompts are generated side by side')
    g.add_argument("-n", type=int, default=32, dest="n", help="tokens to generate (default 32)")
    g.add_argument("--stop", default="", help="token ids that end generation (not printed)")
    _engine_flags(g)
    _sampling_flags(g)
    l = sub.add_parser("logits", help="top-K next-token logits after the prompt")
    l.add_argument("model")
    l.add_argument("prompt")
    l.add_argument("-k", type=int, default=10, dest="k", help="how many to print (default 10)")
    l.add_argument("--all", type=int, default=0, dest="all_n", metavar="N", help="the last N positions, not just the last")
    l.add_argument("--digits", type=int, default=4, help="decimals printed (default 4)")
    _engine_flags(l)
    i = sub.add_parser("info", help="print a summary and exit")
    i.add_argument("model")
    r = sub.add_parser("random-weights", help="write a model folder (config.json, model.safetensors) with random weights")
    r.add_argument("config", help="a config.json of a supported architecture")
    r.add_argument("out", help="the folder to write")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02, help="standard deviation of matrices and biases (default 0.02)")
    r.add_argument("--storage", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    return ap


def _load(args, need_tokens: int, requests: int = 1):
    """`need_tokens`: the positions the longest request reaches; `requests`: how many run side by side."""
    import os

    import axon_amd
    from axon_amd.config import config_from_dict
    from axon_amd.engine.loading import read_model_config
    if args.random_weights is not None:
        path = os.path.join(args.model, "config.json") if os.path.isdir(args.model) else args.model
        with open(path) as f:
            cfg = config_from_dict(json.load(f))
    else:
        cfg = read_model_config(args.model)
    ctx = args.ctx or cfg.model_spec().max_positions
    if need_tokens > ctx:
        _refuse(f"the prompt and the tokens to generate need {need_tokens} positions, the context is {ctx}")
    pages = args.num_pages or requests * (-(-need_tokens // args.page_size) + 1)
    settings = dict(dtype=args.dtype, device=args.device, page_size=args.page_size, num_pages=pages,
                    max_seqs=max(2, requests), max_seq_len=ctx, max_batch_tokens=2048)
    if args.random_weights is not None:
        llm = axon_amd.load(cfg, random_seed=args.random_weights, init_std=args.std, **settings)
    else:
        llm = axon_amd.load(args.model, **settings)
    if args.verbose:
        print(f"model: {cfg.architecture}  {json.dumps(cfg.to_dict())}", file=sys.stderr)
        print(f"engine: dtype {llm.rt.dtype_name}, page {args.page_size}, pages {pages}, context {ctx}", file=sys.stderr)
    return llm, cfg


def run_gen(args) -> int:
    from axon_amd.sampling import SamplingParams, random_seed
    prompts = [parse_ids(p) for p in args.prompt]
    if args.n < 0:
        _refuse("-n needs a whole number")
    temp = args.temp if args.temp is not None else 0.0
    seed = args.seed
    try:
        params = SamplingParams(
            temperature=temp, top_k=40 if args.top_k is None else args.top_k,
            top_p=0.9 if args.top_p is None else args.top_p, min_p=0.0 if args.min_p is None else args.min_p,
            repeat_penalty=1.1 if args.repeat_penalty is None else args.repeat_penalty,
            repeat_last_n=64 if args.repeat_last_n is None else args.repeat_last_n, seed=seed)
    except ValueError as e:
        _refuse(str(e))
    if temp > 0 and seed is None:
        params.seed = random_seed()
        print(f"seed: {params.seed}", file=sys.stderr)
    llm, cfg = _load(args, max(len(ids) for ids in prompts) + args.n, len(prompts))
    vocab = llm.model.vocab_size
    if any(i >= vocab for ids in prompts for i in ids):
        _refuse(f"a token id is outside the vocabulary of {vocab}")
    stop = parse_ids(args.stop) if args.stop.strip() else []
    for out in llm.generate(prompts, max_new_tokens=args.n, stop=stop, sampling=params):
        print(" ".join(str(t) for t in out))
    st = llm.last_stats
    rate = lambda n, s: n / s if s > 0 else float("inf")
    fed = sum(len(ids) for ids in prompts)
    print(f"prompt eval: {fed} tok in {st.prompt_seconds:.3f} s ({rate(fed, st.prompt_seconds):.1f} tok/s)",
          file=sys.stderr)
    print(f"decode: {st.decode_tokens} tok, {st.decode_steps} passes in {st.decode_seconds:.3f} s "
          f"({rate(st.decode_tokens, st.decode_seconds):.1f} tok/s)", file=sys.stderr)
    return 0


def run_logits(args) -> int:
    import torch
    ids = parse_ids(args.prompt)
    llm, cfg = _load(args, len(ids))
    vocab = llm.model.vocab_size
    if any(i >= vocab for i in ids):
        _refuse(f"a token id is outside the vocabulary of {vocab}")
    print("prompt ids:", " ".join(str(i) for i in ids))
    n = min(max(args.all_n, 1), len(ids))
    rows = llm.logits(ids, all_positions=True)[len(ids) - n:].cpu() if n > 1 else llm.logits(ids).cpu()[None, :]
    k = min(args.k, vocab)
    for j, row in enumerate(rows):
        if n > 1:
            print(f"position {len(ids) - n + j}:")
        logprob = torch.log_softmax(row.double(), dim=-1)
        top = torch.topk(row, k)
        for v, i in zip(top.values.tolist(), top.indices.tolist()):
            print(f"  {i:>8}  logit {v:.{args.digits}f}  logprob {logprob[i].item():.{args.digits}f}")
    return 0


def run_info(args) -> int:
    from axon_amd.engine.loading import read_model_config
    from axon_amd.models import build_model_description
    cfg = read_model_config(args.model)
    model = build_model_description(cfg)
    n = sum(math.prod(t.shape) for t in {d.name: d for d in model.tensors() if not d.optional}.values())
    print(f"architecture: {cfg.architecture}")
    for key, value in cfg.to_dict().items():
        print(f"  {key}: {value}")
    print(f"parameters: {n:,}")
    plan = model.cache_plan
    for s, layers in zip(plan.group_specs, plan.group_layers):
        print(f"cache group: {layers} layers x {s.entries} x {s.heads} heads x {s.head_dim}"
              + (f", window {s.window}" if s.window else ""))
    return 0


def run_random_weights(args) -> int:
    from axon_amd.config import config_from_dict
    from axon_amd.weights import write_random_model
    with open(args.config) as f:
        cfg = config_from_dict(json.load(f))
    write_random_model(cfg, args.out, seed=args.seed, std=args.std, storage=args.storage)
    print(f"wrote {args.out}/config.json and {args.out}/model.safetensors")
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    from axon_amd.config import ConfigError
    from axon_amd.weights import SafetensorsError, WeightError
    ap = build_parser()
    args = ap.parse_args(argv)
    if not args.command:
        ap.print_help()
        return 0
    try:
        return {"gen": run_gen, "logits": run_logits, "info": run_info,
                "random-weights": run_random_weights}[args.command](args)
    except (ConfigError, WeightError, SafetensorsError, FileNotFoundError) as e:
        _refuse(str(e))


if __name__ == "__main__":
    sys.exit(main())
