"""The benchmark: decode tokens per second of the Qwen2.5-7B-sized model (random weights,
bfloat16) on one MI355X, plus prefill throughput and the decode step's memory roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--prompt N] [--sizes 7b|14b|32b]

A "step" is one decode step of the whole batch: every live request advances by one token
through the engine's own step function (HIP graph replay) and its device argmax.  Before the
timed steps every request's prompt is prefilled for real through the same step function.
One JSON line is printed.  More than one GPU is not supported: a line says so and the exit
code is 2.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

SIZES_7B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=28, hidden_size=3584,
                intermediate_size=18944, num_attention_heads=28, num_key_value_heads=4, head_dim=128, vocab_size=152064,
                max_position_embeddings=8192, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
# the further sizes of the same architecture (--sizes): layers, width, heads, feed-forward width, eps
SIZES = {"7b": SIZES_7B,
         "14b": dict(SIZES_7B, num_hidden_layers=48, hidden_size=5120, intermediate_size=13824, num_attention_heads=40,
                     num_key_value_heads=8, rms_norm_eps=1e-5),
         "32b": dict(SIZES_7B, num_hidden_layers=64, hidden_size=5120, intermediate_size=27648, num_attention_heads=40,
                     num_key_value_heads=8, rms_norm_eps=1e-5)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="timed decode steps: every request generates this many tokens")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has (0: all)")
    ap.add_argument("--prompt", type=int, default=2048, help="prompt tokens of every request")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--sizes", default="7b", choices=sorted(SIZES), help="layer sizes of Qwen2.5-7B (the default), 14B or 32B")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--phase", default="all", choices=["all", "prefill", "decode"],
                    help="for profiling: time only the prefill step (repeated --steps times) or only decoding")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU: this engine has no multi-GPU path (asked for {args.gpus})")
        return 2

    import torch

    import axon_amd
    from axon_amd.engine import StepEntry

    cfg = dict(SIZES[args.sizes])
    name = f"Qwen2.5-{args.sizes.upper()} sizes"
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    L, dim, ffn, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    ctx_len, page = cfg["max_position_embeddings"], 16
    elem = 2 if args.dtype == "bfloat16" else 4
    most_batch = args.batch if args.no_points else max(args.batch, 64)
    tokens_needed = most_batch * (args.prompt + args.steps + args.warmup + 17)
    llm = axon_amd.load(cfg, dtype=args.dtype, random_seed=0, init_std=0.02, page_size=page,
                        num_pages=-(-tokens_needed // page) + most_batch, max_seqs=most_batch,
                        max_batch_tokens=max(args.prompt, 2048), max_seq_len=ctx_len)
    eng = llm.engine
    gen = torch.Generator().manual_seed(0)

    def prompt():
        return torch.randint(0, V, (args.prompt,), generator=gen).tolist()

    # ---- prefill: one step of `--prompt` tokens with the logits of the last one
    p = prompt()
    eng.step([StepEntry("warm", p, [len(p) - 1])], end=["warm"])
    torch.cuda.synchronize()
    reps = args.steps if args.phase == "prefill" else 4      # back to back: the average of full prefill steps
    t0 = time.perf_counter()
    for _ in range(reps):
        eng.step([StepEntry("pf", p, [len(p) - 1])], end=["pf"])
    torch.cuda.synchronize()
    prefill_s = (time.perf_counter() - t0) / reps
    T = len(p)
    per_layer = 2 * T * dim * ((nh + 2 * nkv) * hd + nh * hd + 3 * ffn) + 4 * nh * hd * T * (T + 1) / 2
    prefill_flops = L * per_layer + 2 * dim * V
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops / prefill_s / PEAK_FLOPS[args.dtype], 4)}

    # ---- decode at a batch size: prefill every request, then time K steps
    weight_bytes = (L * ((nh + 2 * nkv) * hd * dim + nh * hd * dim + 3 * ffn * dim) + V * dim) * elem

    def decode(batch: int, steps: int, warmup: int):
        ids = [f"d{batch}_{i}" for i in range(batch)]
        last = []
        for rid in ids:
            pr = prompt()
            eng.step([StepEntry(rid, pr[:-1], [])])
            last.append(pr[-1])

        # The first step takes its tokens from the host.  Every later step takes each request's
        # token from the pick the step before made for it, on the device, and the greedy picks
        # come back to the host one step behind, while the next step runs: as `generate` decodes.
        eng.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, last)])
        pending = eng.picks_async()

        def one(pending):
            eng.step_from_picks(ids)
            behind = eng.picks_async()
            pending.tolist()
            return behind

        for _ in range(warmup):
            pending = one(pending)
        pending.tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            pending = one(pending)
        pending.tolist()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mid_ctx = args.prompt + 1 + warmup + steps / 2
        for rid in ids:
            eng.release(rid)
        kv_bytes = batch * mid_ctx * L * 2 * nkv * hd * elem
        return batch * steps / dt, dt / steps, weight_bytes + kv_bytes

    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill", "prefill": prefill, "layers": L}))
        return 0
    tok_s, step_s, bytes_read = decode(args.batch, args.steps, args.warmup)
    points = {}
    if not args.no_points and args.phase == "all":
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(tok_s, 1)
            else:
                points[f"decode_b{b}"] = round(decode(b, max(8, args.steps // 2), args.warmup)[0], 1)
    achieved = bytes_read / step_s / 1e9
    line = {
        "metric": f"decode tok/s ({name}, {args.dtype}, batch {args.batch}, {args.prompt}-token prompts)",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: random N(0, 0.02) weights, uniform random token ids",
        "config": {"model": name, "layers": L, "layers_of_config": full_layers, "hidden": dim,
                   "heads": nh, "kv_heads": nkv, "head_dim": hd, "intermediate": ffn, "vocab": V, "batch": args.batch,
                   "global_batch": args.batch, "seq_len": args.prompt, "context": ctx_len, "page_size": page,
                   "parallelism": "single GPU", "graphs": bool(eng.graphs_ok)},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_BYTES_PER_S, 4)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
