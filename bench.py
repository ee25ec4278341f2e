"""The benchmark: decode tokens per second of a Qwen2.5-sized model (random weights, bfloat16) on
one MI355X, with the prefill throughput and the decode step's memory roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--sizes 7b|14b|32b] [--layers L] [--prompt N]
                    [--phase all|prefill|decode|mixed] [--no-points] [--profile]

A "step" is one decode step of the whole batch: every live request advances by one token
through the engine's own step function (HIP graph replay) and its device argmax.  Before the
timed steps every request's prompt is prefilled for real through the same step function.
One JSON line is printed.  More than one GPU is not supported: a line says so and the exit
code is 2.

Each size runs its own workload: 7b (the default) 2,048-token prompts and 256 generated tokens
at context 8,192; 14b 1,024-token prompts, 256 generated tokens and a mixed step of four prompt
portions of 512 tokens beside 32 decoding tokens; 32b 4,096-token prompts, 128 generated tokens,
context 16,384 and a cache pool sized from the memory that is free.  The prefill point is always
one prompt of 2,048 tokens.  Beside the headline batch the line carries decoding at batch 1 and
64, a prompt of 8,192 tokens, and generation through `LLM.generate` with a stop token set and
with sampling (the paths that read every token on the host before the next step).
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
# the further sizes of the same architecture (--sizes): layers, width, heads, feed-forward width, eps, context
SIZES = {"7b": SIZES_7B,
         "14b": dict(SIZES_7B, num_hidden_layers=48, hidden_size=5120, intermediate_size=13824, num_attention_heads=40,
                     num_key_value_heads=8, rms_norm_eps=1e-5),
         "32b": dict(SIZES_7B, num_hidden_layers=64, hidden_size=5120, intermediate_size=27648, num_attention_heads=40,
                     num_key_value_heads=8, rms_norm_eps=1e-5, max_position_embeddings=16384)}
# each size's own workload: prompt tokens of a decoding request, tokens it generates
WORKLOAD = {"7b": (2048, 256), "14b": (1024, 256), "32b": (4096, 128)}
PREFILL_TOKENS = 2048


def bandwidth(torch):
    """What reading memory costs here, measured with the engine's own streaming product (one row of X
    times a packed matrix: every byte of W is read once, 32 KB in flight a wave): a matrix of 1 GB
    (the sustained rate a decoding step can hope for), and matrices of the sizes of a step's smaller
    kernels read cold (right behind a read of 1 GB of other data, with no idle gap) and again right
    after themselves (what a launch of its own costs a kernel, and what the memory-side cache gives)."""
    from axon_amd.kernels import MODE_STORE_F32, kernels
    k = kernels("bfloat16")
    K = 4096
    x = torch.randn(1, K, device="cuda").bfloat16()

    def matrix(mb):
        n = mb * (1 << 20) // (2 * K)
        w = k.prepare_weight((torch.randn(n, K, device="cuda") * 0.05).bfloat16())
        y = torch.empty(1, n, dtype=torch.float32, device="cuda")
        return (lambda: k.gemm(x, w, y, None, MODE_STORE_F32)), n * K * 2

    def timed(fn):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3

    other, _ = matrix(1024)
    out = {"unit": "us and TB/s", "reads": {}}
    for mb in (16, 32, 64, 128, 256, 1024):
        run, nbytes = matrix(mb)
        run()
        cold, warm = [], []
        for _ in range(5):
            other()
            cold.append(timed(run))
            run()
            warm.append(timed(run))
        out["reads"][f"{mb} MB"] = {"cold_us": round(min(cold), 1), "cold_TBps": round(nbytes / min(cold) / 1e6, 2),
                                    "again_us": round(min(warm), 1), "again_TBps": round(nbytes / min(warm) / 1e6, 2)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed decode steps: every request generates this many tokens "
                    "(default: the size's own workload, 256 or 128)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has (0: all)")
    ap.add_argument("--prompt", type=int, default=0, help="prompt tokens of every decoding request (default: the size's own)")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--page-size", type=int, default=16, help="positions in a cache page (default: the 16 that the "
                    "measured configurations name; the engine's own default is 64, a block of its attention kernels)")
    ap.add_argument("--sizes", default="7b", choices=sorted(SIZES), help="layer sizes of Qwen2.5-7B (the default), 14B or 32B")
    ap.add_argument("--no-points", action="store_true", help="only the headline batch and the prefill point")
    ap.add_argument("--phase", default="all", choices=["all", "prefill", "decode", "mixed", "bandwidth"],
                    help="for profiling: time only the prefill step (repeated --steps times), only decoding, or only "
                         "the mixed step; bandwidth: no model, what reading memory once costs on this GPU (a long "
                         "read, and reads of the sizes of a decoding step's kernels, cold and right after themselves)")
    ap.add_argument("--profile", action="store_true", help="also launch one decode step kernel by kernel and print each "
                    "kernel's time and matrix bytes on stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU: this engine has no multi-GPU path (asked for {args.gpus})")
        return 2

    import torch

    import axon_amd
    from axon_amd.engine import StepEntry

    if args.phase == "bandwidth":
        print(json.dumps(bandwidth(torch)))
        return 0

    cfg = dict(SIZES[args.sizes])
    name = f"Qwen2.5-{args.sizes.upper()} sizes"
    prompt_len = args.prompt or WORKLOAD[args.sizes][0]
    steps = args.steps or WORKLOAD[args.sizes][1]
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    L, dim, ffn, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    ctx_len, page = cfg["max_position_embeddings"], args.page_size
    elem = 2 if args.dtype == "bfloat16" else 4
    points_on = not args.no_points and args.phase == "all"
    most_batch = max(args.batch, 64) if points_on else max(args.batch, 36 if args.phase == "mixed" else 1)
    per_request = prompt_len + steps + args.warmup + 17
    tokens_needed = max(most_batch * per_request, ctx_len + 64, 36 * (1024 + 64) + 4 * 1024)
    # the largest size takes its pool from the memory that is free (context 16,384 for up to 64 requests)
    num_pages = 0 if args.sizes == "32b" else -(-tokens_needed // page) + most_batch
    llm = axon_amd.load(cfg, dtype=args.dtype, random_seed=0, init_std=0.02, page_size=page, num_pages=num_pages,
                        max_seqs=most_batch, max_batch_tokens=max(prompt_len, 2048), max_seq_len=ctx_len)
    eng = llm.engine
    gen = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, V, (n,), generator=gen).tolist()

    def layer_flops(T, attended):
        return 2 * T * dim * ((nh + 2 * nkv) * hd + nh * hd + 3 * ffn) + 4 * nh * hd * attended

    # ---- prefill: one step of T tokens with the logits of the last one
    def prefill(T, reps):
        p = prompt(T)
        eng.step([StepEntry("warm", p, [T - 1])], end=["warm"])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):                                    # back to back: the average of full prefill steps
            eng.step([StepEntry("pf", p, [T - 1])], end=["pf"])
        torch.cuda.synchronize()
        s = (time.perf_counter() - t0) / reps
        flops = L * layer_flops(T, T * (T + 1) / 2) + 2 * dim * V
        return {"value": round(T / s, 1), "tokens": T, "ms": round(s * 1e3, 3),
                "frac": round(flops / s / PEAK_FLOPS[args.dtype], 4)}

    prefill_point = prefill(PREFILL_TOKENS, args.steps if args.phase == "prefill" and args.steps else 4)
    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill", "prefill": prefill_point, "prefill_8192": prefill(min(8192, ctx_len), 2),
                          "layers": L}))
        return 0

    # ---- decode at a batch size: prefill every request, then time K steps
    weight_bytes = (L * ((nh + 2 * nkv) * hd * dim + nh * hd * dim + 3 * ffn * dim) + V * dim) * elem

    def decode(batch: int, n_steps: int, warmup: int, profile: bool = False, eng=eng, prompt_len=prompt_len, portion=0):
        ids = [f"d{batch}_{prompt_len}_{i}" for i in range(batch)]
        last = []
        for rid in ids:
            pr = prompt(prompt_len)
            fed = pr[:-1]
            for a in range(0, len(fed), portion or len(fed)):          # long prompts in portions
                eng.step([StepEntry(rid, fed[a:a + (portion or len(fed))], [])])
            last.append(pr[-1])
        if profile:
            rows, total = eng.profile([StepEntry(rid, [t], [0]) for rid, t in zip(ids, last)])
            print(f"one decode step of {batch} rows, kernel by kernel ({total:.3f} ms; times include the wait for the "
                  f"event before each call):", file=sys.stderr)
            for r in sorted(rows, key=lambda r: -r["ms"]):
                rate = f"{r['bytes'] / r['ms'] / 1e9:7.2f} TB/s" if r["bytes"] else ""
                print(f"  {r['ms'] * 1e3 / r['launches']:9.1f} us x {r['launches']:4d} = {r['ms']:8.3f} ms  "
                      f"{r['bytes'] / 1e6:10.1f} MB {rate}  {r['name']}", file=sys.stderr)
            last = eng.last_picks.tolist()

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
        for _ in range(n_steps):
            pending = one(pending)
        pending.tolist()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mid_ctx = prompt_len + 1 + warmup + n_steps / 2
        for rid in ids:
            eng.release(rid)
        kv_bytes = batch * mid_ctx * L * 2 * nkv * hd * elem
        step_s = dt / n_steps
        return {"tok_s": batch * n_steps / dt, "ms": step_s * 1e3,
                "frac": (weight_bytes + kv_bytes) / step_s / HBM_BYTES_PER_S, "bytes": weight_bytes + kv_bytes}

    # ---- a mixed step: four prompt portions of 512 tokens beside 32 decoding tokens, as one batch
    def mixed(reps=3):
        dec = [f"m{i}" for i in range(32)]
        for rid in dec:
            eng.step([StepEntry(rid, prompt(1024), [])])
        times = []
        for r in range(reps + 1):
            entries = [StepEntry(rid, prompt(1), [0]) for rid in dec] + \
                      [StepEntry(f"p{r}_{j}", prompt(512), [511]) for j in range(4)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            eng.step(entries, end=[f"p{r}_{j}" for j in range(4)])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        for rid in dec:
            eng.release(rid)
        s = sum(times[1:]) / reps
        T = 32 + 4 * 512
        flops = L * (layer_flops(T, 32 * 1026 + 4 * 512 * 513 / 2)) + 2 * dim * V * 36
        return {"value": round(T / s, 1), "tokens": T, "ms": round(s * 1e3, 3),
                "frac": round(flops / s / PEAK_FLOPS[args.dtype], 4)}

    if args.phase == "mixed":
        print(json.dumps({"phase": "mixed", "mixed": mixed(max(args.steps, 3)), "layers": L}))
        return 0

    # ---- contexts of 32,768 positions: a second engine over the same weights (the measured
    # configuration names a context of 8,192; positions enter the arithmetic only through the
    # rotary angles), its pool sized for eight such requests.  A prompt of 32,768 tokens in portions
    # of 8,192, then decoding at batch 1 and 8 with every request that deep.
    def long_contexts(decode, first_engine, ctx=32768, portion=8192):
        nonlocal eng
        from axon_amd.config import EngineConfig
        from axon_amd.engine import Engine
        first_engine.release_all()
        llm.engine = eng = None
        del first_engine
        torch.cuda.empty_cache()
        room = ctx + 64 + 64
        long = Engine(llm.model, llm.rt, EngineConfig(dtype=args.dtype, page_size=page, num_pages=8 * -(-room // page) + 8,
                                                      max_seqs=8, max_batch_tokens=portion, max_seq_len=room))
        p = prompt(ctx)
        times = []
        for rep in range(2):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for a in range(0, ctx, portion):
                long.step([StepEntry("long", p[a:a + portion], [portion - 1] if a + portion >= ctx else [])],
                          end=["long"] if a + portion >= ctx else [])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        s = times[-1]
        flops = L * layer_flops(ctx, ctx * (ctx + 1) / 2) + 2 * dim * V
        out = {f"prefill_{ctx}_in_portions_of_{portion}": {"value": round(ctx / s, 1), "tokens": ctx, "ms": round(s * 1e3, 3),
                                                         "frac": round(flops / s / PEAK_FLOPS[args.dtype], 4)}}
        for b in (1, 8):
            r = decode(b, 32, 4, eng=long, prompt_len=ctx, portion=portion)
            out[f"decode_b{b}_ctx{ctx}"] = {"value": round(r["tok_s"], 1), "ms": round(r["ms"], 4), "frac": round(r["frac"], 4)}
        long.release_all()
        return out

    head = decode(args.batch, steps, args.warmup, profile=args.profile)
    cache_pages, graphs_on = eng.cache.plans[0].n_pages, bool(eng.graphs_ok)
    points, points_ms, points_frac, more = {}, {}, {}, {}
    if points_on:
        for b in (1, 64):
            r = head if b == args.batch else decode(b, max(8, steps // 2), args.warmup)
            points[f"decode_b{b}"] = round(r["tok_s"], 1)
            points_ms[f"decode_b{b}"] = round(r["ms"], 4)
            points_frac[f"decode_b{b}"] = round(r["frac"], 4)
        # a long prompt (attention grows with the square of it)
        more["prefill_8192"] = prefill(min(8192, ctx_len), 2)
        if args.sizes == "14b":
            more["mixed_step"] = mixed()
        # generation through the entry point: greedy, greedy with a stop token set (an id that
        # random weights hardly ever pick; both run a step ahead of the host), and sampled
        # tokens, which the host draws and so cannot run ahead
        ps = [prompt(prompt_len) for _ in range(args.batch)]
        n_new = min(steps, 64)
        llm.generate(ps, max_new_tokens=n_new)                        # the graphs of these steps are captured here
        llm.generate(ps, max_new_tokens=n_new, temperature=0.8, top_k=40, seed=1)
        for label, kw in (("greedy", {}), ("stop_token", dict(stop=[V - 1])),
                          ("sampled", dict(temperature=0.8, top_k=40, seed=1))):
            llm.generate(ps, max_new_tokens=n_new, **kw)
            st = llm.last_stats
            points[f"generate_b{args.batch}_{label}"] = round(st.decode_tokens / max(st.decode_seconds, 1e-9), 1)
            points_ms[f"generate_b{args.batch}_{label}"] = round(st.decode_seconds / max(st.decode_steps, 1) * 1e3, 4)
        # generation's clock waits for the device where the kind of step changes and at the end, so its
        # figures cannot beat the synchronised steps above by more than what a shorter context gives
        # (these requests generate fewer tokens than the headline's); if one does, say so
        beyond = {k: v for k, v in points.items() if k.startswith("generate_") and v > 1.02 * head["tok_s"]}
        if beyond:
            more["clock_check"] = f"generate points above 1.02 x the synchronised {head['tok_s']:.1f} tok/s: {beyond}"
            print(f"bench.py: {more['clock_check']}", file=sys.stderr)
        if args.sizes == "7b" and not args.layers:
            more.update(long_contexts(decode, eng))
    achieved = head["bytes"] / (head["ms"] / 1e3) / 1e9
    line = {
        "metric": f"decode tok/s ({name}, {args.dtype}, batch {args.batch}, {prompt_len}-token prompts)",
        "value": round(head["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: random N(0, 0.02) weights, uniform random token ids",
        "config": {"model": name, "layers": L, "layers_of_config": full_layers, "hidden": dim,
                   "heads": nh, "kv_heads": nkv, "head_dim": hd, "intermediate": ffn, "vocab": V, "batch": args.batch,
                   "global_batch": args.batch, "seq_len": prompt_len, "generated": steps, "context": ctx_len,
                   "page_size": page, "cache_pages": cache_pages, "parallelism": "single GPU",
                   "graphs": graphs_on, "batch_invariant": True},
        "prefill": prefill_point,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_BYTES_PER_S, 4)},
        "points": points, "points_ms": points_ms, "points_roofline": points_frac,
    }
    line.update(more)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
