"""What the reference's pool tests pin beyond logits (src/cuda/qwen2/slots.rs:1486-1570, 1629-1796):
the cache rows a request leaves are the same bits however its tokens were fed; a decoding step
replayed from a HIP graph gives the bits of the same step launched kernel by kernel; and the
reduced-precision path is graded against the 32-bit one by the measures of the reference's
oracle script (scripts/oracle/hf_logits.py: KL, top-1 agreement, max |difference|)."""
import pytest
import torch

from axon_amd.engine import StepEntry
from helpers import TINY, engine_for, prompts_for
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def cache_rows(eng, rid):
    """Keys and values of every position a live request has cached, layer by layer:
    [layers, 2, positions, kv heads, head_dim]."""
    req = eng.live[rid]
    group = eng.cache.group(0)
    page = group.page_size
    row = eng.cache.row(0, req.slot)
    layers = []
    for index in range(group.plan.n_layers):
        k, v = group.layer(index)                                   # [pages, heads, page, hd] each, as allocated
        v = v.view(v.shape[0], v.shape[1], v.shape[3], page)        # values are kept [heads, hd, page]
        ks = torch.stack([k[row[t // page], :, t % page, :] for t in range(req.n_cached)])
        vs = torch.stack([v[row[t // page], :, :, t % page] for t in range(req.n_cached)])
        layers.append(torch.stack([ks, vs]))
    return torch.stack(layers)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D", "E"])
def test_cache_rows_are_the_same_bits_however_the_tokens_were_fed(name, dtype, model_dirs):
    d = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    page = TINY[name]["page_size"]
    a, b, c = prompts_for(name, [150, 70, 33], seed=17)
    whole = engine_for(d, dtype, page, 64)
    whole.step([StepEntry("a", a, [])])
    want = cache_rows(whole, "a")
    if dtype == "bfloat16" and name == "B":
        assert want.dtype == torch.bfloat16
    # portions of changing size beside other requests' portions and single tokens, pages shuffled
    mixed = engine_for(d, dtype, page, 64, shuffle_pages_seed=5)
    mixed.step([StepEntry("b", b[:40], [])])
    mixed.step([StepEntry("a", a[:7], []), StepEntry("b", b[40:41], [0])])
    mixed.step([StepEntry("b", b[41:42], [0]), StepEntry("a", a[7:9], [1]), StepEntry("c", c, [])])
    mixed.step([StepEntry("a", a[9:100], []), StepEntry("b", b[42:43], [0])], end=["c"])
    for t in range(100, 118):                                       # single tokens, alone and in company
        mixed.step([StepEntry("a", a[t:t + 1], [0])] + ([StepEntry("b", b[t - 57:t - 56], [0])] if t % 2 else []))
    mixed.step([StepEntry("a", a[118:], [len(a) - 119])])
    got = cache_rows(mixed, "a")
    assert torch.equal(got, want)


@pytest.mark.parametrize("name", ["E"])
def test_a_norm_inside_the_product_after_it_changes_no_bit(name, model_dirs, monkeypatch):
    """Steps of up to sixteen tokens hand their norms to the product after them (the [q; k; v] product
    and the gated product norm their operand on the way; model E's width, a multiple of 256, is one
    that kernel takes): logits and cache rows are those of the same steps with every norm a pass of
    its own, and the kernel did run."""
    from axon_amd.parts.attention import GQAttention
    from axon_amd.parts.mlp import SwiGLUMLP
    d = model_dirs(name, "bfloat16")
    page = TINY[name]["page_size"]
    a, b = prompts_for(name, [90, 60], seed=29)

    def run(eng):
        out = [eng.step([StepEntry("a", a[:70], [69]), StepEntry("b", b[:30], [])])]
        out.append(eng.step([StepEntry("a", a[70:73], [0, 2]), StepEntry("b", b[30:35], [4])]))      # 8 tokens
        for t in range(73, 84):                                                                 # 1 or 2 tokens
            out.append(eng.step([StepEntry("a", a[t:t + 1], [0])] + ([StepEntry("b", b[t - 38:t - 37], [0])] if t % 3 else [])))
        out.append(eng.step([StepEntry("a", a[84:90], [5]), StepEntry("b", b[46:53], [0, 6])]))     # 13 tokens
        return torch.cat([o.clone() for o in out]), cache_rows(eng, "a")

    calls = []
    inside = engine_for(d, "bfloat16", page, 32)
    k = inside.rt.k
    glu, qkv = k.gemm_normed_glu, k.gemm_normed_qkv_rope
    monkeypatch.setattr(k, "gemm_normed_glu", lambda *a_, **kw: (calls.append("glu"), glu(*a_, **kw))[1])
    monkeypatch.setattr(k, "gemm_normed_qkv_rope", lambda *a_, **kw: (calls.append("qkv"), qkv(*a_, **kw))[1])
    got, got_rows = run(inside)
    assert calls.count("glu") >= 13 and calls.count("qkv") >= 13
    monkeypatch.setattr(GQAttention, "applies_preceding_norm", lambda self, ctx: False)
    monkeypatch.setattr(SwiGLUMLP, "applies_preceding_norm", lambda self, ctx: False)
    calls.clear()
    apart = engine_for(d, "bfloat16", page, 32)
    want, want_rows = run(apart)
    assert not calls
    assert torch.equal(got, want) and torch.equal(got_rows, want_rows)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_a_replayed_graph_gives_the_bits_of_the_step_launched_kernel_by_kernel(name, dtype, model_dirs):
    """The same decoding schedule on two engines, graphs on and off: contexts that cross a chunk
    of the decoding attention (255 -> 257, 510 -> 514 positions) and page edges, a request that
    ends in the middle (the batch shrinks), one that joins late into a slot given back, and
    replays of one graph with the program's own eager steps between them."""
    d = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    page = TINY[name]["page_size"]
    prompts = dict(zip("abcd", prompts_for(name, [250, 505, 40, 61], seed=19)))
    stream = torch.randint(0, TINY[name]["config"]["vocab_size"], (64, 4), generator=torch.Generator().manual_seed(3))
    results = []
    for graphs in (True, False):
        eng = engine_for(d, dtype, page, 4 * (640 // page), max_seqs=3, use_graphs=graphs)
        out = []
        for rid in "abc":
            eng.step([StepEntry(rid, prompts[rid][:-1], [])])
        live = ["a", "b", "c"]
        for t in range(24):
            if t == 9:
                eng.release("c")                                    # ends in the middle: two rows a step from here
                live = ["a", "b"]
            if t == 14:                                             # joins late, into the slot given back
                out.append(eng.step([StepEntry("d", prompts["d"], [len(prompts["d"]) - 1])]).clone())
                live = ["a", "b", "d"]
            entries = [StepEntry(rid, [int(stream[t, "abcd".index(rid)])], [0]) for rid in live]
            out.append(eng.step(entries).clone())
        if graphs:
            assert eng.graphs_ok and len(eng._graphs) >= 3          # several shapes were captured and replayed
        results.append(out)
        eng.release_all()
    for with_graph, without in zip(*results):
        assert torch.equal(with_graph, without)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_a_decoding_row_has_the_same_bits_among_two_hundred_rows_as_among_few(name, dtype, model_dirs):
    """Two hundred requests decode a token each: all in one step, in steps of 100, 70 and 30, and in
    steps of 17, 1, 64, 65 and 53 rows, so that every product takes each of its kernels (up to 16
    rows, up to 64, up to 128, more).  A request's logits and cache rows are the same bits."""
    d = model_dirs(name, "float32" if dtype == "float32" else "bfloat16")
    page = TINY[name]["page_size"]
    n = 200
    lengths = [3 + (7 * i) % 23 for i in range(n)]
    prompts = prompts_for(name, lengths, seed=5)
    pages = sum(-(-(length + 1) // page) for length in lengths) + 8

    def decode(groups):
        eng = engine_for(d, dtype, page, pages, max_seqs=n, max_batch_tokens=4096)
        for first in range(0, n, 50):                               # the prompts, fifty requests a step
            eng.step([StepEntry(f"r{i}", prompts[i][:-1], []) for i in range(first, first + 50)])
        rows, at = {}, 0
        for size in groups:
            ids = list(range(at, at + size))
            logits = eng.step([StepEntry(f"r{i}", prompts[i][-1:], [0]) for i in ids])
            for j, i in enumerate(ids):
                rows[i] = logits[j].clone()
            at += size
        assert at == n
        return rows, [cache_rows(eng, f"r{i}") for i in (0, 16, 17, 99, 100, 199)]

    whole, whole_cache = decode([n])
    for groups in ([100, 70, 30], [17, 1, 64, 65, 53]):
        got, got_cache = decode(groups)
        for i in range(n):
            assert torch.equal(got[i], whole[i]), f"request {i} in steps of {groups}"
        for a, b in zip(got_cache, whole_cache):
            assert torch.equal(a, b)


def grade(ref: torch.Tensor, got: torch.Tensor):
    """max |difference| relative to the logits' range, top-1 agreement, mean KL(ref || got)."""
    ref, got = ref.double(), got.double()
    span = float(ref.max() - ref.min())
    kl = (torch.softmax(ref, -1) * (torch.log_softmax(ref, -1) - torch.log_softmax(got, -1))).sum(-1)
    top2 = torch.topk(ref, 2, dim=-1).values
    return dict(max_diff=float((ref - got).abs().max()) / span, top1=float((ref.argmax(-1) == got.argmax(-1)).double().mean()),
                kl=float(kl.mean()), clear=(top2[:, 0] - top2[:, 1]) > 0.02 * span)


@pytest.mark.parametrize("name", ["A", "B", "D", "E"])
def test_bfloat16_is_graded_against_float32(name, model_dirs, capsys):
    """The same bfloat16 weights through both precisions of the engine, every position of four
    prompts: bfloat16 is held to a KL below 5e-5 nats, to 0.6 % of the logits' range, and to the same
    best token wherever the 32-bit logits have a clear winner."""
    d = model_dirs(name, "bfloat16")
    page = TINY[name]["page_size"]
    prompts = prompts_for(name, [100, 64, 33, 9], seed=23)
    rows = {}
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(d, dtype, page, 64)
        rows[dtype] = torch.cat([eng.step([StepEntry(i, p, list(range(len(p))))], end=[i]).cpu()
                                 for i, p in enumerate(prompts)])
    g = grade(rows["float32"], rows["bfloat16"])
    with capsys.disabled():
        print(f"\n[{name}] bfloat16 vs float32: max |diff| {g['max_diff']:.4f} of the range, top-1 {g['top1']:.3f}, "
              f"KL {g['kl']:.2e} nats, {int(g['clear'].sum())} of {len(g['clear'])} rows with a clear winner")
    assert g["kl"] < 5e-5 and g["max_diff"] < 6e-3
    clear = g["clear"]
    assert bool((rows["float32"][clear].argmax(-1) == rows["bfloat16"][clear].argmax(-1)).all())
    # and the 32-bit engine sits on the plain implementation
    cfg, w = P.load_plain(d)
    ref = torch.cat([P.forward_logits(cfg, w, p) for p in prompts])
    assert grade(ref, rows["float32"])["kl"] < 1e-9
