"""Long contexts and a real vocabulary's width, through the engine and at kernel level: what the
tiny configurations never reach (the list of chunks of the decoding attention beyond a few
entries, the kernels a long prompt selects, the head's products from 16,384 rows of W on)."""
import math

import pytest
import torch

from axon_amd.config import config_from_dict
from axon_amd.engine import StepEntry
from axon_amd.kernels import kernels
from axon_amd.weights import write_random_model
from gpu_helpers import paged_cache, tol
from helpers import engine_for, tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

LONG = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=256, intermediate_size=320,
            num_attention_heads=6, num_key_value_heads=2, head_dim=128, vocab_size=300, max_position_embeddings=16384,
            rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
# a vocabulary wide enough that the head's products take the kernels of a real model's head
WIDE = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=256, intermediate_size=384,
            num_attention_heads=4, num_key_value_heads=2, head_dim=64, vocab_size=16411, max_position_embeddings=512,
            rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True)


@pytest.fixture(scope="module")
def long_dir(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("long"))
    write_random_model(config_from_dict(LONG), d, seed=31, std=0.1, storage="bfloat16")
    return d


@pytest.fixture(scope="module")
def wide_dir(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("wide"))
    write_random_model(config_from_dict(WIDE), d, seed=32, std=0.05, storage="bfloat16")
    return d


@pytest.mark.parametrize("dtype,page", [("float32", 64), ("bfloat16", 64), ("bfloat16", 16)])
def test_a_prompt_of_8192_tokens_in_one_step_then_decoding_across_a_chunks_edge(long_dir, dtype, page):
    """8,192 tokens in one step, then 40 tokens one by one (positions 8,192 .. 8,231: the 33rd
    chunk of 256 positions starts there), against the plain implementation; then the same tokens
    fed in portions of 3,000, which must give the same bits."""
    cfg, w = P.load_plain(long_dir)
    g = torch.Generator().manual_seed(5)
    toks = torch.randint(0, 300, (8232,), generator=g).tolist()
    ref = P.forward_logits(cfg, w, toks).float()
    eng = engine_for(long_dir, dtype, page_size=page, num_pages=2 * (8232 // page + 2), max_seqs=2, max_seq_len=16384,
                     use_graphs=True)
    got = [eng.step([StepEntry("a", toks[:8192], [0, 4095, 8191])]).cpu()]
    for t in range(8192, 8232):
        got.append(eng.step([StepEntry("a", [toks[t]], [0])]).cpu().clone())
    got = torch.cat(got)
    want = ref[[0, 4095] + list(range(8191, 8232))]
    assert (got - want).abs().max() <= tolerance(dtype, ref)
    # in portions, beside the first request: the same bits at the same positions
    again = []
    for a in range(0, 8192, 3000):
        b = min(a + 3000, 8192)
        out = eng.step([StepEntry("b", toks[a:b], [b - a - 1] if b == 8192 else [])])
        if out is not None:
            again.append(out.cpu().clone())
    for t in range(8192, 8232):
        again.append(eng.step([StepEntry("b", [toks[t]], [0])]).cpu().clone())
    assert torch.equal(torch.cat(again), got[2:])
    eng.release_all()
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_vocabulary_of_more_than_16384_whole_in_portions_and_decoded(wide_dir, dtype):
    """The head at 1 to 16 rows, at 17 to 64 and beyond takes three kernels; with 16,384 rows of W
    or more each takes two row tiles a wave.  Whole prompts, the last 20 tokens one by one and
    portions of 40 and 23 against the plain implementation, and bit for bit against each other."""
    cfg, w = P.load_plain(wide_dir)
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 16411, (n,), generator=g).tolist() for n in (100, 37)]
    eng = engine_for(wide_dir, dtype, page_size=16, num_pages=24, max_seqs=3, use_graphs=True)
    for i, p in enumerate(prompts):
        ref = P.forward_logits(cfg, w, p).float()
        whole = eng.step([StepEntry(("w", i), p, list(range(len(p))))], end=[("w", i)]).cpu()
        assert (whole - ref).abs().max() <= tolerance(dtype, ref)
        head = len(p) - 20
        rows = [eng.step([StepEntry(("d", i), p[:head], list(range(head)))]).cpu().clone()]
        for t in range(head, len(p)):
            rows.append(eng.step([StepEntry(("d", i), [p[t]], [0])]).cpu().clone())
        eng.release(("d", i))
        assert torch.equal(torch.cat(rows), whole)
        rows, at = [], 0
        for n in (40, 23, 40, 23):
            n = min(n, len(p) - at)
            if n:
                rows.append(eng.step([StepEntry(("p", i), p[at:at + n], list(range(n)))]).cpu().clone())
                at += n
        eng.release(("p", i))
        assert at == len(p) and torch.equal(torch.cat(rows), whole)
    # both prompts' last tokens as one decoding step of two rows
    a, b = prompts
    eng.step([StepEntry("a", a[:-1], []), StepEntry("b", b[:-1], [])])
    both = eng.step([StepEntry("a", a[-1:], [0]), StepEntry("b", b[-1:], [0])], end=["a", "b"]).cpu()
    for row, p in zip(both, prompts):
        ref = P.forward_logits(cfg, w, p).float()
        assert (row - ref[-1]).abs().max() <= tolerance(dtype, ref)


@pytest.mark.parametrize("hd,page", [(128, 64), (64, 16)])
def test_attention_finds_loud_keys_across_9000_positions(hd, page):
    """A context of 9,000 positions in which five keys are loud, each for one query head of the last
    token: at the start, at both sides of position 4,096 and at both sides of 8,192.  The decoding
    kernel (36 chunks) and the prompt kernel (a tile that ends the sequence) must put each head's
    weight on its key, and agree with the plain formula and with each other bit for bit."""
    k = kernels("bfloat16")
    far = [3, 4095, 4096, 8191, 8192]
    nh, nkv, T = len(far), 1, 9000
    g = torch.Generator().manual_seed(9)
    q = torch.randn(T, nh, hd, generator=g) * 0.1
    kk = torch.randn(T, nkv, hd, generator=g) * 0.1
    vv = torch.randn(T, nkv, hd, generator=g)
    for h, p in enumerate(far):
        kk[p, 0] = 0
        kk[p, 0, 2 * h] = 30.0
        q[T - 1, h] = 0
        q[T - 1, h, 2 * h] = 30.0
    qb, kb, vb = q.bfloat16(), kk.bfloat16(), vv.bfloat16()
    kc, vc, table = paged_cache(kb.double(), vb.double(), page, "bfloat16", seed=2)
    scale = 1.0 / math.sqrt(hd)
    ref = torch.stack([torch.softmax((kb[:, 0].double() @ qb[T - 1, h].double()) * scale, 0) @ vb[:, 0].double()
                       for h in range(nh)])
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    qd = qb.cuda().view(T, nh * hd)
    chunks = -(-T // k.attention_decode_chunk)
    partial = torch.empty(k.attention_decode_workspace(1, nh, hd, chunks), dtype=torch.float32, device="cuda")
    decoded = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_decode(qd, nh * hd, kc, vc, table, pos, rows, decoded, torch.tensor([T - 1], dtype=torch.int32).cuda(),
                       partial, chunks, nh, nkv, hd, page, 0, scale)
    prompt = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_prefill(qd, nh * hd, kc, vc, table, pos, rows, prompt, torch.tensor([[T - 100, 100]], dtype=torch.int32).cuda(),
                        nh, nkv, hd, page, 0, scale)
    got = decoded[T - 1].cpu().double().view(nh, hd)
    assert (got - ref).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)
    for h, p in enumerate(far):
        assert (got[h] - vb[p, 0].double()).abs().max() < 2e-2, (h, p)
    assert torch.equal(prompt[T - 1], decoded[T - 1])
