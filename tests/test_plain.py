"""Pins the plain implementation (tests/plain/qwen2_plain.py) by what fixes it beside the
reference's text: vectors the reference's own tests hold, special cases that reduce to a
library routine, and invariants, each chosen so that a plausible misreading fails it; and
mutation checks: a deliberately wrong variant must move the logits far beyond any tolerance
the engine is compared with (the reference's NormBug / RopeBug idea, src/model.rs:4518-4555).
"""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import tolerance
from plain import qwen2_plain as P

torch.manual_seed(0)


# --------------------------------------------------------------------------- RMSNorm

def test_rmsnorm_is_the_library_formula_and_its_invariants():
    x = torch.randn(5, 48, dtype=torch.float64) * 3
    g = torch.rand(48, dtype=torch.float64) + 0.5
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * g
    assert torch.allclose(P.rms_norm(x, g, 1e-5), want, rtol=1e-13, atol=0)
    one = torch.ones(48, dtype=torch.float64)
    out = P.rms_norm(x, one, 0.0)
    assert torch.allclose((out * out).mean(-1), torch.ones(5, dtype=torch.float64))      # unit RMS
    assert torch.allclose(P.rms_norm(7.5 * x, g, 0.0), P.rms_norm(x, g, 0.0))            # scale-free at eps 0
    c = torch.full((1, 48), 3.0, dtype=torch.float64)                                     # constant vector
    assert torch.allclose(P.rms_norm(c, g, 0.5), g * 3.0 / math.sqrt(9.0 + 0.5))
    # eps sits inside the root, added to the MEAN of squares (not the sum, not outside)
    assert not torch.allclose(P.rms_norm(x, g, 0.5), x / (torch.sqrt((x * x).mean(-1, keepdim=True)) + 0.5) * g)


# --------------------------------------------------------------------------- projections

def test_linear_layout_and_bias_placement():
    w = torch.randn(7, 5, dtype=torch.float64)
    b = torch.randn(7, dtype=torch.float64)
    for j in range(5):
        e = torch.zeros(1, 5, dtype=torch.float64)
        e[0, j] = 1.0
        assert torch.equal(P.linear(e, w, b)[0], w[:, j] + b)       # [out, in]: column j, then the bias
    x = torch.randn(3, 5, dtype=torch.float64)
    assert torch.allclose(P.linear(x, w, b), F.linear(x, w, b))


# --------------------------------------------------------------------------- RoPE

def test_rope_frequencies_and_golden_values():
    f = P.rope_freqs(128, 1e6)
    want = torch.tensor([1e6 ** (-2.0 * i / 128.0) for i in range(64)], dtype=torch.float64)  # src/rope.rs:394-396
    assert torch.allclose(f, want, rtol=1e-14, atol=0)
    assert f[0] == 1.0 and abs(f[32].item() - 1e-3) < 1e-15
    assert not torch.allclose(P.rope_freqs(32, 1e4), P.rope_freqs(32, 1e6))   # theta tells A from B


def test_rope_identity_norm_pairing_and_relative_property():
    hd = 16
    freqs = P.rope_freqs(hd, 10000.0)
    v = torch.randn(6, 2, hd, dtype=torch.float64)
    sin0, cos0 = P.rope_table(torch.zeros(6, dtype=torch.long), freqs)
    assert torch.equal(P.apply_rope(v, sin0, cos0), v)                         # position 0 is the identity
    pos = torch.tensor([0, 1, 2, 5, 40, 1000])
    sin, cos = P.rope_table(pos, freqs)
    r = P.apply_rope(v, sin, cos)
    half = hd // 2
    n_before = v[..., :half] ** 2 + v[..., half:] ** 2                         # each (i, i + half) pair keeps its norm
    n_after = r[..., :half] ** 2 + r[..., half:] ** 2
    assert torch.allclose(n_before, n_after)
    wrong_pairs = v.view(6, 2, half, 2).pow(2).sum(-1)                         # (2i, 2i+1) pairs do not
    assert not torch.allclose(wrong_pairs, r.view(6, 2, half, 2).pow(2).sum(-1))
    # pair 0 turns by `pos` radians exactly, counter-clockwise: (1, 0) -> (cos p, sin p)
    e = torch.zeros(1, 1, hd, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    s3, c3 = P.rope_table(torch.tensor([3]), freqs)
    out = P.apply_rope(e, s3, c3)
    assert abs(out[0, 0, 0].item() - math.cos(3.0)) < 1e-15 and abs(out[0, 0, half].item() - math.sin(3.0)) < 1e-15
    # scores depend on the distance only
    q, k = torch.randn(1, 1, hd, dtype=torch.float64), torch.randn(1, 1, hd, dtype=torch.float64)

    def score(p, t):
        sq, cq = P.rope_table(torch.tensor([p]), freqs)
        sk, ck = P.rope_table(torch.tensor([t]), freqs)
        return (P.apply_rope(q, sq, cq) * P.apply_rope(k, sk, ck)).sum().item()

    assert abs(score(9, 4) - score(105, 100)) < 1e-12
    assert abs(score(9, 4) - score(10, 4)) > 1e-6


# --------------------------------------------------------------------------- attention

def library_attention(q, k, v, window=0):
    T, nh, hd = q.shape
    group = nh // k.shape[1]
    kk = k.repeat_interleave(group, dim=1)      # heads kvh*group .. kvh*group+group-1 share kv head kvh
    vv = v.repeat_interleave(group, dim=1)
    s = torch.einsum("thd,shd->hts", q, kk) / math.sqrt(hd)
    i = torch.arange(T)
    mask = i[None, :] > i[:, None]
    if window > 0:
        mask = mask | (i[None, :] < i[:, None] + 1 - window)
    s = s.masked_fill(mask[None], float("-inf"))
    return torch.einsum("hts,shd->thd", torch.softmax(s, dim=-1), vv)


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 32, 0), (6, 3, 8, 0), (4, 4, 16, 0), (4, 2, 16, 5)])
def test_attention_is_the_library_routine(nh, nkv, hd, window):
    q = torch.randn(19, nh, hd, dtype=torch.float64)
    k = torch.randn(19, nkv, hd, dtype=torch.float64)
    v = torch.randn(19, nkv, hd, dtype=torch.float64)
    assert torch.allclose(P.causal_attention(q, k, v, window), library_attention(q, k, v, window), atol=1e-12)


def test_attention_special_cases():
    nh, nkv, hd = 6, 3, 8
    q = torch.randn(1, nh, hd, dtype=torch.float64)
    k = torch.randn(1, nkv, hd, dtype=torch.float64)
    v = torch.randn(1, nkv, hd, dtype=torch.float64)
    out = P.causal_attention(q, k, v)
    for qh in range(nh):                                   # one position: the mapped kv head's v, exactly
        assert torch.equal(out[0, qh], v[0, qh // 2])
    assert not torch.equal(out[0, 1], v[0, 1 % nkv])       # ... not qh % nkv
    # uniform scores (q = 0): the mean of the values seen so far
    T = 7
    q0 = torch.zeros(T, nh, hd, dtype=torch.float64)
    k = torch.randn(T, nkv, hd, dtype=torch.float64)
    v = torch.randn(T, nkv, hd, dtype=torch.float64)
    out = P.causal_attention(q0, k, v)
    for t in range(T):
        assert torch.allclose(out[t, 0], v[:t + 1, 0].mean(0))
    # causality: later tokens change nothing earlier
    q = torch.randn(T, nh, hd, dtype=torch.float64)
    a = P.causal_attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[5:] += 1.0
    v2[5:] -= 2.0
    assert torch.equal(a[:5], P.causal_attention(q, k2, v2)[:5])
    # one head, no rotation, no mask at the last row: softmax(q K^T / sqrt(hd)) V
    s = torch.softmax(k[:, 0] @ q[T - 1, 0] / math.sqrt(hd), -1)
    assert torch.allclose(a[T - 1, 0], s @ v[:, 0])


# --------------------------------------------------------------------------- SwiGLU

def test_swiglu_vectors_and_library():
    f32 = torch.float32
    out = P.swiglu(torch.tensor([-200.0], dtype=f32), torch.tensor([1.0], dtype=f32))     # src/vmath.rs:495-497
    assert out.item() == 0.0 and math.copysign(1.0, out.item()) == -1.0
    assert P.swiglu(torch.tensor([200.0], dtype=f32), torch.tensor([1.0], dtype=f32)).item() == 200.0
    assert P.swiglu(torch.tensor([0.0]), torch.tensor([5.0])).item() == 0.0
    g, u = torch.randn(50, dtype=torch.float64) * 4, torch.randn(50, dtype=torch.float64)
    assert torch.allclose(P.swiglu(g, u), F.silu(g) * u, atol=1e-14)
    assert not torch.allclose(P.swiglu(g, u), F.silu(u) * g)                               # gate is the first argument


# --------------------------------------------------------------------------- whole model

def random_weights(cfg: P.PlainConfig, ffn: int, vocab: int, std: float):
    g = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * std
    gain = lambda n: 1.0 + torch.randn(n, generator=g, dtype=torch.float64) * 0.3
    d, q, kv = cfg.hidden_size, cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    w = {"model.embed_tokens.weight": r(vocab, d), "model.norm.weight": gain(d)}
    if not cfg.tie_word_embeddings:
        w["lm_head.weight"] = r(vocab, d)
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        w.update({p + "input_layernorm.weight": gain(d), p + "post_attention_layernorm.weight": gain(d),
                  p + "self_attn.q_proj.weight": r(q, d), p + "self_attn.q_proj.bias": r(q) * 20,
                  p + "self_attn.k_proj.weight": r(kv, d), p + "self_attn.k_proj.bias": r(kv) * 20,
                  p + "self_attn.v_proj.weight": r(kv, d), p + "self_attn.v_proj.bias": r(kv) * 20,
                  p + "self_attn.o_proj.weight": r(d, q), p + "mlp.gate_proj.weight": r(ffn, d),
                  p + "mlp.up_proj.weight": r(ffn, d), p + "mlp.down_proj.weight": r(d, ffn)})
    return w


def _setup():
    cfg = P.PlainConfig(num_hidden_layers=2, hidden_size=48, num_attention_heads=6, num_key_value_heads=3, head_dim=8,
                        rope_theta=100.0, rms_norm_eps=0.5, tie_word_embeddings=False)
    w = random_weights(cfg, 80, 97, 0.3)
    tokens = torch.randint(0, 97, (23,), generator=torch.Generator().manual_seed(1)).tolist()
    return cfg, w, tokens


def test_forward_properties():
    cfg, w, tokens = _setup()
    full = P.forward_logits(cfg, w, tokens)
    assert full.shape == (23, 97)
    # causality of the whole model: a prefix gives the same logits
    assert torch.allclose(P.forward_logits(cfg, w, tokens[:9]), full[:9], atol=1e-12)
    # positions shifted as a whole change nothing: only distances count
    shifted = P.logits_of(cfg, w, P.hidden_states(cfg, w, tokens, start=37))
    assert torch.allclose(shifted, full, atol=1e-9)
    # tied or not decides the head
    import dataclasses
    tied = dataclasses.replace(cfg, tie_word_embeddings=True)
    h = P.rms_norm(P.hidden_states(cfg, w, tokens), w["model.norm.weight"], cfg.rms_norm_eps)
    assert torch.allclose(P.forward_logits(tied, w, tokens), h @ w["model.embed_tokens.weight"].T)
    assert torch.allclose(full, h @ w["lm_head.weight"].T)


MUTATIONS = {
    "rope pairs (2i, 2i+1)": ("apply_rope", lambda v, sin, cos: torch.stack(
        [v[..., 0::2] * cos[:, None, :] - v[..., 1::2] * sin[:, None, :],
         v[..., 0::2] * sin[:, None, :] + v[..., 1::2] * cos[:, None, :]], dim=-1).flatten(-2)),
    "rope sign flipped": ("apply_rope", lambda v, sin, cos: torch.cat(
        [v[..., :v.shape[-1] // 2] * cos[:, None, :] + v[..., v.shape[-1] // 2:] * sin[:, None, :],
         -v[..., :v.shape[-1] // 2] * sin[:, None, :] + v[..., v.shape[-1] // 2:] * cos[:, None, :]], dim=-1)),
    "norm: gain before scaling by eps outside the root": ("rms_norm", lambda x, g, eps: x * g / (
        torch.sqrt((x * x).mean(-1, keepdim=True)) + eps)),
    "norm: mean forgotten": ("rms_norm", lambda x, g, eps: x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps) * g),
    "bias dropped": ("linear", lambda x, w, b=None: x @ w.T),
    "swiglu halves swapped": ("swiglu", lambda g, u: u / (1 + torch.exp(-u)) * g),
}


@pytest.mark.parametrize("name", list(MUTATIONS))
def test_wrong_variants_move_the_logits(name, monkeypatch):
    cfg, w, tokens = _setup()
    good = P.forward_logits(cfg, w, tokens)
    fn, bad = MUTATIONS[name]
    monkeypatch.setattr(P, fn, bad)
    moved = (P.forward_logits(cfg, w, tokens) - good).abs().max().item()
    assert moved > 100 * tolerance("float32", good) and moved > 2 * tolerance("bfloat16", good), (name, moved)


def test_wrong_attention_variants_move_the_logits(monkeypatch):
    cfg, w, tokens = _setup()
    good = P.forward_logits(cfg, w, tokens)
    real = P.causal_attention

    def scale_by_hd(q, k, v, window=0):          # 1 / hd instead of 1 / sqrt(hd)
        return real(q / math.sqrt(q.shape[-1]), k, v, window)

    def kv_modulo(q, k, v, window=0):            # kv head qh % nkv instead of qh // group
        nh, nkv = q.shape[1], k.shape[1]
        order = [(qh % nkv) for qh in range(nh)]
        return real(q, k[:, order], v[:, order], window) if nh == nkv else \
            torch.stack([real(q[:, qh:qh + 1], k[:, order[qh]:order[qh] + 1], v[:, order[qh]:order[qh] + 1])[:, 0]
                         for qh in range(nh)], dim=1)

    def sees_the_future(q, k, v, window=0):      # no causal bound
        T = q.shape[0]
        return torch.stack([real(q[t:t + 1].expand(T, -1, -1), k, v)[T - 1] for t in range(T)])

    for name, bad in [("scale", scale_by_hd), ("kv mapping", kv_modulo), ("no causality", sees_the_future)]:
        monkeypatch.setattr(P, "causal_attention", bad)
        moved = (P.forward_logits(cfg, w, tokens) - good).abs().max().item()
        assert moved > 100 * tolerance("float32", good), (name, moved)


# --------------------------------------------------------------------------- the arrangement of a layer

def _uniform_attention_weights():
    """The whole-model fixture with q and k projections and their biases zeroed: every score is 0,
    so attention is the running mean of the values over positions 0..t, which library routines
    give (cumsum), whatever the rotation does to the zero vectors."""
    cfg, w, tokens = _setup()
    w = dict(w)
    for l in range(cfg.num_hidden_layers):
        for n in ("q_proj.weight", "q_proj.bias", "k_proj.weight", "k_proj.bias"):
            w[f"model.layers.{l}.self_attn.{n}"] = torch.zeros_like(w[f"model.layers.{l}.self_attn.{n}"])
    return cfg, w, tokens


def _by_library_routines(cfg, w, tokens, order="reference"):
    """The whole model as straight-line calls of torch's own routines (F.embedding, F.rms_norm,
    F.linear, F.silu, cumsum), valid when every attention score is 0.  `order` names the
    arrangement: the reference's (src/model.rs:2967-3059: x += attention(norm1 x); x +=
    feed_forward(norm2 x), norm2 reading the sum; final norm, then the head) or a wrong one."""
    d = cfg.hidden_size
    group = cfg.num_attention_heads // cfg.num_key_value_heads
    T = len(tokens)
    x = F.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    steps = torch.arange(1, T + 1, dtype=torch.float64)[:, None]

    def attention(h, p):
        v = F.linear(h, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])
        mean = torch.cumsum(v, dim=0) / steps                                  # uniform weights over 0..t
        heads = mean.view(T, cfg.num_key_value_heads, cfg.head_dim).repeat_interleave(group, dim=1)
        return F.linear(heads.reshape(T, -1), w[p + "self_attn.o_proj.weight"])

    def feed_forward(h, p):
        return F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                        w[p + "mlp.down_proj.weight"])

    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        n1 = lambda t: F.rms_norm(t, (d,), w[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        n2 = lambda t: F.rms_norm(t, (d,), w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        if order == "reference":
            x = x + attention(n1(x), p)
            x = x + feed_forward(n2(x), p)
        elif order == "parallel":                      # both parts read the same stream
            x = x + attention(n1(x), p) + feed_forward(n2(x), p)
        elif order == "no residual after attention":
            x = attention(n1(x), p)
            x = x + feed_forward(n2(x), p)
        elif order == "no residual after the feed-forward":
            x = x + attention(n1(x), p)
            x = feed_forward(n2(x), p)
        elif order == "norms after the parts":        # post-norm
            x = n1(x + attention(x, p))
            x = n2(x + feed_forward(x, p))
        elif order == "norms swapped":
            x = x + attention(n2(x), p)
            x = x + feed_forward(n1(x), p)
    if order != "no final norm":
        x = F.rms_norm(x, (d,), w["model.norm.weight"], cfg.rms_norm_eps)
    return F.linear(x, w["lm_head.weight"])


def test_the_arrangement_of_a_layer_reduces_to_library_routines():
    """What no part's own test pins: the order of norm, attention, sum, norm, feed-forward, sum
    and the final norm before the head.  With uniform attention the whole model is a few lines of
    library calls; the plain implementation equals them in the reference's order and in no other."""
    cfg, w, tokens = _uniform_attention_weights()
    got = P.forward_logits(cfg, w, tokens)
    want = _by_library_routines(cfg, w, tokens)
    assert (got - want).abs().max() <= 1e-10 * want.abs().max()
    for wrong in ("parallel", "no residual after attention", "no residual after the feed-forward",
                  "norms after the parts", "norms swapped", "no final norm"):
        off = (_by_library_routines(cfg, w, tokens, wrong) - got).abs().max().item()
        assert off > 100 * tolerance("float32", got) and off > 2 * tolerance("bfloat16", got), (wrong, off)
    # with both output projections zero the residual stream carries the embedding through, unscaled
    for l in range(cfg.num_hidden_layers):
        for n in ("self_attn.o_proj.weight", "mlp.down_proj.weight"):
            w[f"model.layers.{l}.{n}"] = torch.zeros_like(w[f"model.layers.{l}.{n}"])
    bare = F.linear(F.rms_norm(F.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"]), (cfg.hidden_size,),
                               w["model.norm.weight"], cfg.rms_norm_eps), w["lm_head.weight"])
    assert (P.forward_logits(cfg, w, tokens) - bare).abs().max() <= 1e-12 * bare.abs().max()


# --------------------------------------------------------------------------- picking

def test_argmax_rules():
    inf, nan = float("inf"), float("nan")
    assert P.argmax_last([-inf] * 5) == 4                       # src/generate.rs:292
    assert P.argmax_last([1.0, 3.0, 3.0, 2.0]) == 2             # ties: the last
    assert P.argmax_last([nan, 1.0, nan]) == 1                  # NaN never
    assert P.argmax_last([nan, nan, nan]) == 2                  # all NaN: the last index
    assert P.argmax_last([-1.0, 0.0, -0.0]) == 2                # -0.0 ties +0.0
    assert P.argmax_last([0.0, -0.0, -1.0]) == 1


def test_rng_vectors():
    # splitmix64 from state 0 and xoshiro256** from state (1, 2, 3, 4): published sequences
    s, z = P.splitmix64(0)
    assert z == 0xE220A8397B1DCDAF
    s, z = P.splitmix64(s)
    assert z == 0x6E789E6AA1B965F4
    r = P.PlainRng(0)
    r.s = [1, 2, 3, 4]
    assert [r.next_u64() for _ in range(4)] == [11520, 0, 1509978240, 1215971899390074240]
    r = P.PlainRng(42)
    xs = [r.f64() for _ in range(1000)]
    assert all(0.0 <= x < 1.0 for x in xs) and 0.4 < sum(xs) / 1000 < 0.6
    assert [P.PlainRng(7).next_u64() for _ in range(2)] == [P.PlainRng(7).next_u64() for _ in range(2)]


def test_repeat_penalty_vectors():
    # src/sample.rs:1020-1060
    l = [4.0, -1.0, 0.0, 3.0, 1.0, 2.0]
    recent = [3, 5, 1, 1, 2, 1]
    out = P.penalize(l, recent, 4, 2.0)
    assert out == [4.0, -2.0, 0.0, 3.0, 1.0, 2.0]
    assert [i for _, i in P.candidates(out, 6)] == [0, 3, 5, 4, 2, 1]
    assert P.penalize(l, recent, 4, 1.0) == l and P.penalize(l, recent, 0, 2.0) == l
    assert P.penalize([4.0, 1.0, 0.0, 3.0, 1.0, 2.0], [1, 0], 64, 0.5) == [8.0, 2.0, 0.0, 3.0, 1.0, 2.0]
    l4 = P.penalize([3.0, 2.8], [0], 64, 1.1)
    assert [i for _, i in P.candidates(l4, 2)] == [1, 0]


def test_filters_by_hand():
    # src/sample.rs:1065-1163: probabilities 0.5, 0.3, 0.2 as logits
    l = [math.log(0.5), math.log(0.3), math.log(0.2)]
    c = P.candidates(l, 0)
    for p, n in [(0.0, 1), (0.49, 1), (0.51, 2), (0.79, 2), (0.81, 3), (1.0, 3)]:
        assert P.kept(c, p, 0.0) == n, p
    for m, n in [(0.0, 3), (0.39, 3), (0.41, 2), (0.59, 2), (0.61, 1), (1.0, 1)]:
        assert P.kept(c, 1.0, m) == n, m
    assert P.kept(c, 0.81, 0.5) == 2
    c2 = P.candidates(l, 2)
    assert P.kept(c2, 0.6, 0.0) == 1 and P.kept(c2, 0.63, 0.0) == 2
    for u, i in [(0.0, 0), (0.499, 0), (0.501, 1), (0.799, 1), (0.801, 2), (0.9999, 2)]:
        assert P.pick(c, 1.0, 1.0, 0.0, u) == i, u
    inf, nan = float("inf"), float("nan")
    assert P.pick(P.candidates([1.0], 0), 1.0, 1.0, 0.0, 0.7) == 0
    c3 = P.candidates([-inf, 2.0, nan], 0)
    assert [i for _, i in c3] == [1, 0, 2] and P.pick(c3, 1.0, 1.0, 0.0, 0.9999) == 1
    assert P.pick(P.candidates([-inf] * 3, 0), 1.0, 1.0, 0.0, 0.5) == 2
    assert P.pick(P.candidates([nan] * 3, 0), 1.0, 1.0, 0.0, 0.5) == 2
    # temperature after the cut: p^(1/T)
    for t in (0.25, 0.5, 2.0, 7.0):
        w = [p ** (1.0 / t) for p in (0.5, 0.3, 0.2)]
        cum = w[0] / sum(w)
        assert P.pick(c, t, 1.0, 0.0, cum - 1e-9) == 0 and P.pick(c, t, 1.0, 0.0, cum + 1e-9) == 1


def test_draw_skips_zero_weights():
    # src/sample.rs:1218-1232
    w = [1.0, 0.7, 0.3, 0.0, 0.0]
    assert P.draw(w, 0.0) == 0
    assert P.draw(w, 1.0 - 2.0 ** -53) == 2 and P.draw(w, 1.0) == 2 and P.draw(w, 7.0) == 2
    assert P.draw([1.0, 0.0], 1.0) == 0
    assert P.pick(P.candidates([3.0, 1.0, float("-inf")], 0), 0.8, 1.0, 0.0, 1.0 - 2.0 ** -53) != 2
