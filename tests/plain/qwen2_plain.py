"""A plain, slow implementation of the Qwen2.5 dense decoder: whole sequences, no cache,
one function for each part.  It is the oracle of the test suite and shares no code with
the engine (it imports nothing from ``axon_amd``).

Every function is written from the formulas of the reference's CPU forward pass and
cites the lines it follows (paths are relative to the reference's root).  The default
arithmetic is float64, as the reference's own independent check ``dense_ref`` is
(src/model.rs:4575-4834); pass ``dtype=torch.float32`` to see 32-bit rounding.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass

import torch


# --------------------------------------------------------------------------- config

@dataclass
class PlainConfig:
    """The numbers the forward pass needs, by their config.json names
    (src/safetensors.rs:637-660 lists the keys, src/model.rs:1777-1785 the defaults)."""
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    window: int = 0          # 0: every earlier position is seen (qwen2 has no window)

    @staticmethod
    def from_json(path: str) -> "PlainConfig":
        with open(path) as f:
            c = json.load(f)
        nh = c["num_attention_heads"]
        return PlainConfig(
            num_hidden_layers=c["num_hidden_layers"],
            hidden_size=c["hidden_size"],
            num_attention_heads=nh,
            num_key_value_heads=c["num_key_value_heads"],
            # head_dim is optional: hidden_size / heads without it (src/model.rs:1782-1783)
            head_dim=c.get("head_dim") or c["hidden_size"] // nh,
            # theta defaults to 10000 (src/model.rs:639), eps to 1e-6 (src/model.rs:1784)
            # the loader keeps theta as a 32-bit float and widens it (src/safetensors.rs:649-651)
            rope_theta=float(torch.tensor(float(c.get("rope_theta", 10000.0)), dtype=torch.float32)),
            rms_norm_eps=float(c.get("rms_norm_eps", 1e-6)),
            # tie_word_embeddings defaults to false (src/safetensors.rs:1608-1609)
            tie_word_embeddings=bool(c.get("tie_word_embeddings", False)),
        )


def load_plain(model_dir: str, dtype=torch.float64):
    """config + tensors of a model folder, read with the safetensors package (the engine has
    a reader of its own, so the two also check each other)."""
    from safetensors.torch import load_file
    cfg = PlainConfig.from_json(os.path.join(model_dir, "config.json"))
    w = load_file(os.path.join(model_dir, "model.safetensors"))
    return cfg, {k: v.to(dtype) for k, v in w.items()}


# --------------------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm over the last axis: ss = sum x^2; ms = ss / n; inv = 1 / sqrt(ms + eps);
    out = (x * inv) * gain  (src/model.rs:3888-3898: x times inv first, then the gain)."""
    ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    inv = 1.0 / torch.sqrt(ms + eps)
    return (x * inv) * gain


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y[o] = row o of W . x, then the bias: weights are [out][in] row-major, the bias is
    added after the product (src/model.rs:2982-2991)."""
    y = x @ weight.T
    return y if bias is None else y + bias


def rope_freqs(head_dim: int, theta: float, dtype=torch.float64) -> torch.Tensor:
    """freq_i = theta^(-2i / head_dim) for each pair i < head_dim / 2, in f64
    (src/model.rs:638-657)."""
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(theta, dtype=torch.float64), -2.0 * i / head_dim).to(dtype)


def rope_table(positions: torch.Tensor, freqs: torch.Tensor):
    """(sin, cos) of angle = pos * freq_i, computed in f64 (src/model.rs:2612-2621)."""
    angle = positions.to(torch.float64)[:, None] * freqs.to(torch.float64)[None, :]
    return torch.sin(angle), torch.cos(angle)


def apply_rope(v: torch.Tensor, sin: torch.Tensor, cos: torch.Tensor) -> torch.Tensor:
    """Rotate-half on heads: v is [T, heads, head_dim]; dim i is paired with dim i + head_dim/2:
    out[i] = a cos - b sin, out[i + half] = a sin + b cos  (src/model.rs:3922-3929)."""
    half = v.shape[-1] // 2
    a, b = v[..., :half], v[..., half:]
    s = sin[:, None, :].to(v.dtype)
    c = cos[:, None, :].to(v.dtype)
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """q [T, nh, hd], k and v [T, nkv, hd] -> [T, nh, hd].  Query head qh reads kv head
    qh // group (src/model.rs:3386-3389, 3414).  s_t = dot(q, k_t) * scale with
    scale = 1 / sqrt(hd), multiplied after the dot (src/model.rs:3392); softmax over
    t = 0..=pos: subtract the max, exp, divide by the sum (src/vmath.rs:344-352); the output
    is sum_t w_t v_t (src/model.rs:3635-3669).  There is no mask tensor: token b sees
    positions 0..=b (src/model.rs:2837-2856).  With a window w a token sees only the last w
    positions, itself included (src/model.rs:599-604)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    scale = 1.0 / math.sqrt(hd)
    out = torch.zeros_like(q)
    for t in range(T):
        lo = 0 if window <= 0 else max(0, t + 1 - window)
        for qh in range(nh):
            kvh = qh // group
            s = (k[lo:t + 1, kvh, :] @ q[t, qh, :]) * scale
            m = s.max()
            e = torch.exp(s - m)
            w = e * (1.0 / e.sum())
            out[t, qh, :] = w @ v[lo:t + 1, kvh, :]
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """act = (g / (1 + exp(-g))) * u: divide, then multiply (src/vmath.rs:128-132)."""
    return gate / (1.0 + torch.exp(-gate)) * up


def attention_block(cfg: PlainConfig, w: dict, layer: int, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """Steps 2-6 of the reference's layer (src/model.rs:2980-3038): q, k, v projections with
    bias, RoPE on q and k, causal GQA attention, output projection (no bias)."""
    p = f"model.layers.{layer}.self_attn."
    T = h.shape[0]
    nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    q = linear(h, w[p + "q_proj.weight"], w.get(p + "q_proj.bias")).view(T, nh, hd)
    k = linear(h, w[p + "k_proj.weight"], w.get(p + "k_proj.bias")).view(T, nkv, hd)
    v = linear(h, w[p + "v_proj.weight"], w.get(p + "v_proj.bias")).view(T, nkv, hd)
    sin, cos = rope_table(positions, rope_freqs(hd, cfg.rope_theta))
    q = apply_rope(q, sin, cos)
    k = apply_rope(k, sin, cos)
    att = causal_attention(q, k, v, cfg.window).reshape(T, nh * hd)
    return linear(att, w[p + "o_proj.weight"])


def mlp_block(w: dict, layer: int, h: torch.Tensor) -> torch.Tensor:
    """Steps 7-8 (src/model.rs:3042-3055): down(swiglu(gate h, up h)), no biases."""
    p = f"model.layers.{layer}.mlp."
    act = swiglu(linear(h, w[p + "gate_proj.weight"]), linear(h, w[p + "up_proj.weight"]))
    return linear(act, w[p + "down_proj.weight"])


def hidden_states(cfg: PlainConfig, w: dict, tokens, start: int = 0) -> torch.Tensor:
    """Embedding and every layer for a whole sequence at positions start.. (no cache):
    the loop of src/model.rs:2967-3059 (embed, then per layer norm1, attention, add, norm2,
    feed-forward, add).  The embedding row is used as it is (src/model.rs:2657-2675)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][tokens]
    positions = torch.arange(start, start + len(tokens))
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        h = rms_norm(x, w[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        x = x + attention_block(cfg, w, l, h, positions)
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        x = x + mlp_block(w, l, h)
    return x


def logits_of(cfg: PlainConfig, w: dict, x: torch.Tensor) -> torch.Tensor:
    """Final norm, then the head: lm_head.weight if the model is untied, else the embedding
    matrix (src/model.rs:2640-2645, 1800-1803)."""
    h = rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps)
    head = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return linear(h, head)


def forward_logits(cfg: PlainConfig, w: dict, tokens) -> torch.Tensor:
    """Logits [T, V] at every position of a whole sequence."""
    return logits_of(cfg, w, hidden_states(cfg, w, tokens))


# --------------------------------------------------------------------------- picking

def argmax_last(logits) -> int:
    """The largest logit by `>`; of equal maxima the last index; NaN is never picked; all NaN
    gives the last index; -0.0 ties +0.0 (src/generate.rs:222-264)."""
    best, arg = -math.inf, None
    vals = [float(v) for v in logits]
    for v in vals:
        if v > best:
            best = v
    for i in range(len(vals) - 1, -1, -1):
        if vals[i] == best:
            arg = i
            break
    return len(vals) - 1 if arg is None else arg


def greedy_generate(cfg: PlainConfig, w: dict, prompt, n_new: int, stop=()) -> list:
    """The greedy loop of src/generate.rs:154-219 without a cache: pick, stop before emitting a
    stop token, emit, stop at n_new."""
    hist = list(prompt)
    out = []
    while len(out) < n_new:
        pick = argmax_last(forward_logits(cfg, w, hist)[-1])
        if pick in stop:
            break
        out.append(pick)
        hist.append(pick)
    return out


# --------------------------------------------------------------------------- sampling

MASK64 = (1 << 64) - 1


def splitmix64(state: int):
    """One step of splitmix64 (src/sample.rs:202-208): returns (new state, output)."""
    state = (state + 0x9E3779B97F4A7C15) & MASK64
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return state, z ^ (z >> 31)


class PlainRng:
    """xoshiro256** seeded by four splitmix64 outputs (src/sample.rs:212-242)."""

    def __init__(self, seed: int):
        s = seed & MASK64
        self.s = []
        for _ in range(4):
            s, z = splitmix64(s)
            self.s.append(z)

    @staticmethod
    def _rotl(x, k):
        return ((x << k) | (x >> (64 - k))) & MASK64

    def next_u64(self) -> int:
        s = self.s
        r = (self._rotl((s[1] * 5) & MASK64, 7) * 9) & MASK64
        t = (s[1] << 17) & MASK64
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = self._rotl(s[3], 45)
        return r

    def f64(self) -> float:
        """Uniform in [0, 1), 53 bits (src/sample.rs:238-241)."""
        return (self.next_u64() >> 11) * (1.0 / (1 << 53))


def penalize(logits: list, recent: list, last_n: int, penalty: float) -> list:
    """llama.cpp's repeat penalty on the distinct ids among the last `last_n` of `recent`:
    a positive logit is divided by p, any other multiplied (src/sample.rs:307-326)."""
    out = list(logits)
    if penalty == 1.0 or last_n == 0:
        return out
    for i in sorted(set(recent[max(0, len(recent) - last_n):])):
        out[i] = out[i] / penalty if out[i] > 0 else out[i] * penalty
    return out


def candidates(logits: list, k: int) -> list:
    """The k best (logit, id), best first; equal logits: the larger id first; NaN last
    (src/sample.rs:280-305, 391-429).  k = 0: all of them."""
    def key(item):
        v, i = item
        if v != v:
            return (0, -math.inf, i)
        return (1, v + 0.0, i)
    items = sorted(((float(v), i) for i, v in enumerate(logits)), key=key, reverse=True)
    return items if k == 0 else items[:k]


def kept(cands: list, top_p: float, min_p: float) -> int:
    """How many candidates survive top-p, then min-p (src/sample.rs:465-500)."""
    n = 0
    for v, _ in cands:
        if v != v:
            break
        n += 1
    l0 = cands[0][0]
    if n <= 1 or not math.isfinite(l0):
        return 1
    if top_p < 1.0:
        e = [math.exp(v - l0) for v, _ in cands[:n]]
        z = 0.0
        for x in e:
            z += x
        cum, cut = 0.0, len(e)
        for i, x in enumerate(e):
            cum += x / z
            if cum >= top_p:
                cut = i + 1
                break
        n = cut
    if min_p > 0.0:
        lo = l0 + math.log(min_p)
        m = 0
        for v, _ in cands[:n]:
            if v >= lo:
                m += 1
            else:
                break
        n = max(m, 1)
    return n


def draw(weights: list, u: float) -> int:
    """The inverse CDF: the first i whose cumulative weight passes u * total, never a
    zero-weight index (src/sample.rs:542-556)."""
    z = 0.0
    for x in weights:
        z += x
    target = min(u * z, math.nextafter(z, -math.inf))
    cum, last = 0.0, 0
    for i, x in enumerate(weights):
        if x > 0:
            last = i
        cum += x
        if target < cum:
            return i
    return last


def pick(cands: list, temp: float, top_p: float, min_p: float, u: float) -> int:
    """top-p, min-p, temperature, then the draw (src/sample.rs:523-536)."""
    n = kept(cands, top_p, min_p)
    if n == 1:
        return cands[0][1]
    l0 = cands[0][0]
    w = [math.exp((v - l0) / temp) for v, _ in cands[:n]]
    return cands[draw(w, u)][1]


def sample_generate(cfg: PlainConfig, w: dict, prompt, n_new: int, *, temp, top_k, top_p, min_p,
                    repeat_penalty, repeat_last_n, seed, stop=()) -> list:
    """The sampled loop of src/sample.rs:574-654 without drafting: penalty -> top-k ->
    top-p -> min-p -> temperature -> one draw per decided token."""
    rng = PlainRng(seed)
    hist = list(prompt)
    out = []
    while len(out) < n_new:
        logits = [float(v) for v in forward_logits(cfg, w, hist)[-1].to(torch.float32)]
        c = candidates(penalize(logits, hist, repeat_last_n, repeat_penalty), top_k)
        nxt = pick(c, temp, top_p, min_p, rng.f64())
        if nxt in stop:
            break
        out.append(nxt)
        hist.append(nxt)
    return out
