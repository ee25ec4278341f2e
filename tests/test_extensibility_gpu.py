"""(c)'s generality, shown with toy parts that exist only in this file: a mixer with state of
its own, a feed-forward that routes between experts, another position encoding, windowed
attention layers with pages of their own, a layer that runs twice and a run that reads another
run's cache.  The toy architecture is registered,
built, loaded from a folder written by the random-weights mode and stepped, without a change
to the framework's files, and compared with a plain implementation written here."""
import json
import os
from ctypes import c_float, c_int, c_void_p

import pytest
import torch

import axon_amd
from axon_amd.config import (LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, register_architecture)
from axon_amd.config.base import get_number, get_whole
from axon_amd.engine import StepEntry
from axon_amd.kernels import MODE_ADD_F32, MODE_STORE_F32, KernelError, current_stream, ptr, register_kernel_source
from axon_amd.parts import (FeedForward, Mixer, StateSpec, TensorDecl, build_part, register_feed_forward, register_mixer,
                            register_position)
from axon_amd.parts.rope import RotaryEncoding
from axon_amd.weights import write_random_model
from helpers import tolerance
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


# --------------------------------------------------------------------------- toy parts
# The toy mixer brings a HIP kernel of its own: a file in the tests' folder, registered with its entry
# point's argument types.  The engine compiles it (per compute dtype, at the first call) into a
# library of its own; no file of the framework names it.
register_kernel_source(os.path.join(os.path.dirname(os.path.abspath(__file__)), "toy_kernels", "decay_scan.hip"),
                       {"toy_decay_scan": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int, c_void_p]})


class DecayMixer(Mixer):
    """A toy recurrent mixer: s_t = decay * s_{t-1} + W_in h_t, out_t = W_out s_t.  Its state
    (one vector per request) lives in the cache manager's state slots; it has no pages.  The two
    products are the engine's own kernels, the scan over a request's tokens its own."""

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden, self.width, self.decay = int(params["hidden_size"]), int(params["state_size"]), float(params["decay"])
        self.n_in, self.n_out = prefix + "mixer.in.weight", prefix + "mixer.out.weight"

    def tensors(self):
        return [TensorDecl(self.n_in, (self.width, self.hidden)), TensorDecl(self.n_out, (self.hidden, self.width))]

    def state_spec(self):
        return StateSpec(self.width)

    def load(self, store, rt):
        self.w_in, self.w_out = store.matrix(self.n_in), store.matrix(self.n_out)       # in the compute dtype

    # values of its own on the device in steps of single tokens (here only to show the way: the
    # positions, padded to a multiple of four)
    def decode_input(self, positions):
        return "toy_positions", list(positions) + [-1] * (-len(positions) % 4)

    def decode_input_capacity(self, max_seqs, max_seq_len):
        return max_seqs + 3

    def forward(self, ctx, binding, h, residual):
        if ctx.decode_only:
            self.seen_on_device = ctx.decode_inputs["toy_positions"].clone()
        k, T = ctx.rt.k, h.shape[0]
        arena = ctx.cache.state(binding.state_index)             # [slots, elements] float32
        u = torch.empty((T, self.width), dtype=torch.float32, device=h.device)
        k.gemm(h, self.w_in, u, None, MODE_STORE_F32)
        spans = torch.tensor([[s.slot, s.q_start, s.q_len] for s in ctx.spans], dtype=torch.int32).to(h.device)
        outs = torch.empty((T, self.width), dtype=ctx.rt.dtype, device=h.device)
        k.call("toy_decay_scan", ptr(u), ptr(arena), arena.stride(0), ptr(spans), len(ctx.spans), self.decay, ptr(outs),
               self.width, current_stream())                     # each request's tokens, in order
        k.gemm(outs, self.w_out, residual, None, MODE_ADD_F32)


class HalvedRope(RotaryEncoding):
    """Another position encoding: positions count half (linear scaling); only the table changes."""

    def frequencies(self):
        return super().frequencies() * 0.5


class RoutedFFN(FeedForward):
    """A toy mixture of experts: router logits (32-bit) -> softmax -> the experts' outputs weighted
    by it.  Each expert is the framework's own dense feed-forward under a scope of its own; every
    expert sees every token here (a soft router: no token changes expert by rounding)."""

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden, self.n = int(params["hidden_size"]), int(params["experts"])
        self.router_name = prefix + "mlp.router.weight"
        self.experts = [build_part("feed_forward", PartSpec("swiglu_mlp", {
            "hidden_size": self.hidden, "intermediate_size": int(params["intermediate_size"]),
            "names": {"scope": f"mlp.experts.{e}."}}), prefix) for e in range(self.n)]

    def tensors(self):
        return [TensorDecl(self.router_name, (self.n, self.hidden))] + [d for e in self.experts for d in e.tensors()]

    def load(self, store, rt):
        self.router = store.matrix(self.router_name).float()
        for e in self.experts:
            e.load(store, rt)

    def forward(self, ctx, h, residual):
        weights = torch.softmax(h.float() @ self.router.T, dim=-1)          # [T, experts], 32-bit
        for e, expert in enumerate(self.experts):
            out = torch.zeros_like(residual)
            expert.forward(ctx, h, out)                                     # adds its output into `out`
            residual += weights[:, e:e + 1] * out


register_mixer("toy_decay", DecayMixer)
register_position("toy_halved_rope", HalvedRope)
register_feed_forward("toy_routed", RoutedFFN)


class ToyConfig(ModelConfig):
    architecture = "ToyForCausalLM"

    def __init__(self, cfg):
        self.cfg = dict(cfg)
        self.hidden, self.vocab = get_whole(cfg, "hidden_size"), get_whole(cfg, "vocab_size")
        self.window, self.eps = get_whole(cfg, "window"), get_number(cfg, "eps")
        self.heads, self.kv_heads, self.head_dim = (get_whole(cfg, k) for k in ("heads", "kv_heads", "head_dim"))
        self.ffn, self.state, self.decay = get_whole(cfg, "ffn"), get_whole(cfg, "state_size"), get_number(cfg, "decay")
        self.max_pos = get_whole(cfg, "max_positions")

    @classmethod
    def from_dict(cls, cfg):
        return cls(cfg)

    def to_dict(self):
        return dict(self.cfg)

    def model_spec(self):
        norm = PartSpec("rmsnorm", {"size": self.hidden, "eps": self.eps})
        ffn = PartSpec("swiglu_mlp", {"hidden_size": self.hidden, "intermediate_size": self.ffn})

        def attn(window, position):
            return PartSpec("gqa_attention", {"hidden_size": self.hidden, "num_heads": self.heads,
                                              "num_kv_heads": self.kv_heads, "head_dim": self.head_dim, "qkv_bias": True,
                                              "window": window, "position": position})
        rope = PartSpec("rope", {"head_dim": self.head_dim, "theta": 1000.0})
        halved = PartSpec("toy_halved_rope", {"head_dim": self.head_dim, "theta": 1000.0})
        decay = PartSpec("toy_decay", {"hidden_size": self.hidden, "state_size": self.state, "decay": self.decay})
        routed = PartSpec("toy_routed", {"hidden_size": self.hidden, "intermediate_size": self.ffn, "experts": 3})
        layers = [LayerSpec("prenorm", attn(self.window, rope), ffn, norm, "layers.0."),     # windowed attention
                  LayerSpec("prenorm", decay, routed, norm, "layers.1."),                   # state of its own; routed experts
                  LayerSpec("prenorm", attn(0, halved), ffn, norm, "layers.2.")]            # full, other positions
        # layer 0 runs twice (each run its own cache); the last run reads what layer 2 stored
        order = [Run(0, cache=0), Run(1, cache=1), Run(2, cache=2), Run(0, cache=3), Run(2, cache=2, writes_cache=False)]
        return ModelSpec(self.hidden, self.vocab,
                         PartSpec("token_embedding", {"vocab_size": self.vocab, "hidden_size": self.hidden, "tensor": "embed.weight"}),
                         layers, order, PartSpec("rmsnorm", {"size": self.hidden, "eps": self.eps, "tensor": "norm.weight"}),
                         PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.hidden, "tensor": "head.weight",
                                              "tied_to": "embed.weight", "tied": False}), self.max_pos)


register_architecture("ToyForCausalLM", ToyConfig, "toy")

TOY = dict(architectures=["ToyForCausalLM"], model_type="toy", hidden_size=40, vocab_size=90, window=11, eps=1e-4, heads=4,
           kv_heads=2, head_dim=16, ffn=72, state_size=24, decay=0.8, max_positions=256)


# --------------------------------------------------------------------------- its plain twin
def toy_plain(w, tokens):
    c = TOY
    x = w["embed.weight"][torch.as_tensor(tokens)]
    T = len(tokens)
    pos = torch.arange(T)
    kept = {}

    def attention(x, l, window, scale_pos, store_as=None, read_from=None):
        p = f"layers.{l}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], c["eps"])
        pre = p + "self_attn."
        q = P.linear(h, w[pre + "q_proj.weight"], w[pre + "q_proj.bias"]).view(T, c["heads"], c["head_dim"])
        sin, cos = P.rope_table(pos, P.rope_freqs(c["head_dim"], 1000.0) * scale_pos)
        q = P.apply_rope(q, sin, cos)
        if read_from is None:
            k = P.apply_rope(P.linear(h, w[pre + "k_proj.weight"], w[pre + "k_proj.bias"]).view(T, c["kv_heads"], c["head_dim"]), sin, cos)
            v = P.linear(h, w[pre + "v_proj.weight"], w[pre + "v_proj.bias"]).view(T, c["kv_heads"], c["head_dim"])
            if store_as is not None:
                kept[store_as] = (k, v)
        else:
            k, v = kept[read_from]
        att = P.causal_attention(q, k, v, window).reshape(T, -1)
        x = x + P.linear(att, w[pre + "o_proj.weight"])
        return x + P.mlp_block({k2.replace(p, "model.layers.0."): v2 for k2, v2 in w.items() if k2.startswith(p + "mlp")}, 0,
                               P.rms_norm(x, w[p + "post_attention_layernorm.weight"], c["eps"]))

    def decay(x, l):
        p = f"layers.{l}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], c["eps"])
        u = h @ w[p + "mixer.in.weight"].T
        s = torch.zeros(c["state_size"], dtype=x.dtype)
        outs = []
        for t in range(T):
            s = c["decay"] * s + u[t]
            outs.append(s)
        x = x + torch.stack(outs) @ w[p + "mixer.out.weight"].T
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], c["eps"])
        weights = torch.softmax(h @ w[p + "mlp.router.weight"].T, dim=-1)
        for e in range(3):
            scope = f"{p}mlp.experts.{e}."
            expert = {k2.replace(scope, "model.layers.0.mlp."): v2 for k2, v2 in w.items() if k2.startswith(scope)}
            x = x + weights[:, e:e + 1] * P.mlp_block(expert, 0, h)
        return x

    x = attention(x, 0, c["window"], 1.0)
    x = decay(x, 1)
    x = attention(x, 2, 0, 0.5, store_as="l2")
    x = attention(x, 0, c["window"], 1.0)
    x = attention(x, 2, 0, 0.5, read_from="l2")
    return P.linear(P.rms_norm(x, w["norm.weight"], c["eps"]), w["head.weight"])


@pytest.fixture(scope="module")
def toy_dir(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("toy"))
    write_random_model(ToyConfig.from_dict(TOY), d, seed=2, std=0.08)
    return d


def test_the_toy_architecture_is_described_by_its_parts(toy_dir):
    from axon_amd.models import build_model_description
    model = build_model_description(ToyConfig.from_dict(TOY))
    plan = model.cache_plan
    # two cache groups with pages of their own: the windowed runs (two of them: layer 0 twice)
    # and the full one (layer 2 once; its second run stores nothing); one state arena
    assert [(s.window, n) for s, n in zip(plan.group_specs, plan.group_layers)] == [(11, 2), (0, 1)]
    assert plan.state_elems == [(24, "float32")]                 # the state's size and its element type
    assert [(b.group, b.index, b.writes, b.state_index) for b in plan.bindings] == [
        (0, 0, True, -1), (-1, -1, True, 0), (1, 0, True, -1), (0, 1, True, -1), (1, 0, False, -1)]
    names = {d.name for d in model.tensors()}
    assert "layers.1.mixer.in.weight" in names and "layers.0.self_attn.q_proj.bias" in names
    assert "layers.1.mlp.router.weight" in names and "layers.1.mlp.experts.2.down_proj.weight" in names
    assert json.load(open(os.path.join(toy_dir, "config.json")))["architectures"] == ["ToyForCausalLM"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_toy_model_steps_like_its_plain_twin(toy_dir, dtype):
    from safetensors.torch import load_file
    w = {k: v.double() for k, v in load_file(os.path.join(toy_dir, "model.safetensors")).items()}
    g = torch.Generator().manual_seed(4)
    seqs = [torch.randint(0, 90, (n,), generator=g).tolist() for n in (60, 37, 90)]
    refs = [toy_plain(w, s).float() for s in seqs]
    llm = axon_amd.load(toy_dir, dtype=dtype, page_size=4, num_pages=56, max_seqs=3)
    eng = llm.engine
    # bfloat16 here: the toy folder holds float32 weights that the engine rounds, so the
    # comparison carries the weights' rounding too
    slack = 1.0 if dtype == "float32" else 2.0
    # whole
    for s, ref in zip(seqs, refs):
        got = llm.logits(s, all_positions=True).cpu()
        assert (got - ref).abs().max() <= slack * tolerance(dtype, ref)
    # in portions, three requests interleaved, with single tokens beside portions
    cuts = [(7, 2, 1, 16, 1, 33), (20, 1, 1, 15), (2, 40, 3, 1, 44)]
    at = [0, 0, 0]
    got = [[], [], []]
    step = 0
    while any(a < len(s) for a, s in zip(at, seqs)):
        entries = []
        for i, s in enumerate(seqs):
            if at[i] >= len(s):
                continue
            n = min(cuts[i][step % len(cuts[i])], len(s) - at[i])
            entries.append(StepEntry(i, s[at[i]:at[i] + n], list(range(n))))
        out = eng.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.id].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
            at[e.id] += len(e.tokens)
        step += 1
    for i, ref in enumerate(refs):
        assert (torch.cat(got[i]) - ref).abs().max() <= slack * tolerance(dtype, ref)
    # the windowed group gave pages back on the way: 90 positions of window 11 hold at most 4 pages of 4
    slot = eng.live[2].slot
    assert eng.cache.pages_of(0, slot) <= 4 and eng.cache.pages_of(1, slot) == 23
    eng.release_all()
    eng.cache.check()
    assert eng.cache.free_pages(0) == 56 and eng.cache.free_pages(1) == 56
    # a slot that is used again starts from a zero state
    again = llm.logits(seqs[1], all_positions=True).cpu()
    assert (again - refs[1]).abs().max() <= slack * tolerance(dtype, refs[1])
    # and generation works through the same entry point
    out = llm.generate([seqs[0][:9], seqs[1][:5]], max_new_tokens=6)
    assert [len(o) for o in out] == [6, 6]
    # decoding steps replay graphs for the runs whose parts allow it; the toy mixer's run, which
    # keeps state and reads host values, is launched between two graphs, once a step
    assert eng.graphs_ok and [(c, a, b) for c, a, b in eng._segments] == [(True, 0, 1), (False, 1, 2), (True, 2, 5)]
    assert eng._graphs and all(g is not None for e in eng._graphs.values() for g, (c, _, _) in
                               zip(e["graphs"], eng._segments) if c)
    # what the toy mixer asked to have on the device in the last step of single tokens
    decay = next(b.mixer for b in llm.model.blocks if isinstance(b.mixer, DecayMixer))
    assert decay.seen_on_device.tolist() == [13, 9, -1, -1]
    if dtype == "float32":
        for p, o in zip((seqs[0][:9], seqs[1][:5]), out):
            hist = list(p)
            for tok in o:
                assert tok == P.argmax_last(toy_plain(w, hist)[-1].float())
                hist.append(tok)


def test_a_parts_own_kernel_source_is_built_and_called_without_a_change_to_the_framework(toy_dir):
    """The registered source compiles into a library of its own for each compute dtype, its entry
    point is reached through `Kernels.call`, refuses what it says it refuses with its own message,
    and an unknown name is an error."""
    from axon_amd.kernels import kernels
    for dtype, torch_dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        k = kernels(dtype)
        u = torch.arange(12, dtype=torch.float32).view(4, 3).cuda()
        state = torch.tensor([[1.0, 2.0, 3.0, 0.0], [0.0, 0.0, 0.0, 0.0]]).cuda()           # stride 4, width 3
        spans = torch.tensor([[1, 0, 1], [0, 1, 3]], dtype=torch.int32).cuda()
        out = torch.zeros(4, 3, dtype=torch_dtype, device="cuda")
        k.call("toy_decay_scan", ptr(u), ptr(state), 4, ptr(spans), 2, 0.5, ptr(out), 3, current_stream())
        want, s = [], torch.tensor([1.0, 2.0, 3.0])
        for t in (1, 2, 3):
            s = 0.5 * s + u[t].cpu()
            want.append(s)
        assert torch.equal(out[0].float().cpu(), u[0].cpu())                                # slot 1 started from zero
        assert torch.equal(out[1:].float().cpu(), torch.stack(want).to(torch_dtype).float())
        assert torch.equal(state[0, :3].cpu(), s) and state[0, 3] == 0
        with pytest.raises(KernelError, match="toy_decay_scan: 1 spans, width 5, state stride 4"):
            k.call("toy_decay_scan", ptr(u), ptr(state), 4, ptr(spans), 1, 0.5, ptr(out), 5, current_stream())
        with pytest.raises(KernelError, match="no registered kernel source"):
            k.call("toy_missing")

