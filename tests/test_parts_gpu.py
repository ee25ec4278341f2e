"""Each part of a layer alone, built from a PartSpec with sizes of its own, against the plain
function of the same part."""

import pytest
import torch

from axon_amd.config import PartSpec
from axon_amd.parts import CacheBinding, build_block, build_part
from axon_amd.weights import WeightStore
from gpu_helpers import DTYPES, TORCH, DictSource, PartHarness, tol
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def rounded(t, dtype):
    return t.to(TORCH[dtype]).float()


def load(part, tensors, h):
    part.load(WeightStore(DictSource(tensors), h.rt.device, h.rt.dtype), h.rt)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    h = PartHarness(dtype)
    part = build_part("norm", PartSpec("rmsnorm", {"size": 72, "eps": 0.02, "tensor": "g"}), "layer.")
    assert [(d.name, d.shape, d.role) for d in part.tensors()] == [("layer.g", (72,), "gain")]
    gain = 1 + rnd(72, seed=1) * 0.2
    load(part, {"layer.g": gain}, h)
    x = rnd(5, 72, seed=2, scale=2.0)
    out = part.forward(h.ctx([0] * 5), x.cuda())
    ref = P.rms_norm(x.double(), gain.double(), 0.02)
    assert out.dtype == TORCH[dtype] and (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 1e-6, 8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,hidden,theta,window,bias", [(4, 2, 16, 40, 1e4, 0, True), (3, 1, 32, 50, 1e6, 0, True),
                                                                (6, 2, 48, 72, 500.0, 9, False)])
def test_attention_mixer_alone(dtype, nh, nkv, hd, hidden, theta, window, bias):
    spec = PartSpec("gqa_attention", {"hidden_size": hidden, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd,
                                      "qkv_bias": "optional", "out_bias": False, "window": window,
                                      "position": PartSpec("rope", {"head_dim": hd, "theta": theta})})
    mixer = build_part("mixer", spec, "L.")
    cs = mixer.cache_spec()
    assert (cs.entries, cs.heads, cs.head_dim, cs.window) == (2, nkv, hd, window)
    h = PartHarness(dtype, cs, page_size=4, n_pages=40)
    w = {"L.self_attn.q_proj.weight": rnd(nh * hd, hidden, seed=1, scale=0.2),
         "L.self_attn.k_proj.weight": rnd(nkv * hd, hidden, seed=2, scale=0.2),
         "L.self_attn.v_proj.weight": rnd(nkv * hd, hidden, seed=3, scale=0.2),
         "L.self_attn.o_proj.weight": rnd(hidden, nh * hd, seed=4, scale=0.2)}
    if bias:
        w.update({"L.self_attn.q_proj.bias": rnd(nh * hd, seed=5), "L.self_attn.k_proj.bias": rnd(nkv * hd, seed=6),
                  "L.self_attn.v_proj.bias": rnd(nkv * hd, seed=7)})
    w = {k: rounded(v, dtype) for k, v in w.items()}
    load(mixer, w, h)
    T = 37
    x = rounded(rnd(T, hidden, seed=8), dtype)
    cfg = P.PlainConfig(1, hidden, nh, nkv, hd, theta, 1e-6, False, window)
    plain_w = {k.replace("L.", "model.layers.0."): v.double() for k, v in w.items()}
    ref = P.attention_block(cfg, plain_w, 0, x.double(), torch.arange(T))
    binding = CacheBinding(group=0, index=0, writes=True)
    # in portions: 20 tokens, then 16, then 1 (a decode token); the residual starts at 1.0
    got = []
    at = 0
    for n in (20, 16, 1):
        res = torch.ones(n, hidden, dtype=torch.float32, device="cuda")
        mixer.forward(h.ctx([0] * n), binding, x[at:at + n].to(TORCH[dtype]).cuda(), res)
        got.append(res.cpu().double() - 1.0)
        at += n
    got = torch.cat(got)
    assert (got - ref).abs().max() <= tol(dtype, ref, 5e-6, 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_mlp_alone(dtype):
    h = PartHarness(dtype)
    part = build_part("feed_forward", PartSpec("swiglu_mlp", {"hidden_size": 56, "intermediate_size": 150}), "L.")
    w = {"L.mlp.gate_proj.weight": rnd(150, 56, seed=1, scale=0.3), "L.mlp.up_proj.weight": rnd(150, 56, seed=2, scale=0.3),
         "L.mlp.down_proj.weight": rnd(56, 150, seed=3, scale=0.3)}
    w = {k: rounded(v, dtype) for k, v in w.items()}
    assert sorted(d.name for d in part.tensors()) == sorted(w)
    load(part, w, h)
    x = rounded(rnd(9, 56, seed=4), dtype)
    res = torch.full((9, 56), 2.0, dtype=torch.float32, device="cuda")
    part.forward(h.ctx([0] * 9), x.to(TORCH[dtype]).cuda(), res)
    ref = P.mlp_block({k.replace("L.", "model.layers.0."): v.double() for k, v in w.items()}, 0, x.double())
    assert (res.cpu().double() - 2.0 - ref).abs().max() <= tol(dtype, ref, 5e-6, 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head(dtype):
    h = PartHarness(dtype)
    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": 33, "hidden_size": 24, "tensor": "E"}))
    table = rounded(rnd(33, 24, seed=1), dtype)
    head_w = rounded(rnd(33, 24, seed=2), dtype)
    store = WeightStore(DictSource({"E": table, "H": head_w}), h.rt.device, h.rt.dtype)
    emb.load(store, h.rt)
    toks = [5, 0, 32, 5]
    x = emb.forward(h.ctx(toks))
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table[toks])
    hidden = rounded(rnd(4, 24, seed=3), dtype)
    for tied, weight in ((False, head_w), (True, table)):
        params = {"vocab_size": 33, "hidden_size": 24, "tensor": "H" if not tied else "absent", "tied_to": "E", "tied": tied}
        head = build_part("head", PartSpec("lm_head", params))
        head.load(store, h.rt)
        out = head.forward(h.ctx([0] * 4), hidden.to(TORCH[dtype]).cuda())
        ref = hidden.double() @ weight.double().T
        assert out.dtype == torch.float32 and (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 5e-6, 1e-4)
    assert head.weight.data_ptr() == emb.table.data_ptr()                      # tied: one matrix in memory


@pytest.mark.parametrize("dtype", DTYPES)
def test_prenorm_block_arrangement(dtype):
    hidden, nh, nkv, hd, ffn, eps = 48, 4, 2, 16, 100, 0.3
    mixer = build_part("mixer", PartSpec("gqa_attention", {
        "hidden_size": hidden, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd, "qkv_bias": True,
        "position": PartSpec("rope", {"head_dim": hd, "theta": 100.0})}), "model.layers.0.")
    ffn_part = build_part("feed_forward", PartSpec("swiglu_mlp", {"hidden_size": hidden, "intermediate_size": ffn}),
                          "model.layers.0.")
    block = build_block("prenorm", PartSpec("rmsnorm", {"size": hidden, "eps": eps}), mixer, ffn_part, "model.layers.0.")
    from test_plain import random_weights
    cfg = P.PlainConfig(1, hidden, nh, nkv, hd, 100.0, eps, True)
    w = {k: rounded(v.float(), dtype) for k, v in random_weights(cfg, ffn, 10, 0.3).items() if "layers.0" in k}
    assert sorted(d.name for d in block.tensors()) == sorted(w)
    h = PartHarness(dtype, mixer.cache_spec())
    load(block, w, h)
    x0 = rnd(13, hidden, seed=9)
    x = x0.clone().cuda()
    block.forward(h.ctx([0] * 13), CacheBinding(0, 0, True), x)
    wd = {k: v.double() for k, v in w.items()}
    p = "model.layers.0."
    r = x0.double()
    r = r + P.attention_block(cfg, wd, 0, P.rms_norm(r, wd[p + "input_layernorm.weight"], eps), torch.arange(13))
    r = r + P.mlp_block(wd, 0, P.rms_norm(r, wd[p + "post_attention_layernorm.weight"], eps))
    assert (x.cpu().double() - r).abs().max() <= tol(dtype, r, 1e-5, 3e-2)


def test_prenorm_block_whose_products_finish_the_norms_behind_them():
    """A step of some tens of rows in bfloat16 with narrow products, whose segments of K run in
    blocks of their own: the output projection writes the second norm's rows and the down
    projection the next block's first norm; only a norm nobody did for the block runs on its
    own.  Against the plain formulas, and the same bits as with every norm on its own."""
    dtype = "bfloat16"
    hidden, nh, nkv, hd, ffn, eps, T = 256, 8, 2, 64, 512, 1e-3, 80
    mixer = build_part("mixer", PartSpec("gqa_attention", {
        "hidden_size": hidden, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd, "qkv_bias": True,
        "position": PartSpec("rope", {"head_dim": hd, "theta": 100.0})}), "model.layers.0.")
    ffn_part = build_part("feed_forward", PartSpec("swiglu_mlp", {"hidden_size": hidden, "intermediate_size": ffn}),
                          "model.layers.0.")
    block = build_block("prenorm", PartSpec("rmsnorm", {"size": hidden, "eps": eps}), mixer, ffn_part, "model.layers.0.")
    from test_plain import random_weights
    cfg = P.PlainConfig(1, hidden, nh, nkv, hd, 100.0, eps, True)
    w = {k: rounded(v.float(), dtype) for k, v in random_weights(cfg, ffn, 10, 0.1).items() if "layers.0" in k}
    p = "model.layers.0."
    w[p + "input_layernorm.weight"] = 1.0 + 0.5 * rnd(hidden, seed=3)
    w[p + "post_attention_layernorm.weight"] = 1.0 + 0.5 * rnd(hidden, seed=4)
    h = PartHarness(dtype, mixer.cache_spec())
    load(block, w, h)
    ctx = h.ctx([0] * T)
    assert mixer.finishes_following_norm(ctx) and block.last_part().finishes_following_norm(ctx)
    x0 = rnd(T, hidden, seed=9, scale=3.0)
    x0[2] *= 30.0
    next_gain = (1.0 + 0.5 * rnd(hidden, seed=5)).cuda()
    nxt = block.following_of(ctx, block.last_part(), block.first_norm(), T)
    nxt.gain, nxt.eps = next_gain, 1e-5
    calls = []
    real = h.rt.k.rmsnorm
    h.rt.k.rmsnorm = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
    try:
        x = x0.clone().cuda()
        block.forward(ctx, CacheBinding(0, 0, True), x, None, nxt)
    finally:
        h.rt.k.rmsnorm = real
    assert len(calls) == 1                                                    # the first norm alone
    wd = {k: v.double() for k, v in w.items()}
    r = x0.double()
    r = r + P.attention_block(cfg, wd, 0, P.rms_norm(r, wd[p + "input_layernorm.weight"], eps), torch.arange(T))
    r = r + P.mlp_block(wd, 0, P.rms_norm(r, wd[p + "post_attention_layernorm.weight"], eps))
    assert (x.cpu().double() - r).abs().max() <= tol(dtype, r, 1e-5, 3e-2)
    rows = nxt.values
    want = P.rms_norm(r, next_gain.cpu().double(), 1e-5)
    assert (rows.cpu().double() - want).abs().max() <= tol(dtype, want, 0, 3e-2)
    # the same block and rows with every norm on its own: the same bits
    x2 = x0.clone().cuda()
    block.forward(ctx, CacheBinding(0, 0, True), x2)
    assert torch.equal(x2, x)
    assert torch.equal(real(x2, next_gain, 1e-5, torch.empty(T, hidden, dtype=torch.bfloat16, device="cuda")), rows)
    # a short step: no product offers it, the block runs its norms itself
    small = PartHarness(dtype, mixer.cache_spec())
    assert not mixer.finishes_following_norm(small.ctx([0] * 9))


def test_tied_head_and_embedding_share_the_packed_matrix(tmp_path):
    """bfloat16, widths the matrix cores take: the head's matrix is repacked for its product and
    the embedding reads rows out of that same copy (one matrix in memory); the rows are exact."""
    from axon_amd.engine import Runtime
    from axon_amd.engine.loading import load_model
    from axon_amd.kernels import PackedMatrix
    from helpers import make_model_dir
    from axon_amd.weights.safetensors_io import Checkpoint
    d = make_model_dir(str(tmp_path / "m"), "D", storage="bfloat16")            # tied, hidden 192
    rt = Runtime("bfloat16")
    model = load_model(d, rt)
    assert isinstance(model.head.weight, PackedMatrix) and model.embedding.table is model.head.weight
    table = Checkpoint(d).tensor("model.embed_tokens.weight")
    toks = torch.tensor([0, 1, 15, 16, 17, 299, 150], dtype=torch.int32).cuda()
    out = torch.empty(7, 192, dtype=torch.float32, device="cuda")
    rt.k.embed(toks, model.embedding.table, out)
    assert torch.equal(out.cpu(), table[toks.cpu().long()].float())
    # a leading slice of whole row tiles is a view of the same storage; other cuts are refused
    part = model.head.weight[:32]
    assert part.shape == (32, 192) and part.data.data_ptr() == model.head.weight.data.data_ptr()
    x = torch.randn(5, 192, device="cuda").bfloat16()
    got = torch.empty(5, 32, dtype=torch.float32, device="cuda")
    rt.k.gemm(x, part, got, None, 2)
    ref = x.float().cpu().double() @ table[:32].double().T
    assert (got.cpu().double() - ref).abs().max() <= 1e-4 * max(1.0, float(ref.abs().max()))
    with pytest.raises(Exception):
        model.head.weight[:40]
