"""Every kernel instance that is compiled into the library is launched by a test and its result
checked: the products and the attention are templates of which a dispatch picks one by the sizes
of a call, and an instance that only a real model's sizes select would otherwise be unverified
arithmetic (the reference tests its products at model sizes for the same reason:
src/cuda/prefill.cu:1100 `gemv_ref`, src/model.rs:6238-6319).

Each case below names the instances it is meant to select, runs a call of such sizes, checks the
result (against a float64 product, or bit for bit against the unfused kernels, which other cases
check against float64), and asserts that those instances were what the library launched.  The
last test asserts that the cases together cover every instance the library says it contains: a
new instance without a case fails it."""
import math

import pytest
import torch

from axon_amd.kernels import MODE_ADD_F32, MODE_STORE, MODE_STORE_F32, MODE_SWIGLU, kernels
from gpu_helpers import paged_cache, tol
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

SEEN = {"bfloat16": set(), "float32": set()}
RAN = set()


def rnd(*shape, seed=0, scale=1.0, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn(*shape, generator=g, device=device) * scale


def launched(k, dtype, run):
    """What `run()` launched."""
    torch.cuda.synchronize()
    k.reset_instances()
    run()
    torch.cuda.synchronize()
    hit = set(k.instances(launched=True))
    SEEN[dtype] |= hit
    return hit


# --------------------------------------------------------------------------- the checks
def check_gemm(dtype, M, N, K, mode, bias=False):
    """out = epilogue(x w^T + bias) against the float64 product of the rounded operands (on the
    device: the matrices of a real vocabulary are large), and, for packed matrices, the first rows
    bit for bit as a step of those rows alone gives them."""
    k = kernels(dtype)
    td = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    x = rnd(M, K, seed=1, device="cuda").to(td)
    rows_w = 2 * N if mode == MODE_SWIGLU else N
    w = rnd(rows_w, K, seed=2, scale=0.2, device="cuda").to(td)
    b = rnd(N, seed=3, device="cuda") if bias else None
    wp = k.prepare_weight(w, mode == MODE_SWIGLU)
    prod = x.double() @ w.double().T
    if mode == MODE_SWIGLU:
        g, u = prod[:, :N], prod[:, N:]
        want = g / (1 + torch.exp(-g)) * u
    else:
        want = prod if b is None else prod + b.double()
    base = rnd(M, N, seed=4, device="cuda")
    out_dt = td if mode in (MODE_STORE, MODE_SWIGLU) else torch.float32

    def run(m):
        out = base[:m].clone().to(out_dt)
        k.gemm(x[:m], wp, out, b, mode)
        return out
    got = {}
    hit = launched(k, dtype, lambda: got.setdefault("out", run(M)))
    out = got["out"].double()
    if mode == MODE_ADD_F32:
        out = out - base.double()
    loose = mode in (MODE_STORE, MODE_SWIGLU)
    scale = max(1.0, float(want.abs().max()))
    limit = (1e-2 if loose else 2e-5 * math.sqrt(K)) * scale if dtype == "bfloat16" else 2e-6 * math.sqrt(K) * scale
    assert float((out - want).abs().max()) <= limit, (M, N, K, mode)
    for m in sorted({1, min(M, 9), min(M, 17), min(M, 65)}):            # a row's bits do not depend on the step
        assert torch.equal(run(m), got["out"][:m]), (M, N, K, mode, m)
    return hit


def check_then_norm(M, H, F):
    """The product that adds into the rows with the norm behind it written by the kernel that adds
    the segments' sums: bit for bit the product and the norm one after the other."""
    k = kernels("bfloat16")
    a = rnd(M, F, seed=5, device="cuda").bfloat16()
    w = k.prepare_weight(rnd(H, F, seed=6, scale=0.3, device="cuda").bfloat16())
    res = rnd(M, H, seed=7, scale=2.0, device="cuda")
    gain = (1.0 + 0.3 * rnd(H, seed=8, device="cuda")).bfloat16()
    x1 = res.clone()
    k.gemm(a, w, x1, None, MODE_ADD_F32)
    h1 = k.rmsnorm(x1, gain, 1e-5, torch.empty(M, H, dtype=torch.bfloat16, device="cuda"))
    x2, h2 = res.clone(), torch.zeros(M, H, dtype=torch.bfloat16, device="cuda")
    hit = launched(k, "bfloat16", lambda: k.gemm(a, w, x2, None, MODE_ADD_F32, following_norm=(gain, h2, 1e-5)))
    assert torch.equal(x1, x2) and torch.equal(h1, h2)
    return hit


def _qkv_case(M, nh, nkv, hd, hidden, page, seed):
    k = kernels("bfloat16")
    width = (nh + 2 * nkv) * hd
    w = k.pack_matrix(rnd(width, hidden, seed=seed, scale=0.2, device="cuda").bfloat16())
    bias = rnd(width, seed=seed + 1, device="cuda")
    g = torch.Generator().manual_seed(seed + 2)
    n_pages, max_pages = 3 * -(-(M + 8) // page) + 2, -(-(M + 8) // page)
    slots = torch.randperm(3 * max_pages * page, generator=g)[:M]
    seq = (slots // (max_pages * page)).to(torch.int32).cuda()
    pos = (slots % (max_pages * page)).to(torch.int32).cuda()
    pages = torch.randperm(n_pages, generator=g)[:3 * max_pages].view(3, max_pages).to(torch.int32).cuda()
    table = torch.empty(M, hd // 2, 2, dtype=torch.float32, device="cuda")
    k.rope_table(pos, P.rope_freqs(hd, 10000.0).cuda(), table)

    def fresh():
        return (torch.zeros(M, width, dtype=torch.bfloat16, device="cuda"),
                torch.full((n_pages, nkv, page, hd), 7.0, dtype=torch.bfloat16, device="cuda"),
                torch.full((n_pages, nkv, hd, page), 7.0, dtype=torch.bfloat16, device="cuda"))
    return k, w, bias, seq, pos, pages, table, fresh


def check_qkv_rope(M, nh, nkv, hd, hidden, page):
    """The [q; k; v] product with bias, rotation and the store into the pages in its own launches
    against the plain product followed by the rotary kernel: the same bits."""
    k, w, bias, seq, pos, pages, table, fresh = _qkv_case(M, nh, nkv, hd, hidden, page, 20)
    x = rnd(M, hidden, seed=19, device="cuda").bfloat16()
    q1, k1, v1 = fresh()
    k.gemm(x, w, q1, bias, MODE_STORE)
    k.rope_kv_write(q1, table, pos, seq, pages, k1, v1, nh, nkv, hd, hd, page, True)
    q2, k2, v2 = fresh()
    hit = launched(k, "bfloat16", lambda: k.gemm_qkv_rope(x, w, bias, q2, table, pos, seq, pages, k2, v2, nh, nkv, hd, page))
    assert torch.equal(q1[:, :nh * hd], q2[:, :nh * hd]) and torch.equal(k1, k2) and torch.equal(v1, v2)
    return hit


def check_normed_qkv(M, nh, nkv, hd, hidden, page):
    """The same with the RMS norm of the operand inside, against the norm kernel before it."""
    k, w, bias, seq, pos, pages, table, fresh = _qkv_case(M, nh, nkv, hd, hidden, page, 30)
    rows = rnd(M, hidden, seed=29, scale=2.0, device="cuda")
    gain = (1.0 + rnd(hidden, seed=28, device="cuda")).bfloat16()
    assert k.gemm_normed_ok(M, (nh + 2 * nkv) * hd, hidden)
    x = k.rmsnorm(rows, gain, 1e-6, torch.empty(M, hidden, dtype=torch.bfloat16, device="cuda"))
    q1, k1, v1 = fresh()
    k.gemm_qkv_rope(x, w, bias, q1, table, pos, seq, pages, k1, v1, nh, nkv, hd, page)
    q2, k2, v2 = fresh()
    hit = launched(k, "bfloat16", lambda: k.gemm_normed_qkv_rope(rows, gain, 1e-6, w, bias, q2, table, pos, seq, pages, k2, v2,
                                                                  nh, nkv, hd, page))
    assert torch.equal(q1[:, :nh * hd], q2[:, :nh * hd]) and torch.equal(k1, k2) and torch.equal(v1, v2)
    return hit


def check_normed_glu(M, hidden, ffn):
    """The gated product with the RMS norm of its operand inside, against the norm kernel followed by
    the gated product: the same bits."""
    k = kernels("bfloat16")
    assert k.gemm_normed_ok(M, ffn, hidden, gated=True)
    rows = rnd(M, hidden, seed=40, scale=3.0, device="cuda")
    gain = (1.0 + rnd(hidden, seed=41, device="cuda")).bfloat16()
    w = k.pack_matrix(rnd(2 * ffn, hidden, seed=42, scale=0.2, device="cuda").bfloat16())
    x = k.rmsnorm(rows, gain, 1e-5, torch.empty(M, hidden, dtype=torch.bfloat16, device="cuda"))
    want = torch.empty(M, ffn, dtype=torch.bfloat16, device="cuda")
    k.gemm(x, w, want, None, MODE_SWIGLU)
    got = torch.zeros(M, ffn, dtype=torch.bfloat16, device="cuda")
    hit = launched(k, "bfloat16", lambda: k.gemm_normed_glu(rows, gain, 1e-5, w, got))
    assert torch.equal(got, want)
    return hit


def _attention_case(nh, nkv, hd, page, T, window, dtype="bfloat16"):
    td = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    q, kk, vv = (rnd(T, n, hd, seed=s).to(td) for n, s in ((nh, 51), (nkv, 52), (nkv, 53)))
    kc, vc, table = paged_cache(kk.double(), vv.double(), page, dtype, seed=3)
    ref = P.causal_attention(q.double(), kk.double(), vv.double(), window).view(T, nh * hd)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    return q.cuda().view(T, nh * hd), kc, vc, table, pos, torch.zeros(T, dtype=torch.int32).cuda(), ref


def check_attention_rows(dtype, nh, nkv, hd, page, T, window):
    k = kernels(dtype)
    q, kc, vc, table, pos, rows, ref = _attention_case(nh, nkv, hd, page, T, window, dtype)
    out = torch.empty(T, nh * hd, dtype=q.dtype, device="cuda")
    hit = launched(k, dtype, lambda: k.attention(q, nh * hd, kc, vc, table, pos, rows, out, nh, nkv, hd, page, window,
                                                  1.0 / math.sqrt(hd)))
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 2e-6, 1e-2)
    # the last tokens alone (few tokens: eight waves each) give the bits they have among all of them
    few = min(T, 1023 // nh, 40)
    alone = torch.empty(few, nh * hd, dtype=q.dtype, device="cuda")
    k.attention(q[T - few:], nh * hd, kc, vc, table, pos[T - few:], rows[T - few:], alone, nh, nkv, hd, page, window,
                1.0 / math.sqrt(hd))
    assert torch.equal(alone, out[T - few:])
    return hit


def check_attention_mfma(nh, nkv, hd, page, T, window, every=1):
    """The prompt kernel over the whole sequence against the plain formula, and every position bit
    for bit as the decoding kernel gives it."""
    k = kernels("bfloat16")
    q, kc, vc, table, pos, rows, ref = _attention_case(nh, nkv, hd, page, T, window)
    scale = 1.0 / math.sqrt(hd)
    tiles = torch.tensor([(a, min(128, T - a)) for a in range(0, T, 128)], dtype=torch.int32).cuda()
    prompt = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    hit = launched(k, "bfloat16", lambda: k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, prompt, tiles, nh, nkv, hd,
                                                              page, window, scale))
    assert not torch.isnan(prompt).any()
    assert (prompt.cpu().double() - ref).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)
    # the decoding kernel for every `every`-th position and the edges of blocks and chunks
    picks = sorted(set(range(0, T, every)) | ({0, 1, 63, 64, 255, 256, 257, T - 2, T - 1} & set(range(T))))
    idx = torch.tensor(picks, dtype=torch.int32).cuda()
    ch = k.attention_decode_chunk
    chunks = max((p - ((max(0, p + 1 - window) if window else 0) // ch * ch)) // ch + 1 for p in picks)
    partial = torch.empty(k.attention_decode_workspace(len(picks), nh, hd, chunks), dtype=torch.float32, device="cuda")
    decoded = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    hit |= launched(k, "bfloat16", lambda: k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, decoded, idx, partial, chunks,
                                                               nh, nkv, hd, page, window, scale))
    assert torch.equal(decoded[picks], prompt[picks])
    return hit


def check_rmsnorm(dtype, dim):
    k = kernels(dtype)
    x = rnd(5, dim, seed=60, scale=3.0)
    gain = 1 + 0.3 * rnd(dim, seed=61)
    out = torch.empty(5, dim, dtype=k.dtype, device="cuda")
    hit = launched(k, dtype, lambda: k.rmsnorm(x.cuda(), gain.cuda(), 1e-5, out))
    ref = P.rms_norm(x.double(), gain.double(), 1e-5)
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 1e-6, 8e-3)
    return hit


# --------------------------------------------------------------------------- the cases
# (names of the instances the case is meant to select, the check, its arguments)
BF, F32 = "bfloat16", "float32"
CASES = [
    # 32-bit FMA products: the float32 build's, and the bfloat16 build's for what cannot be packed
    (F32, ["gemm_fma<16,0>"], check_gemm, (F32, 5, 100, 70, MODE_STORE_F32, True)),
    (F32, ["gemm_fma<64,0>"], check_gemm, (F32, 70, 259, 130, MODE_ADD_F32)),
    (F32, ["gemm_fma<16,1>"], check_gemm, (F32, 9, 96, 70, MODE_SWIGLU)),
    (F32, ["gemm_fma<64,1>"], check_gemm, (F32, 33, 48, 100, MODE_SWIGLU)),
    (BF, ["gemm_fma<16,0>"], check_gemm, (BF, 5, 100, 70, MODE_STORE, True)),
    (BF, ["gemm_fma<64,0>"], check_gemm, (BF, 70, 259, 130, MODE_STORE_F32)),
    (BF, ["gemm_fma<16,1>"], check_gemm, (BF, 9, 96, 70, MODE_SWIGLU)),
    (BF, ["gemm_fma<64,1>"], check_gemm, (BF, 33, 48, 100, MODE_SWIGLU)),
    (F32, ["rmsnorm<0>"], check_rmsnorm, (F32, 777)),
    (F32, ["rmsnorm<1>"], check_rmsnorm, (F32, 3584)),
    (BF, ["rmsnorm<0>"], check_rmsnorm, (BF, 777)),
    (BF, ["rmsnorm<1>"], check_rmsnorm, (BF, 3584)),
    # eight waves a (token, head) below 1,024 of them, one from there
    (F32, ["attention_rows<0,8>"], check_attention_rows, (F32, 6, 3, 80, 4, 65, 0)),
    (F32, ["attention_rows<0,1>"], check_attention_rows, (F32, 6, 3, 80, 4, 700, 0)),
    (BF, ["attention_rows<1,8>"], check_attention_rows, (BF, 4, 2, 32, 16, 133, 37)),
    (BF, ["attention_rows<1,1>"], check_attention_rows, (BF, 4, 2, 32, 16, 600, 37)),
    # up to 16 rows: a wave a segment of K.  One row tile a block below 16,384 rows of W, two from there
    (BF, ["gemm_stream<1,1,1,0>"], check_gemm, (BF, 3, 100, 128, MODE_STORE, True)),
    (BF, ["gemm_stream<1,1,2,0>"], check_gemm, (BF, 16, 100, 512, MODE_ADD_F32)),
    (BF, ["gemm_stream<1,1,4,0>"], check_gemm, (BF, 8, 3584, 3584, MODE_ADD_F32)),
    (BF, ["gemm_stream<2,1,1,0>"], check_gemm, (BF, 8, 16400, 256, MODE_STORE_F32)),
    (BF, ["gemm_stream<2,1,2,0>"], check_gemm, (BF, 16, 16400, 3584, MODE_STORE_F32)),
    (BF, ["gemm_stream<2,1,1,0>"], check_gemm, (BF, 8, 152064, 3584, MODE_STORE_F32)),      # the head of a real model
    (BF, ["gemm_stream<2,1,1,1>"], check_gemm, (BF, 9, 96, 64, MODE_SWIGLU)),
    (BF, ["gemm_stream<2,1,2,1>"], check_gemm, (BF, 1, 176, 512, MODE_SWIGLU)),
    (BF, ["gemm_stream<2,1,4,1>"], check_gemm, (BF, 16, 320, 1024, MODE_SWIGLU)),
    (BF, ["gemm_stream<2,1,1,2>"], check_qkv_rope, (5, 4, 1, 64, 256, 32)),
    (BF, ["gemm_stream<2,1,2,2>"], check_qkv_rope, (16, 6, 2, 64, 512, 16)),
    (BF, ["gemm_stream<2,1,4,2>"], check_qkv_rope, (8, 28, 4, 128, 3584, 64)),
    # up to 16 rows behind an RMS norm: the norm inside.  (pairs of tiles a wave, segments, epilogue,
    # rows of X in LDS, float4 of a row a lane holds)
    (BF, ["gemm_normed<1,1,1,8,16>"], check_normed_glu, (3, 256, 320)),
    (BF, ["gemm_normed<1,1,1,16,16>"], check_normed_glu, (13, 256, 320)),
    (BF, ["gemm_normed<1,1,1,8,20>"], check_normed_glu, (8, 4352, 12288)),
    (BF, ["gemm_normed<2,1,1,8,16>"], check_normed_glu, (6, 3584, 18944)),                    # a 7B layer's
    (BF, ["gemm_normed<2,1,1,16,16>"], check_normed_glu, (16, 256, 16400)),
    (BF, ["gemm_normed<2,1,1,8,20>"], check_normed_glu, (8, 5120, 27648)),                    # a 32B layer's
    (BF, ["gemm_normed<3,1,1,8,16>"], check_normed_glu, (8, 256, 32784)),
    (BF, ["gemm_normed<3,1,1,16,16>"], check_normed_glu, (9, 256, 32784)),
    (BF, ["gemm_normed<3,1,1,8,20>"], check_normed_glu, (2, 4352, 32784)),
    (BF, ["gemm_normed<1,2,1,8,16>"], check_normed_glu, (8, 512, 320)),
    (BF, ["gemm_normed<1,2,1,16,16>"], check_normed_glu, (16, 768, 4864)),
    (BF, ["gemm_normed<1,2,1,8,20>"], check_normed_glu, (5, 4352, 6144)),
    (BF, ["gemm_normed<2,2,1,8,16>"], check_normed_glu, (8, 512, 8208)),
    (BF, ["gemm_normed<2,2,1,16,16>"], check_normed_glu, (12, 1024, 8208)),
    (BF, ["gemm_normed<2,2,1,8,20>"], check_normed_glu, (7, 5120, 8208)),
    (BF, ["gemm_normed<1,4,1,8,16>"], check_normed_glu, (8, 3584, 2368)),
    (BF, ["gemm_normed<1,4,1,16,16>"], check_normed_glu, (15, 4096, 640)),
    (BF, ["gemm_normed<1,4,1,8,20>"], check_normed_glu, (8, 5120, 1728)),
    (BF, ["gemm_normed<2,4,1,8,16>"], check_normed_glu, (1, 1024, 4112)),
    (BF, ["gemm_normed<2,4,1,16,16>"], check_normed_glu, (10, 1024, 4112)),
    (BF, ["gemm_normed<2,4,1,8,20>"], check_normed_glu, (4, 4352, 4112)),
    (BF, ["gemm_normed<1,1,2,8,16>"], check_normed_qkv, (6, 7, 1, 128, 256, 8)),
    (BF, ["gemm_normed<1,1,2,16,16>"], check_normed_qkv, (11, 4, 2, 64, 256, 16)),
    (BF, ["gemm_normed<1,1,2,8,20>"], check_normed_qkv, (3, 160, 16, 128, 4352, 64)),
    (BF, ["gemm_normed<1,2,2,8,16>"], check_normed_qkv, (7, 3, 3, 96, 512, 4)),
    (BF, ["gemm_normed<1,2,2,16,16>"], check_normed_qkv, (16, 6, 2, 64, 512, 16)),
    (BF, ["gemm_normed<1,2,2,8,20>"], check_normed_qkv, (8, 80, 8, 128, 4352, 64)),
    (BF, ["gemm_normed<1,4,2,8,16>"], check_normed_qkv, (8, 28, 4, 128, 3584, 64)),           # a 7B layer's
    (BF, ["gemm_normed<1,4,2,16,16>"], check_normed_qkv, (12, 28, 4, 128, 3584, 16)),
    (BF, ["gemm_normed<1,4,2,8,20>"], check_normed_qkv, (8, 40, 8, 128, 5120, 64)),           # a 14B layer's
    # 17 to 64 rows: W streamed, X shared through LDS; as many waves a block as give each CU a block.
    # With several segments the sums go through the workspace (gemm_split_reduce<0>).
    (BF, ["gemm_rows<1,4,2,0>"], check_gemm, (BF, 17, 100, 128, MODE_STORE, True)),
    (BF, ["gemm_rows<1,4,3,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 33, 4100, 512, MODE_STORE_F32, True)),
    (BF, ["gemm_rows<1,4,4,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 64, 3584, 1024, MODE_ADD_F32)),
    (BF, ["gemm_rows<1,4,5,0>"], check_gemm, (BF, 40, 4100, 1024, MODE_STORE)),
    (BF, ["gemm_rows<1,4,6,0>"], check_gemm, (BF, 20, 5600, 1024, MODE_STORE_F32)),
    (BF, ["gemm_rows<1,4,7,0>"], check_gemm, (BF, 64, 6400, 1024, MODE_ADD_F32, True)),
    (BF, ["gemm_rows<1,4,8,0>"], check_gemm, (BF, 48, 9600, 1024, MODE_STORE)),
    (BF, ["gemm_rows<2,4,2,0>"], check_gemm, (BF, 17, 16384, 256, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,4,3,0>"], check_gemm, (BF, 64, 16400, 256, MODE_STORE_F32, True)),
    (BF, ["gemm_rows<2,4,4,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 32, 16384, 512, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,4,5,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 17, 16400, 3584, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,4,6,0>"], check_gemm, (BF, 64, 20500, 512, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,4,7,0>"], check_gemm, (BF, 33, 50000, 256, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,4,8,0>"], check_gemm, (BF, 64, 152064, 3584, MODE_STORE_F32)),          # the head of a real model
    (BF, ["gemm_rows<2,4,2,1>"], check_gemm, (BF, 40, 96, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,4,3,1>"], check_gemm, (BF, 17, 8208, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,4,4,1>", "gemm_split_reduce<0>"], check_gemm, (BF, 64, 3584, 1024, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,4,5,1>"], check_gemm, (BF, 64, 18944, 3584, MODE_SWIGLU)),              # a 7B layer's
    (BF, ["gemm_rows<2,4,6,1>"], check_gemm, (BF, 33, 5600, 1024, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,4,7,1>"], check_gemm, (BF, 20, 24592, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,4,8,1>"], check_gemm, (BF, 64, 28688, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<1,4,2,0>", "gemm_split_reduce<3>"], check_gemm, (BF, 48, 130, 1024, MODE_STORE_F32, True)),   # N % 4 != 0
    (BF, ["gemm_rows<1,4,4,0>", "gemm_split_reduce<1>"], check_then_norm, (64, 3584, 1024)),
    (BF, ["gemm_rows<1,4,5,0>", "gemm_split_reduce<2>"], check_qkv_rope, (64, 28, 4, 128, 3584, 64)),
    # 65 to 128 rows: the same kernel with eight tiles of 16 rows of X a step
    (BF, ["gemm_rows<1,8,3,0>"], check_gemm, (BF, 65, 100, 128, MODE_STORE, True)),
    (BF, ["gemm_rows<1,8,3,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 97, 4100, 512, MODE_STORE_F32, True)),
    (BF, ["gemm_rows<1,8,4,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 128, 3584, 1024, MODE_ADD_F32)),
    (BF, ["gemm_rows<1,8,5,0>"], check_gemm, (BF, 100, 4100, 1024, MODE_STORE)),
    (BF, ["gemm_rows<1,8,6,0>"], check_gemm, (BF, 80, 5600, 1024, MODE_STORE_F32)),
    (BF, ["gemm_rows<1,8,7,0>"], check_gemm, (BF, 128, 6400, 1024, MODE_ADD_F32, True)),
    (BF, ["gemm_rows<1,8,8,0>"], check_gemm, (BF, 112, 9600, 1024, MODE_STORE)),
    (BF, ["gemm_rows<2,8,3,0>"], check_gemm, (BF, 65, 16384, 256, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,3,0>"], check_gemm, (BF, 128, 16400, 256, MODE_STORE_F32, True)),
    (BF, ["gemm_rows<2,8,4,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 96, 16384, 512, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,5,0>", "gemm_split_reduce<0>"], check_gemm, (BF, 66, 16400, 3584, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,6,0>"], check_gemm, (BF, 128, 20500, 512, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,7,0>"], check_gemm, (BF, 97, 50000, 256, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,8,0>"], check_gemm, (BF, 127, 152064, 3584, MODE_STORE_F32)),
    (BF, ["gemm_rows<2,8,3,1>"], check_gemm, (BF, 100, 96, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,3,1>"], check_gemm, (BF, 65, 8208, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,4,1>", "gemm_split_reduce<0>"], check_gemm, (BF, 128, 3584, 1024, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,5,1>"], check_gemm, (BF, 128, 18944, 3584, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,6,1>"], check_gemm, (BF, 97, 5600, 1024, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,7,1>"], check_gemm, (BF, 80, 24592, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<2,8,8,1>"], check_gemm, (BF, 128, 28688, 64, MODE_SWIGLU)),
    (BF, ["gemm_rows<1,8,3,0>", "gemm_split_reduce<3>"], check_gemm, (BF, 112, 130, 1024, MODE_STORE_F32, True)),   # N % 4 != 0
    (BF, ["gemm_rows<1,8,4,0>", "gemm_split_reduce<1>"], check_then_norm, (128, 3584, 1024)),
    (BF, ["gemm_rows<1,8,5,0>", "gemm_split_reduce<2>"], check_qkv_rope, (128, 28, 4, 128, 3584, 64)),
    # more than 128 rows: tiles of the output through LDS
    # (129 to 256 rows in no more blocks than CUs: four stages)
    (BF, ["gemm_tile<128,128,2,2,0,4>", "gemm_split_reduce<0>"], check_gemm, (BF, 140, 132, 2048, MODE_STORE, True)),
    (BF, ["gemm_tile<128,128,2,2,0,4>", "gemm_split_reduce<3>"], check_gemm, (BF, 200, 130, 1024, MODE_ADD_F32)),
    (BF, ["gemm_tile<128,128,2,2,1,4>", "gemm_split_reduce<0>"], check_gemm, (BF, 130, 96, 2048, MODE_SWIGLU)),
    (BF, ["gemm_tile<128,128,2,2,0,4>", "gemm_split_reduce<0>"], check_gemm, (BF, 256, 3584, 18944, MODE_ADD_F32)),  # a 7B layer's
    (BF, ["gemm_tile<128,128,2,2,0,2>", "gemm_split_reduce<0>"], check_gemm, (BF, 200, 4608, 3584, MODE_STORE, True)),
    (BF, ["gemm_tile<128,128,2,2,0,2>", "gemm_split_reduce<3>"], check_gemm, (BF, 300, 130, 1024, MODE_ADD_F32)),
    (BF, ["gemm_tile<128,128,2,2,1,2>", "gemm_split_reduce<0>"], check_gemm, (BF, 300, 96, 2048, MODE_SWIGLU)),
    (BF, ["gemm_tile<128,128,2,2,1,2>"], check_gemm, (BF, 200, 8320, 256, MODE_SWIGLU)),
    (BF, ["gemm_tile<256,192,4,2,0,2>"], check_gemm, (BF, 2048, 4608, 192, MODE_STORE, True)),
    (BF, ["gemm_tile<256,256,4,2,0,2>"], check_gemm, (BF, 1100, 9300, 128, MODE_STORE_F32)),
    (BF, ["gemm_tile<256,256,4,2,0,2>", "gemm_split_reduce<0>"], check_gemm, (BF, 2049, 3584, 3584, MODE_ADD_F32)),
    (BF, ["gemm_tile<256,256,4,2,1,2>"], check_gemm, (BF, 2048, 2608, 64, MODE_SWIGLU)),
    (BF, ["gemm_tile<128,128,2,2,0,4>", "gemm_split_reduce<1>"], check_then_norm, (150, 256, 1024)),
    (BF, ["gemm_tile<256,256,4,2,1,2>"], check_gemm, (BF, 200, 18944, 3584, MODE_SWIGLU)),              # a 7B layer's at 200 rows
    (BF, ["gemm_tile<256,256,4,2,0,2>", "gemm_split_reduce<2>"], check_qkv_rope, (2048, 28, 4, 128, 3584, 64)),
    # attention on the matrix cores: (head size, query heads a block, pages of 64 positions or more)
    # and (head size, waves a block) (one wave a block in the decoding kernel up to 2,560 blocks of
    # positions, four beyond; two heads a block in the prompt kernel where tiles x heads are more
    # than 256: the long prompts of real models)
    (BF, ["attention_prefill<64,1,0>", "attention_decode<64,1>"], check_attention_mfma, (4, 2, 64, 16, 200, 0)),
    (BF, ["attention_prefill<64,1,1>"], check_attention_mfma, (4, 2, 64, 64, 200, 0)),
    (BF, ["attention_prefill<128,1,1>", "attention_decode<128,1>"], check_attention_mfma, (7, 1, 128, 64, 333, 90)),
    (BF, ["attention_prefill<128,1,0>"], check_attention_mfma, (7, 1, 128, 16, 333, 90)),
    (BF, ["attention_prefill<64,2,1>", "attention_decode<64,4>"], check_attention_mfma, (32, 1, 64, 64, 1700, 0, 5)),
    (BF, ["attention_prefill<64,2,0>"], check_attention_mfma, (64, 2, 64, 16, 800, 0, 3)),
    (BF, ["attention_prefill<128,2,0>", "attention_decode<128,4>"], check_attention_mfma, (14, 2, 128, 16, 3400, 0, 37)),
    (BF, ["attention_prefill<128,2,1>"], check_attention_mfma, (64, 2, 128, 64, 800, 300, 3)),
]
IDS = [f"{dtype[:2]}-{'+'.join(names)}-{i}" for i, (dtype, names, _, _) in enumerate(CASES)]


def run_case(i):
    dtype, names, check, args = CASES[i]
    hit = check(*args)
    RAN.add(i)
    assert set(names) <= hit, f"meant to select {names}, the library launched {sorted(hit)}"
    torch.cuda.empty_cache()


@pytest.mark.parametrize("i", range(len(CASES)), ids=IDS)
def test_the_instance_a_call_selects_gives_the_right_result(i):
    run_case(i)


def test_every_compiled_instance_was_launched_and_checked():
    for i in range(len(CASES)):            # run alone, this test runs the cases itself
        if i not in RAN:
            run_case(i)
    for dtype in (BF, F32):
        known = set(kernels(dtype).instances())
        named = {n for d, names, _, _ in CASES if d == dtype for n in names}
        assert known <= named, f"{dtype}: no case selects {sorted(known - named)}"
        assert known <= SEEN[dtype], f"{dtype}: never launched: {sorted(known - SEEN[dtype])}"
