"""Each kernel alone against its plain reference, at other sizes than the engine's tests use,
in float32 and in bfloat16.  Where random inputs would hide a fault (a far key among hundreds,
a window's edge, a page's edge) the inputs are made so that it shows."""
import math

import pytest
import torch

from axon_amd.kernels import MODE_ADD_F32, MODE_STORE, MODE_STORE_F32, MODE_SWIGLU, KernelError, kernels
from gpu_helpers import DTYPES, TORCH, paged_cache, tol
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def as_dtype(x, dtype):
    """Round to the compute dtype and return (device tensor, float64 copy of the rounded values)."""
    d = x.to(TORCH[dtype])
    return d.cuda(), d.double()


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    k = kernels(dtype)
    table, ref = as_dtype(rnd(37, 100), dtype)
    tokens = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32).cuda()
    out = torch.empty(5, 100, dtype=torch.float32, device="cuda")
    k.embed(tokens, table, out)
    assert torch.equal(out.cpu().double(), ref[tokens.cpu().long()])          # exact: a widening copy


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,eps", [(100, 1e-6), (777, 0.5), (3584, 1e-5), (8, 1e-3)])
def test_rmsnorm(dtype, dim, eps):
    k = kernels(dtype)
    x = rnd(6, dim, seed=1, scale=3.0)
    for gdt in (torch.float32, torch.bfloat16):                                # a gain keeps its stored precision
        gain = (1 + 0.3 * rnd(dim, seed=2)).to(gdt)
        out = torch.empty(6, dim, dtype=TORCH[dtype], device="cuda")
        k.rmsnorm(x.cuda(), gain.cuda(), eps, out)
        ref = P.rms_norm(x.double(), gain.double(), eps)
        assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 1e-6, 8e-3)
    rows = torch.tensor([4, 0, 4], dtype=torch.int32).cuda()                   # gathered rows (the wanted places)
    out = torch.empty(3, dim, dtype=TORCH[dtype], device="cuda")
    k.rmsnorm(x.cuda(), gain.cuda(), eps, out, rows)
    ref = P.rms_norm(x[[4, 0, 4]].double(), gain.double(), eps)
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 1e-6, 8e-3)


def test_rope_table_is_float64_accurate():
    k = kernels("float32")
    pos = torch.tensor([0, 1, 2, 77, 4095, 32767, 131071], dtype=torch.int32)
    for hd, theta in [(16, 1e4), (128, 1e6), (80, 5e4)]:
        freqs = P.rope_freqs(hd, theta)
        out = torch.empty(len(pos), hd // 2, 2, dtype=torch.float32, device="cuda")
        k.rope_table(pos.cuda(), freqs.cuda(), out)
        sin, cos = P.rope_table(pos, freqs)
        assert (out[..., 0].cpu().double() - sin).abs().max() < 1e-7           # float32 rounding of a float64 value
        assert (out[..., 1].cpu().double() - cos).abs().max() < 1e-7
        assert torch.equal(out[0, :, 0].cpu(), torch.zeros(hd // 2)) and torch.equal(out[0, :, 1].cpu(), torch.ones(hd // 2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,page", [(4, 2, 16, 8), (3, 1, 32, 16), (6, 3, 80, 4), (7, 7, 48, 5), (28, 4, 128, 16)])
def test_rope_and_cache_store(dtype, nh, nkv, hd, page):
    k = kernels(dtype)
    T = 11
    qkv, ref = as_dtype(rnd(T, (nh + 2 * nkv) * hd, seed=3), dtype)
    pos = torch.tensor([5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15], dtype=torch.int32)
    rows = torch.zeros(T, dtype=torch.int32)
    n_pages = 9
    table = torch.tensor([[7, 2, 5, 0, 3, 1, 8, 4]], dtype=torch.int32)       # scattered pages
    kc = torch.zeros(n_pages, nkv, page, hd, dtype=TORCH[dtype], device="cuda")
    vc = torch.zeros(n_pages, nkv, hd, page, dtype=TORCH[dtype], device="cuda")
    freqs = P.rope_freqs(hd, 1e4)
    tab = torch.empty(T, hd // 2, 2, dtype=torch.float32, device="cuda")
    k.rope_table(pos.cuda(), freqs.cuda(), tab)
    k.rope_kv_write(qkv, tab, pos.cuda(), rows.cuda(), table.cuda(), kc, vc, nh, nkv, hd, hd, page)
    sin, cos = P.rope_table(pos, freqs)
    q_ref = P.apply_rope(ref[:, :nh * hd].view(T, nh, hd), sin, cos)
    k_ref = P.apply_rope(ref[:, nh * hd:(nh + nkv) * hd].view(T, nkv, hd), sin, cos)
    v_ref = ref[:, (nh + nkv) * hd:].view(T, nkv, hd)
    t = tol(dtype, q_ref, 1e-6, 8e-3)
    assert (qkv[:, :nh * hd].cpu().double().view(T, nh, hd) - q_ref).abs().max() <= t
    for i, p in enumerate(pos.tolist()):
        pg, o = int(table[0, p // page]), p % page
        assert (kc[pg, :, o].cpu().double() - k_ref[i]).abs().max() <= t
        assert torch.equal(vc[pg, :, :, o].cpu().double(), v_ref[i])           # values are stored as they are
    written = sum(1 for _ in pos)
    assert int((vc.abs().sum(dim=(1, 2)) > 0).sum()) == written                # nothing else was touched


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,page,T,window", [
    (4, 2, 16, 8, 70, 0), (3, 1, 32, 16, 133, 0), (6, 3, 80, 4, 65, 0), (8, 2, 128, 16, 200, 0), (4, 4, 64, 64, 130, 0),
    (4, 2, 16, 8, 150, 37), (2, 1, 48, 5, 129, 64), (5, 5, 256, 16, 40, 0)])
def test_attention_over_the_paged_cache(dtype, nh, nkv, hd, page, T, window):
    k = kernels(dtype)
    q, qr = as_dtype(rnd(T, nh, hd, seed=4), dtype)
    kk, kr = as_dtype(rnd(T, nkv, hd, seed=5), dtype)
    vv, vr = as_dtype(rnd(T, nkv, hd, seed=6), dtype)
    kc, vc, table = paged_cache(kr, vr, page, dtype)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    out = torch.empty(T, nh * hd, dtype=TORCH[dtype], device="cuda")
    k.attention(q.view(T, nh * hd), nh * hd, kc, vc, table, pos, rows, out, nh, nkv, hd, page, window,
                1.0 / math.sqrt(hd))
    ref = P.causal_attention(qr, kr, vr, window).view(T, nh * hd)
    assert not torch.isnan(out).any()                                          # rows past a token's position hold NaN
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 2e-6, 1e-2)
    # a decode row alone (one token at the last position, queried out of order) is the same row
    last = torch.tensor([T - 1], dtype=torch.int32).cuda()
    one = torch.empty(1, nh * hd, dtype=TORCH[dtype], device="cuda")
    k.attention(q[T - 1:].view(1, nh * hd), nh * hd, kc, vc, table, last, rows[:1], one, nh, nkv, hd, page, window,
                1.0 / math.sqrt(hd))
    assert torch.equal(one[0], out[T - 1])
    # pages of another size, one that goes through LDS in whole loads if this one does not (a
    # multiple of 4 positions does) and vice versa: the same bits
    other = page + 1 if page % 4 == 0 else 4 * page
    kc2, vc2, table2 = paged_cache(kr, vr, other, dtype)
    out2 = torch.empty_like(out)
    k.attention(q.view(T, nh * hd), nh * hd, kc2, vc2, table2, pos, rows, out2, nh, nkv, hd, other, window,
                1.0 / math.sqrt(hd))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key_and_respects_the_windows_edge(dtype):
    k = kernels(dtype)
    nh, nkv, hd, page, T = 4, 2, 32, 16, 700
    q = rnd(T, nh, hd, seed=7) * 0.1
    kk = rnd(T, nkv, hd, seed=8) * 0.1
    vv = rnd(T, nkv, hd, seed=9)
    far = 15                                              # the last slot of the first page, hundreds of keys away
    kk[far, 1] = 0
    kk[far, 1, 3] = 40.0
    q[T - 1, 2] = 0
    q[T - 1, 2, 3] = 40.0                                 # head 2 reads kv head 1: score 1600 / sqrt(32) stands out
    qd, qr = as_dtype(q, dtype)
    _, kr = as_dtype(kk, dtype)
    _, vr = as_dtype(vv, dtype)
    kc, vc, table = paged_cache(kr, vr, page, dtype)
    pos = torch.tensor([T - 1], dtype=torch.int32).cuda()
    rows = torch.zeros(1, dtype=torch.int32).cuda()
    out = torch.empty(1, nh * hd, dtype=TORCH[dtype], device="cuda")
    scale = 1.0 / math.sqrt(hd)
    k.attention(qd[T - 1:].view(1, -1), nh * hd, kc, vc, table, pos, rows, out, nh, nkv, hd, page, 0, scale)
    got = out.cpu().double().view(nh, hd)
    assert (got[2] - vr[far, 1]).abs().max() < 1e-2       # all the weight is on the far key
    ref = P.causal_attention(qr, kr, vr)[T - 1]
    assert (got - ref).abs().max() <= tol(dtype, ref, 2e-6, 1e-2)
    # the window's edge: with window w the token at T-1 sees T-w .. T-1.  Put the loud key just
    # outside, then just inside.
    for w, seen in ((T - 1 - far, False), (T - far, True)):
        k.attention(qd[T - 1:].view(1, -1), nh * hd, kc, vc, table, pos, rows, out, nh, nkv, hd, page, w, scale)
        got = out.cpu().double().view(nh, hd)
        ref = P.causal_attention(qr, kr, vr, w)[T - 1]
        assert (got - ref).abs().max() <= tol(dtype, ref, 2e-6, 1e-2)
        assert ((got[2] - vr[far, 1]).abs().max() < 1e-2) == seen


def packed(k, w, gated=False):
    """The matrix as a model's weights reach the products: packed for the matrix cores where it can
    be (never in the float32 build), else row-major."""
    return k.prepare_weight(w, gated)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (3, 100, 70), (17, 259, 130), (70, 96, 33), (130, 48, 257),
                                   (5, 1000, 512), (64, 256, 256), (200, 384, 1024), (33, 152, 3584), (64, 1000, 2048),
                                   (20, 8200, 512), (48, 130, 1024), (100, 132, 2048), (256, 260, 1024),
                                   (2048, 4608, 192), (1100, 9300, 128), (700, 260, 8192)])
def test_gemm_every_epilogue(dtype, M, N, K):
    k = kernels(dtype)
    x, xr = as_dtype(rnd(M, K, seed=10), dtype)
    w, wr = as_dtype(rnd(N, K, seed=11, scale=0.2), dtype)
    w = packed(k, w)
    ref = xr @ wr.T
    for bias_dt in (None, torch.float32, torch.bfloat16):
        bias = None if bias_dt is None else rnd(N, seed=12).to(bias_dt)
        want = ref if bias is None else ref + bias.double()
        b = None if bias is None else bias.cuda()
        out = torch.empty(M, N, dtype=TORCH[dtype], device="cuda")
        k.gemm(x, w, out, b, MODE_STORE)
        assert (out.cpu().double() - want).abs().max() <= tol(dtype, want, 2e-6 * math.sqrt(K), 1e-2)
        f32 = torch.empty(M, N, dtype=torch.float32, device="cuda")
        k.gemm(x, w, f32, b, MODE_STORE_F32)
        assert (f32.cpu().double() - want).abs().max() <= tol(dtype, want, 2e-6 * math.sqrt(K), 2e-5 * math.sqrt(K))
        res = rnd(M, N, seed=13).cuda()
        acc = res.clone()
        k.gemm(x, w, acc, b, MODE_ADD_F32)
        assert (acc.cpu().double() - (want + res.cpu().double())).abs().max() <= tol(dtype, want, 2e-6 * math.sqrt(K),
                                                                                      2e-5 * math.sqrt(K))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,F,K", [(1, 96, 64), (9, 176, 64), (40, 320, 192), (64, 130, 128), (70, 300, 128),
                                   (300, 512, 256), (600, 1000, 128), (5, 100, 70), (33, 19, 33), (2100, 384, 64),
                                   (40, 320, 1024), (17, 132, 2048), (64, 96, 4096), (130, 96, 2048), (2048, 2600, 64)])
def test_gemm_with_the_gated_epilogue(dtype, M, F, K):
    """One product over [gate; up] whose epilogue is silu(gate) * up."""
    k = kernels(dtype)
    x, xr = as_dtype(rnd(M, K, seed=30), dtype)
    w, wr = as_dtype(rnd(2 * F, K, seed=31, scale=0.3), dtype)
    w = packed(k, w, gated=True)
    out = torch.empty(M, F, dtype=TORCH[dtype], device="cuda")
    k.gemm(x, w, out, None, MODE_SWIGLU)
    ref = P.swiglu(xr @ wr[:F].T, xr @ wr[F:].T)
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 2e-6 * math.sqrt(K), 1e-2)
    with pytest.raises(KernelError):
        k.gemm(x, w, out, rnd(F).cuda(), MODE_SWIGLU)


ROW_COUNTS = (1, 2, 3, 7, 16, 17, 32, 33, 64, 65, 128, 130, 256, 257, 1000, 2049)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_rows_do_not_depend_on_the_batch(dtype):
    """The same row of x gives the same bits whatever rows ride along, in both builds and for any
    number of rows (src/lm.rs:272-278): every kernel a product may meet adds in the one order its
    matrix fixes."""
    k = kernels(dtype)
    # the last three: blocks of 3, 6 and 8 waves in the kernel for 17 to 64 rows
    for N, K in [(96, 80), (256, 512), (130, 1000), (512, 1024), (300, 4096), (200, 8192), (4100, 256), (9600, 256),
                 (6144, 2048), (8192, 2048)]:
        x, _ = as_dtype(rnd(2100, K, seed=14), dtype)
        w, _ = as_dtype(rnd(N, K, seed=15, scale=0.2), dtype)
        w = packed(k, w)
        whole = torch.empty(2100, N, dtype=torch.float32, device="cuda")
        k.gemm(x, w, whole, None, MODE_STORE_F32)
        for m in ROW_COUNTS:
            part = torch.empty(m, N, dtype=torch.float32, device="cuda")
            k.gemm(x[:m], w, part, None, MODE_STORE_F32)
            assert torch.equal(part, whole[:m]), (N, K, m)


@pytest.mark.parametrize("N", [16400, 152064])
@pytest.mark.parametrize("K", [256, 3584])
def test_products_with_the_rows_of_a_real_vocabulary(N, K):
    """From 16,384 rows of W on the products for up to 16 rows and for 17 to 64 take two row tiles a
    wave: the head of every real model runs through those.  1 to 65 rows against the float64 product
    (computed on the device: W has up to a gigabyte), and a row bit for bit whatever its step."""
    k = kernels("bfloat16")
    g = torch.Generator(device="cuda").manual_seed(21)
    x = torch.randn(65, K, generator=g, device="cuda").bfloat16()
    w = (torch.randn(N, K, generator=g, device="cuda") * 0.05).bfloat16()
    want = x.double() @ w.double().T
    wp = k.prepare_weight(w)
    del w
    whole = torch.empty(65, N, dtype=torch.float32, device="cuda")
    k.gemm(x, wp, whole, None, MODE_STORE_F32)
    assert float((whole.double() - want).abs().max()) <= 2e-5 * math.sqrt(K) * max(1.0, float(want.abs().max()))
    for m in (1, 8, 16, 17, 64):
        part = torch.empty(m, N, dtype=torch.float32, device="cuda")
        k.gemm(x[:m], wp, part, None, MODE_STORE_F32)
        assert torch.equal(part, whole[:m]), (N, K, m)


# the products of a layer of the measured sizes (hidden, q rows, kv rows, feed-forward width, head_dim)
LAYER_SIZES = {"7b": (3584, 3584, 512, 18944, 128), "14b": (5120, 5120, 1024, 13824, 128)}


@pytest.mark.parametrize("sizes", sorted(LAYER_SIZES))
def test_products_of_the_measured_sizes_give_a_row_the_same_bits_in_any_step(sizes):
    """bfloat16, the matrices of a Qwen2.5-7B and a 14B layer, every epilogue the model uses: a
    row's result does not depend on the number of rows in the step, from 1 to 2,049."""
    k = kernels("bfloat16")
    hidden, q_dim, kv_dim, ffn, hd = LAYER_SIZES[sizes]
    most = max(ROW_COUNTS)
    cases = [("qkv", q_dim + 2 * kv_dim, hidden, MODE_STORE), ("o", hidden, q_dim, MODE_ADD_F32),
             ("gate_up", ffn, hidden, MODE_SWIGLU), ("down", hidden, ffn, MODE_ADD_F32), ("head", 4096 + 40, hidden, MODE_STORE_F32)]
    for name, N, K, mode in cases:
        x, _ = as_dtype(rnd(most, K, seed=16), "bfloat16")
        w, _ = as_dtype(rnd(2 * N if mode == MODE_SWIGLU else N, K, seed=17, scale=0.05), "bfloat16")
        w = packed(k, w, gated=mode == MODE_SWIGLU)
        assert k.gemm_segments(N, K, mode == MODE_SWIGLU) in (1, 2, 4, 8)
        bias = rnd(N, seed=18).cuda() if name == "qkv" else None
        dt = torch.float32 if mode in (MODE_ADD_F32, MODE_STORE_F32) else torch.bfloat16
        base = rnd(most, N, seed=19).to(dt).cuda()
        whole = base.clone()
        k.gemm(x, w, whole, bias, mode)
        for m in ROW_COUNTS:
            part = base[:m].clone()
            k.gemm(x[:m], w, part, bias, mode)
            assert torch.equal(part, whole[:m]), (sizes, name, m)


@pytest.mark.parametrize("M,H,F", [(65, 384, 2048), (100, 256, 1024), (256, 128, 512), (300, 256, 8192),
                                   (128, 4352, 512)])
def test_gemm_followed_by_the_whole_norm(M, H, F):
    """residual += a . Wo^T + bias; h = rmsnorm(residual) * gain, the norm written by the kernel
    that adds the sums of the product's segments: the same bits as the product and the norm one
    after the other, and right against the plain formulas.  Where no such kernel runs the
    product refuses."""
    k = kernels("bfloat16")
    eps = 2e-5
    assert k.gemm_then_norm_ok(M, H, F)
    a, ar = as_dtype(rnd(M, F, seed=50), "bfloat16")
    wo, wor = as_dtype(rnd(H, F, seed=51, scale=0.3), "bfloat16")
    w = packed(k, wo)
    res = rnd(M, H, seed=52, scale=2.0)
    res[M // 2] *= 40.0
    bias = rnd(H, seed=53)
    for gain_dt, b in ((torch.float32, None), (torch.bfloat16, bias.cuda())):
        gain = (1.0 + 0.3 * rnd(H, seed=54)).to(gain_dt).cuda()
        x1 = res.clone().cuda()
        k.gemm(a, w, x1, b, MODE_ADD_F32)
        h1 = k.rmsnorm(x1, gain, eps, torch.empty(M, H, dtype=torch.bfloat16, device="cuda"))
        x2 = res.clone().cuda()
        h2 = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device="cuda")
        k.gemm(a, w, x2, b, MODE_ADD_F32, following_norm=(gain, h2, eps))
        assert torch.equal(x1, x2) and torch.equal(h1, h2)
        x_ref = res.double() + ar @ wor.T + (0 if b is None else bias.double())
        h_ref = P.rms_norm(x_ref, gain.cpu().double(), eps)
        assert (h2.cpu().double() - h_ref).abs().max() <= tol("bfloat16", h_ref, bf16=1.5e-2)
        # and the rows are those of a step of eight
        x3 = res[:8].clone().cuda()
        k.gemm(a[:8], w, x3, b, MODE_ADD_F32)
        assert torch.equal(x3, x2[:8])
    assert not k.gemm_then_norm_ok(8, H, F) and not k.gemm_then_norm_ok(3000, 16384, F)
    with pytest.raises(KernelError):
        k.gemm(a[:8], w, res[:8].clone().cuda(), None, MODE_ADD_F32, following_norm=(gain, h2[:8], eps))


@pytest.mark.parametrize("M,nh,nkv,hd,hidden,page", [(1, 4, 2, 32, 64, 8), (8, 6, 2, 64, 192, 16), (16, 7, 1, 128, 256, 8),
                                                      (13, 3, 3, 96, 128, 4), (5, 4, 1, 64, 320, 32),
                                                      (16, 2, 2, 128, 64, 16), (40, 6, 2, 64, 512, 16),
                                                      (100, 7, 1, 128, 1024, 8), (300, 4, 2, 64, 3072, 16)])
def test_qkv_product_with_rotation_and_cache_store_in_one(M, nh, nkv, hd, hidden, page):
    """The fused launch against the product followed by the rotary kernel: the same bits in q, in
    the pages of keys and in the pages of values; other pages untouched."""
    k = kernels("bfloat16")
    width = (nh + 2 * nkv) * hd
    assert k.gemm_qkv_rope_ok(M, width, hidden, hd, hd) and k.gemm_qkv_rope_ok(M, nh * hd, hidden, hd, hd)
    assert not k.gemm_qkv_rope_ok(M, width, hidden, hd, hd // 2) and not k.gemm_qkv_rope_ok(100, width, 64, hd, hd)
    assert not k.gemm_qkv_rope_ok(M, 48 * (nh + 2 * nkv), hidden, 48, 48)
    assert not kernels("float32").gemm_qkv_rope_ok(M, width, hidden, hd, hd)
    x, _ = as_dtype(rnd(M, hidden, seed=50), "bfloat16")
    w, _ = as_dtype(rnd(width, hidden, seed=51, scale=0.2), "bfloat16")
    g = torch.Generator().manual_seed(52)
    # tokens of three requests at scattered positions, every (request, position) once
    n_pages, max_pages = 40, 8
    slots = torch.randperm(3 * max_pages * page, generator=g)[:M]
    rows = (slots // (max_pages * page)).to(torch.int32)
    pos = (slots % (max_pages * page)).to(torch.int32)
    table_of_pages = torch.randperm(n_pages, generator=g)[:3 * max_pages].view(3, max_pages).to(torch.int32).cuda()
    freqs = P.rope_freqs(hd, 10000.0).cuda()
    table = torch.empty(M, hd // 2, 2, dtype=torch.float32, device="cuda")
    k.rope_table(pos.cuda(), freqs, table)
    for bias_dt, write_kv in ((None, True), (torch.float32, True), (torch.bfloat16, False)):
        bias = None if bias_dt is None else rnd(width, seed=53).to(bias_dt).cuda()
        n_rows = width if write_kv else nh * hd
        ww, bb = k.pack_matrix(w[:n_rows].contiguous()), (None if bias is None else bias[:n_rows])
        got, want = [], []
        for fused in (True, False):
            kc = torch.full((n_pages, nkv, page, hd), 7.0, dtype=torch.bfloat16, device="cuda")
            vc = torch.full((n_pages, nkv, hd, page), 7.0, dtype=torch.bfloat16, device="cuda")
            qkv = torch.zeros(M, width, dtype=torch.bfloat16, device="cuda")
            if fused:
                k.gemm_qkv_rope(x, ww, bb, qkv, table, pos.cuda(), rows.cuda(), table_of_pages, kc, vc, nh, nkv, hd, page,
                                write_kv)
            else:
                k.gemm(x, ww, qkv[:, :n_rows], bb, MODE_STORE)
                k.rope_kv_write(qkv, table, pos.cuda(), rows.cuda(), table_of_pages, kc, vc, nh, nkv, hd, hd, page, write_kv)
            (got if fused else want).extend([qkv[:, :nh * hd].clone(), kc, vc])
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        assert write_kv == bool((got[1] != 7.0).any())


@pytest.mark.parametrize("M,hidden,ffn", [(1, 256, 32), (8, 3584, 4864), (3, 768, 320), (8, 256, 9600), (7, 1024, 8192),
                                          (8, 4096, 256), (5, 512, 4864), (2, 3584, 2368), (6, 3584, 18944), (9, 3584, 4864), (13, 768, 1280),
                                          (16, 3584, 2368), (16, 256, 9600), (15, 4096, 640), (8, 5120, 1728), (3, 4352, 320)])
def test_gated_product_with_the_norm_inside(M, hidden, ffn):
    """The norm worked out inside the product against the norm kernel followed by the product: the
    same bits (the norm is the norm kernel's arithmetic, the product's order of addition the same)."""
    k = kernels("bfloat16")
    assert k.gemm_normed_ok(M, ffn, hidden, gated=True)
    assert not k.gemm_normed_ok(17, ffn, hidden, gated=True) and not k.gemm_normed_ok(M, ffn, 8192, gated=True)
    assert k.gemm_normed_ok(8, ffn, 5120, gated=True) and not k.gemm_normed_ok(9, ffn, 5120, gated=True)   # wide rows: up to 8 of them
    assert not k.gemm_normed_ok(M, ffn, hidden + 64, gated=True)          # rows in whole rounds of 256 columns
    assert not kernels("float32").gemm_normed_ok(M, ffn, hidden, gated=True)
    rows = (rnd(M + 2, hidden + 8, seed=60) * 3.0).float().cuda()[1:M + 1, :hidden]      # strided rows
    gain = (1.0 + rnd(hidden, seed=61)).to(torch.bfloat16).cuda()
    assert not k.gemm_normed_ok(M, ffn, hidden, gated=True, gain=gain.float())          # the gain as it is stored: bfloat16
    w, _ = as_dtype(rnd(2 * ffn, hidden, seed=62, scale=0.2), "bfloat16")
    ww = k.pack_matrix(w)
    x = torch.empty(M, hidden, dtype=torch.bfloat16, device="cuda")
    k.rmsnorm(rows.contiguous(), gain, 1e-5, x)
    want = torch.empty(M, ffn, dtype=torch.bfloat16, device="cuda")
    k.gemm(x, ww, want, None, MODE_SWIGLU)
    got = torch.full((M + 1, ffn + 8), 7.0, dtype=torch.bfloat16, device="cuda")
    k.gemm_normed_glu(rows, gain, 1e-5, ww, got[:M, :ffn])
    assert torch.equal(got[:M, :ffn], want)
    assert (got[M] == 7.0).all() and (got[:, ffn:] == 7.0).all()
    with pytest.raises(KernelError):
        k.gemm_normed_glu(rows, gain.float(), 1e-5, ww, got[:M, :ffn])


@pytest.mark.parametrize("M,nh,nkv,hd,hidden,page", [(1, 4, 2, 32, 256, 8), (8, 28, 4, 128, 3584, 64), (6, 7, 1, 128, 256, 8),
                                                      (7, 3, 3, 96, 512, 4), (5, 4, 1, 64, 768, 32), (3, 14, 2, 64, 1024, 16),
                                                      (12, 28, 4, 128, 3584, 64), (16, 6, 2, 64, 512, 16), (8, 40, 8, 128, 5120, 64)])
def test_qkv_product_with_the_norm_inside(M, nh, nkv, hd, hidden, page):
    """As above for the [q; k; v] product with rotation and cache store: the same bits in q and in
    the pages as the norm kernel followed by `gemm_qkv_rope`."""
    k = kernels("bfloat16")
    width = (nh + 2 * nkv) * hd
    assert k.gemm_normed_ok(M, width, hidden)
    rows = (rnd(M, hidden, seed=70) * 2.0).float().cuda()
    gain = (1.0 + rnd(hidden, seed=71)).to(torch.bfloat16).cuda()
    w, _ = as_dtype(rnd(width, hidden, seed=72, scale=0.2), "bfloat16")
    g = torch.Generator().manual_seed(73)
    n_pages, max_pages = 40, 8
    slots = torch.randperm(3 * max_pages * page, generator=g)[:M]
    seq = (slots // (max_pages * page)).to(torch.int32)
    pos = (slots % (max_pages * page)).to(torch.int32)
    table_of_pages = torch.randperm(n_pages, generator=g)[:3 * max_pages].view(3, max_pages).to(torch.int32).cuda()
    table = torch.empty(M, hd // 2, 2, dtype=torch.float32, device="cuda")
    k.rope_table(pos.cuda(), P.rope_freqs(hd, 10000.0).cuda(), table)
    x = torch.empty(M, hidden, dtype=torch.bfloat16, device="cuda")
    k.rmsnorm(rows, gain, 1e-6, x)
    for bias_dt, write_kv in ((None, True), (torch.float32, True), (torch.bfloat16, False)):
        bias = None if bias_dt is None else rnd(width, seed=74).to(bias_dt).cuda()
        n_rows = width if write_kv else nh * hd
        ww, bb = k.pack_matrix(w[:n_rows].contiguous()), (None if bias is None else bias[:n_rows])
        got, want = [], []
        for inside in (True, False):
            kc = torch.full((n_pages, nkv, page, hd), 7.0, dtype=torch.bfloat16, device="cuda")
            vc = torch.full((n_pages, nkv, hd, page), 7.0, dtype=torch.bfloat16, device="cuda")
            qkv = torch.zeros(M, width, dtype=torch.bfloat16, device="cuda")
            if inside:
                k.gemm_normed_qkv_rope(rows, gain, 1e-6, ww, bb, qkv, table, pos.cuda(), seq.cuda(), table_of_pages, kc, vc,
                                       nh, nkv, hd, page, write_kv)
            else:
                k.gemm_qkv_rope(x, ww, bb, qkv, table, pos.cuda(), seq.cuda(), table_of_pages, kc, vc, nh, nkv, hd, page,
                                write_kv)
            (got if inside else want).extend([qkv[:, :nh * hd].clone(), kc, vc])
        for a, b in zip(got, want):
            assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_strided_rows(dtype):
    k = kernels(dtype)
    big, br = as_dtype(rnd(9, 300, seed=16), dtype)
    w, wr = as_dtype(rnd(50, 100, seed=17, scale=0.3), dtype)
    out = torch.zeros(9, 80, dtype=TORCH[dtype], device="cuda")
    k.gemm(big[:, 100:200], w, out[:, 10:60], None, MODE_STORE)              # a slice in, a slice out
    want = br[:, 100:200] @ wr.T
    assert (out[:, 10:60].cpu().double() - want).abs().max() <= tol(dtype, want, 1e-5, 1e-2)
    assert out[:, :10].abs().sum() == 0 and out[:, 60:].abs().sum() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(dtype):
    k = kernels(dtype)
    T, Fn = 7, 203
    gu, gr = as_dtype(rnd(T, 2 * Fn, seed=18, scale=4.0), dtype)
    gu[0, 0], gu[0, Fn] = -200.0, 1.0
    gu[0, 1], gu[0, Fn + 1] = 200.0, 1.0
    gr = gu.cpu().double()
    out = torch.empty(T, Fn, dtype=TORCH[dtype], device="cuda")
    k.swiglu(gu, out)
    ref = P.swiglu(gr[:, :Fn], gr[:, Fn:])
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype, ref, 1e-6, 8e-3)
    assert out[0, 0].item() == 0.0 and out[0, 1].item() == 200.0               # src/vmath.rs:495-497


def test_argmax_rules_on_the_device():
    k = kernels("float32")
    inf, nan = float("inf"), float("nan")
    rows = [[-inf] * 5, [1.0, 3.0, 3.0, 2.0, 0.0], [nan, 1.0, nan, 0.5, 1.0], [nan] * 5, [-1.0, 0.0, -0.0, -2.0, -3.0]]
    logits = torch.tensor(rows, dtype=torch.float32).cuda()
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    k.argmax(logits, out)
    assert out.tolist() == [P.argmax_last(r) for r in rows] == [4, 2, 4, 4, 2]
    big = rnd(3, 152064, seed=19).cuda()
    big[1, 777] = big[1, 150000] = 9.0                                         # a tie far apart: the last wins
    out = torch.empty(3, dtype=torch.int32, device="cuda")
    k.argmax(big, out)
    assert out.tolist() == [int(big[0].argmax()), 150000, int(big[2].argmax())]
    for view in (big[:, 1:9000], big[:, 4096:12288], big[:, :4097]):           # unaligned rows, whole chunks, one over
        k.argmax(view, out)
        assert out.tolist() == [P.argmax_last(r) for r in view.cpu().tolist()]


@pytest.mark.parametrize("V,width", [(5003, 256), (40961, 1024), (300, 64)])
def test_topk_with_penalty_on_the_device(V, width):
    """Slices of 4,096 logits leave their own k best, of which the k best are taken: vocabularies of
    one slice, of two with a short last one (shorter than k), and of eleven."""
    k = kernels("float32")
    logits = rnd(4, V, seed=20, scale=2.0)
    far = V - 3                                                                 # an id in the last slice
    logits[1, 10] = logits[1, far] = logits[1].max() + 1                        # ties at the top
    logits[2, 5] = float("nan")
    recent = torch.tensor([[3, 5, 1, 1, 2, 1, 0, 0], [10, 10, far, 7, 0, 0, 0, 0], [0] * 8, [9] * 8], dtype=torch.int32)
    n_recent = torch.tensor([6, 4, 0, 8], dtype=torch.int32)
    penalty = torch.tensor([2.0, 1.3, 1.0, 1.1])
    ks = torch.tensor([40, 7, min(width, V), 1], dtype=torch.int32)
    dev = logits.clone().cuda()
    cands = torch.zeros(4, width, dtype=torch.int64, device="cuda")
    k.topk(dev, recent.cuda(), n_recent.cuda(), penalty.cuda(), ks.cuda(), cands, k_max=int(ks.max()))
    for r in range(4):
        pen = P.penalize(logits[r].tolist(), recent[r, :n_recent[r]].tolist(), 10 ** 6, float(penalty[r]))
        pen = torch.tensor(pen, dtype=torch.float32)
        assert torch.equal(dev[r].cpu().nan_to_num(7.0), pen.nan_to_num(7.0))   # penalised in place, each id once
        want = [i for _, i in P.candidates(pen.tolist(), int(ks[r]))]
        got = sorted((c & 0xFFFFFFFFFFFFFFFF for c in cands[r, :int(ks[r])].tolist()), reverse=True)   # keys are unsigned
        assert [g & 0xFFFFFFFF for g in got] == want, r


@pytest.mark.parametrize("V", [1, 2, 7, 64, 65, 300])
def test_topk_of_a_whole_small_vocabulary(V):
    """k as large as the vocabulary: logits of both signs, zeros of both signs, infinities and NaN
    all among the candidates, in the plain sampler's order (NaN last, equal logits: the larger id
    first; src/sample.rs:280-305, 391-429)."""
    k = kernels("float32")
    logits = rnd(5, V, seed=21, scale=2.0)
    if V >= 7:
        logits[0, 1], logits[0, 3] = 0.0, -0.0
        logits[1, 2], logits[1, 5] = float("nan"), float("-inf")
        logits[2, 0], logits[2, 6] = float("inf"), float("nan")
        logits[3, 4] = logits[3, 2] = logits[3].max() + 1
    else:
        logits[1, 0] = float("nan")
        logits[2, V - 1] = float("-inf")
    ks = torch.full((5,), V, dtype=torch.int32)
    dev = logits.clone().cuda()
    cands = torch.zeros(5, max(V, 8), dtype=torch.int64, device="cuda")
    none = torch.zeros(5, 8, dtype=torch.int32, device="cuda")
    k.topk(dev, none, torch.zeros(5, dtype=torch.int32, device="cuda"), torch.ones(5, device="cuda"), ks.cuda(), cands, k_max=V)
    for r in range(5):
        want = [i for _, i in P.candidates(logits[r].tolist(), V)]
        got = sorted((c & 0xFFFFFFFFFFFFFFFF for c in cands[r, :V].tolist()), reverse=True)
        assert [g & 0xFFFFFFFF for g in got] == want, (V, r)


# --------------------------------------------------------------------------- matrix-core attention
def _mfma_case(nh, nkv, hd, page, T, window, seed=0, scale_q=1.0):
    q = rnd(T, nh, hd, seed=seed + 1) * scale_q
    kk = rnd(T, nkv, hd, seed=seed + 2)
    vv = rnd(T, nkv, hd, seed=seed + 3)
    qd, qr = as_dtype(q, "bfloat16")
    _, kr = as_dtype(kk, "bfloat16")
    _, vr = as_dtype(vv, "bfloat16")
    kc, vc, table = paged_cache(kr, vr, page, "bfloat16", seed=seed)
    ref = P.causal_attention(qr, kr, vr, window).view(T, nh * hd)
    return qd.view(T, nh * hd), kc, vc, table, ref


@pytest.mark.parametrize("nh,nkv,hd,page,T,window", [
    (4, 2, 64, 16, 300, 0), (7, 1, 128, 16, 257, 0), (6, 2, 128, 8, 130, 0), (2, 2, 64, 64, 200, 0),
    (8, 2, 128, 32, 333, 0), (4, 1, 64, 16, 400, 100), (14, 2, 128, 16, 129, 37), (16, 1, 64, 8, 70, 0),
    (7, 1, 128, 64, 300, 0), (4, 2, 128, 128, 333, 90), (6, 3, 64, 256, 290, 0)])
def test_prompt_attention_on_the_matrix_cores(nh, nkv, hd, page, T, window):
    k = kernels("bfloat16")
    assert k.attention_fast_ok(hd, page, nh, nkv)
    q, kc, vc, table, ref = _mfma_case(nh, nkv, hd, page, T, window)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    scale = 1.0 / math.sqrt(hd)
    # the whole sequence in tiles of 128, then a portion that starts in the middle of a block
    for start in (0, 77 if T > 100 else 3):
        tiles = [(a, min(128, T - a)) for a in range(start, T, 128)]
        out = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
        k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, out, torch.tensor(tiles, dtype=torch.int32).cuda(), nh, nkv,
                            hd, page, window, scale)
        assert not torch.isnan(out).any()                      # unused cache rows hold NaN: they must not leak
        assert (out[start:].cpu().double() - ref[start:]).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)
        assert out[:start].abs().sum() == 0                    # rows outside the tiles are not touched
    # two tiles a block, paired as the engine pairs them: the same bits as one tile a block
    from axon_amd.parts.attention import pair_tiles
    tiles = [(a, min(128, T - a)) for a in range(0, T, 128)]
    single = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, single, torch.tensor(tiles, dtype=torch.int32).cuda(), nh, nkv,
                        hd, page, window, scale)
    pairs = pair_tiles(tiles, [a + n for a, n in tiles])
    assert sorted(t for row in pairs for t in (row[:2], row[2:]) if t[1]) == tiles
    paired = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, paired, torch.tensor(pairs, dtype=torch.int32).cuda(), nh, nkv,
                        hd, page, window, scale)
    assert torch.equal(single, paired)
    # odd tiles: 2 tokens, 33 tokens, one token short of a block edge
    tiles = [(5, 2), (60, min(33, T - 63)), (T - 3, 3)]          # every tile lies inside the T tokens
    out = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, out, torch.tensor(tiles, dtype=torch.int32).cuda(), nh, nkv, hd,
                        page, window, scale)
    for a, n in tiles:
        assert (out[a:a + n].cpu().double() - ref[a:a + n]).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)


@pytest.mark.parametrize("nh,nkv,hd,page,T,window", [
    (4, 2, 64, 16, 300, 0), (7, 1, 128, 16, 1030, 0), (28, 4, 128, 16, 600, 0), (6, 2, 128, 8, 255, 0),
    (2, 2, 64, 64, 257, 0), (16, 1, 64, 32, 513, 0), (4, 1, 64, 16, 900, 300), (5, 5, 128, 16, 64, 0), (3, 1, 128, 16, 700, 70), (4, 1, 128, 16, 4100, 0), (2, 1, 64, 32, 3000, 1000),
    (28, 4, 128, 64, 600, 0), (4, 1, 128, 128, 700, 200), (6, 2, 64, 256, 1000, 0)])
def test_decoding_attention_on_the_matrix_cores(nh, nkv, hd, page, T, window):
    k = kernels("bfloat16")
    q, kc, vc, table, ref = _mfma_case(nh, nkv, hd, page, T, window, seed=5)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    scale = 1.0 / math.sqrt(hd)
    # single tokens at chosen positions: first, block and chunk edges, last
    picks = sorted({0, 1, 15, 16, 63, 64, 65, 255, 256, 257, 511, 512, T // 2, T - 2, T - 1} & set(range(T)))
    idx = torch.tensor(picks, dtype=torch.int32).cuda()
    ch = k.attention_decode_chunk
    chunks = max((p - ((max(0, p + 1 - window) if window else 0) // ch * ch)) // ch + 1 for p in picks)
    partial = torch.empty(k.attention_decode_workspace(len(picks), nh, hd, chunks), dtype=torch.float32, device="cuda")
    out = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, out, idx, partial, chunks, nh, nkv, hd, page, window, scale)
    assert not torch.isnan(out).any()
    got, want = out[picks].cpu().double(), ref[picks]
    assert (got - want).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)
    untouched = sorted(set(range(T)) - set(picks))
    assert out[untouched].abs().sum() == 0
    # a token's row does not depend on which other tokens share the launch
    solo = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    one = torch.tensor([picks[-1]], dtype=torch.int32).cuda()
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, solo, one, partial, chunks, nh, nkv, hd, page, window, scale)
    assert torch.equal(solo[picks[-1]], out[picks[-1]])
    # the list of chunks given by the caller, padded and in another order: the same bits
    import random
    work = k.attention_decode_work(picks, window, pad_to=len(picks) * chunks + 7)
    assert sum(1 for w in work if w >= 0) == sum((p - ((max(0, p + 1 - window) if window else 0) // ch * ch)) // ch + 1
                                                 for p in picks)
    random.Random(3).shuffle(work)
    listed = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, listed, idx, partial, chunks, nh, nkv, hd, page, window, scale,
                       work=torch.tensor(work, dtype=torch.int32).cuda())
    assert torch.equal(listed, out)
    # without an index list: the first tokens of the step
    first = min(T, 70)
    named, plain = torch.zeros_like(out), torch.zeros_like(out)
    wide = torch.empty(k.attention_decode_workspace(first, nh, hd, chunks), dtype=torch.float32, device="cuda")
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, named, torch.arange(first, dtype=torch.int32).cuda(), wide,
                       chunks, nh, nkv, hd, page, window, scale)
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, plain, first, wide, chunks, nh, nkv, hd, page, window, scale)
    assert torch.equal(named, plain) and (plain[:first].cpu().double() - ref[:first]).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)


@pytest.mark.parametrize("nh,nkv,hd,page,T,window", [
    (28, 4, 128, 16, 700, 0), (40, 8, 128, 16, 300, 0), (4, 2, 64, 8, 333, 0), (6, 1, 128, 64, 600, 150),
    (32, 1, 64, 16, 200, 0), (3, 3, 128, 32, 1100, 0), (7, 1, 128, 128, 500, 0), (4, 2, 64, 64, 330, 100)])
def test_a_position_gets_the_same_bits_from_the_prompt_kernel_and_the_decoding_kernel(nh, nkv, hd, page, T, window):
    """Every position of a sequence once as a row of a prompt portion (tiles cut at several places)
    and once as a single decoding token: bit for bit the same result, whatever the cut, because
    both kernels fold the same blocks of 64 positions with the same instructions
    (src/lm.rs:272-278; docs/determinism.md:53-57 of the reference)."""
    k = kernels("bfloat16")
    assert k.attention_fast_ok(hd, page, nh, nkv)
    q, kc, vc, table, ref = _mfma_case(nh, nkv, hd, page, T, window, seed=11)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    scale = 1.0 / math.sqrt(hd)
    ch = k.attention_decode_chunk
    chunks = max((p - ((max(0, p + 1 - window) if window else 0) // ch * ch)) // ch + 1 for p in range(T))
    partial = torch.empty(k.attention_decode_workspace(T, nh, hd, chunks), dtype=torch.float32, device="cuda")
    decoded = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, decoded, T, partial, chunks, nh, nkv, hd, page, window, scale)
    assert (decoded.cpu().double() - ref).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2)
    for cuts in ([0], [0, 2, 7, 64, 130, 131], [0, 63, 129, 190]):
        cuts = [c for c in cuts if c < T] + [T]
        tiles = [(a + o, min(128, b - a - o)) for a, b in zip(cuts, cuts[1:]) for o in range(0, b - a, 128)]
        tiles = [t for t in tiles if t[1] >= 1]
        prompt = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
        k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, prompt, torch.tensor(tiles, dtype=torch.int32).cuda(),
                            nh, nkv, hd, page, window, scale)
        assert torch.equal(prompt, decoded), cuts


@pytest.mark.parametrize("nh,nkv,hd,T,window", [(7, 1, 128, 450, 0), (4, 2, 64, 300, 0), (6, 2, 128, 333, 120)])
def test_the_page_size_does_not_change_a_bit_of_the_attention(nh, nkv, hd, T, window):
    """Pages of 64 positions or more hold a whole block of the kernels, which then take the page
    from one table entry for the wave; smaller pages are looked up lane by lane.  Both read the
    same keys and values, so the results are the same bits, from both kernels."""
    k = kernels("bfloat16")
    scale = 1.0 / math.sqrt(hd)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    ch = k.attention_decode_chunk
    chunks = max((p - ((max(0, p + 1 - window) if window else 0) // ch * ch)) // ch + 1 for p in range(T))
    tiles = torch.tensor([(a, min(128, T - a)) for a in range(0, T, 128)], dtype=torch.int32).cuda()
    results = []
    for page in (8, 16, 64, 128):
        q, kc, vc, table, ref = _mfma_case(nh, nkv, hd, page, T, window, seed=21)
        prompt = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
        k.attention_prefill(q, nh * hd, kc, vc, table, pos, rows, prompt, tiles, nh, nkv, hd, page, window, scale)
        partial = torch.empty(k.attention_decode_workspace(T, nh, hd, chunks), dtype=torch.float32, device="cuda")
        decoded = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
        k.attention_decode(q, nh * hd, kc, vc, table, pos, rows, decoded, T, partial, chunks, nh, nkv, hd, page, window, scale)
        assert not torch.isnan(prompt).any() and torch.equal(prompt, decoded), page
        results.append(prompt)
    assert all(torch.equal(results[0], r) for r in results[1:])


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("far", [15, 63, 64, 255, 256])
def test_matrix_core_attention_finds_a_far_key_and_respects_the_windows_edge(hd, far):
    """One loud key hundreds of positions back, in the first blocks of the context: found without a
    window, excluded when the window starts one position after it, found when it starts at it.
    `far` puts that edge inside a block of 64 positions (15), at the last place of a block and the
    first of the next (63, 64) and at the edge of the decoding kernel's chunks of 256 (255, 256)."""
    k = kernels("bfloat16")
    nh, nkv, page, T = 4, 2, 16, 700
    q = rnd(T, nh, hd, seed=7) * 0.1
    kk = rnd(T, nkv, hd, seed=8) * 0.1
    vv = rnd(T, nkv, hd, seed=9)
    kk[far, 1] = 0
    kk[far, 1, 3] = 40.0
    q[T - 1, 2] = 0
    q[T - 1, 2, 3] = 40.0
    qd, qr = as_dtype(q, "bfloat16")
    _, kr = as_dtype(kk, "bfloat16")
    _, vr = as_dtype(vv, "bfloat16")
    kc, vc, table = paged_cache(kr, vr, page, "bfloat16")
    pos = torch.arange(T, dtype=torch.int32).cuda()
    rows = torch.zeros(T, dtype=torch.int32).cuda()
    scale = 1.0 / math.sqrt(hd)
    one = torch.tensor([T - 1], dtype=torch.int32).cuda()
    tile = torch.tensor([[T - 40, 40]], dtype=torch.int32).cuda()
    partial = torch.empty(k.attention_decode_workspace(1, nh, hd, 16), dtype=torch.float32, device="cuda")
    for w, seen in ((0, True), (T - 1 - far, False), (T - far, True)):
        # the last token alone: its row of the plain formula
        lo = 0 if w == 0 else max(0, T - w)
        ref = torch.stack([torch.softmax((kr[lo:T, h // 2] @ qr[T - 1, h]) * scale, 0) @ vr[lo:T, h // 2] for h in range(nh)])
        for which in ("decode", "prefill"):
            out = torch.zeros(T, nh * hd, dtype=torch.bfloat16, device="cuda")
            if which == "decode":
                k.attention_decode(qd.view(T, -1), nh * hd, kc, vc, table, pos, rows, out, one, partial, 16, nh, nkv, hd,
                                   page, w, scale)
            else:
                k.attention_prefill(qd.view(T, -1), nh * hd, kc, vc, table, pos, rows, out, tile, nh, nkv, hd, page, w, scale)
            got = out[T - 1].cpu().double().view(nh, hd)
            assert (got - ref).abs().max() <= tol("bfloat16", ref, bf16=1.5e-2), (w, which)
            assert ((got[2] - vr[far, 1]).abs().max() < 2e-2) == seen, (w, which)


def test_matrix_core_attention_refuses_other_sizes():
    k = kernels("bfloat16")
    assert not k.attention_fast_ok(80, 16, 4, 2) and not k.attention_fast_ok(128, 5, 4, 2)
    assert not k.attention_fast_ok(128, 16, 66, 2)             # a group of 33 heads
    assert not kernels("float32").attention_fast_ok(128, 16, 4, 2)
    q = torch.zeros(4, 160, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(2, 1, 16, 80, dtype=torch.bfloat16, device="cuda")
    i32 = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(KernelError) as e:
        k.attention_prefill(q, 160, kc, kc.view(2, 1, 80, 16), i32.view(1, 4), i32, i32, torch.zeros_like(q),
                            torch.tensor([[0, 4]], dtype=torch.int32).cuda(), 2, 1, 80, 16, 0, 1.0)
    assert "head_dim 80" in str(e.value)


def test_kernels_refuse_what_they_cannot_run():
    k = kernels("float32")
    x = torch.zeros(2, 8, device="cuda")
    with pytest.raises(KernelError):
        k.gemm(x, torch.zeros(4, 9, device="cuda"), torch.zeros(2, 4, device="cuda"))       # K differs
    with pytest.raises(KernelError):
        k.gemm(x.bfloat16(), torch.zeros(4, 8, device="cuda"), torch.zeros(2, 4, device="cuda"))   # wrong dtype
    with pytest.raises(KernelError):
        k.gemm(x.cpu(), torch.zeros(4, 8), torch.zeros(2, 4))                               # not on the device
    q = torch.zeros(1, 24, device="cuda")
    cache = torch.zeros(2, 1, 8, 24, device="cuda")
    i32 = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(KernelError) as e:
        k.attention(q, 24, cache, cache.view(2, 1, 24, 8), i32.view(1, 1), i32, i32, torch.zeros(1, 24, device="cuda"), 1, 1, 24, 8, 0,
                    1.0)
    assert "head_dim 24" in str(e.value)
