"""Helpers of the GPU tests: paged caches from plain tensors, a context for a part alone."""
import torch

from axon_amd.cache import CacheManager, GroupPlan
from axon_amd.engine import Runtime, Workspace
from axon_amd.engine.step import Span, StepContext

DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def tol(dtype, ref, f32=2e-5, bf16=2e-2):
    return (f32 if dtype == "float32" else bf16) * max(1.0, float(ref.abs().max()))


def paged_cache(k, v, page_size, dtype, n_extra_pages=3, seed=0, fill=None):
    """Scatter k, v [T, nkv, hd] of ONE request into shuffled pages.  Returns
    (k_cache [pages, nkv, page, hd], v_cache [pages, nkv, hd, page], block_table [1, pages]);
    unused rows hold `fill` (NaN by default, so a
    kernel that reads past what it may is caught)."""
    T, nkv, hd = k.shape
    n_logical = -(-T // page_size)
    n_pages = n_logical + n_extra_pages
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages, generator=g)[:n_logical]
    fill = float("nan") if fill is None else fill
    kc = torch.full((n_pages, nkv, page_size, hd), fill, dtype=torch.float32)
    vc = torch.full((n_pages, nkv, page_size, hd), fill, dtype=torch.float32)
    for t in range(T):
        p, o = int(perm[t // page_size]), t % page_size
        kc[p, :, o] = k[t].float()
        vc[p, :, o] = v[t].float()
    dt = TORCH[dtype]
    vc = vc.permute(0, 1, 3, 2).contiguous()          # values: [pages, heads, head_dim, page_size]
    return kc.to(dt).cuda(), vc.to(dt).cuda(), perm.to(torch.int32)[None, :].contiguous().cuda()


class PartHarness:
    """Runs one part alone: a runtime, a cache made for the part's own need, and the context of
    a step with one request at given positions."""

    def __init__(self, dtype, cache_spec=None, n_layers=1, page_size=8, n_pages=32, max_seq_len=256, state_elems=()):
        self.rt = Runtime(dtype)
        plans = [GroupPlan(cache_spec, n_layers, page_size, n_pages)] if cache_spec is not None else []
        self.cache = CacheManager(plans, list(state_elems), 4, max_seq_len, self.rt.device, self.rt.dtype,
                                  shuffle_seed=7)
        self.ws = Workspace(self.rt.device)
        self.slot = self.cache.open()
        self.n_cached = 0

    def ctx(self, tokens):
        """The context for the request's next len(tokens) tokens."""
        n = len(tokens)
        self.cache.reserve(self.slot, self.n_cached + n)
        self.cache.sync_tables()
        meta = torch.tensor([list(tokens), list(range(self.n_cached, self.n_cached + n)), [self.slot] * n],
                            dtype=torch.int32).cuda()
        ctx = StepContext(self.rt, self.cache, self.ws, meta, n, [Span(self.slot, 0, n, self.n_cached)])
        self.n_cached += n
        return ctx


class DictSource:
    """Tensors from a dict, with the interface of a checkpoint."""

    def __init__(self, tensors):
        self.t = tensors

    def names(self):
        return list(self.t)

    def __contains__(self, n):
        return n in self.t

    def shape(self, n):
        return tuple(self.t[n].shape)

    def dtype(self, n):
        return self.t[n].dtype

    def tensor(self, n, device=None):
        return self.t[n]
