"""Grouped-query attention over the paged cache: the mixer of this architecture.

q = Wq h + bq, k = Wk h + bk, v = Wv h + bv (bias after the product, before the rotation;
used iff the tensor exists: src/model.rs:2982-2991), rotate-half on q and k, k and v stored in
the request's pages, causal attention in which query head qh reads kv head qh // group with
scale 1/sqrt(head_dim) (src/model.rs:3373-3463), then the output projection, whose result is
added to the residual stream (src/model.rs:3031-3038).

The three projections run as one product over a fused [q_dim + 2 kv_dim, hidden] matrix
(fused when the weights are loaded; the reference fuses at launch: src/model.rs:2199-2238).

Parameters: `hidden_size`, `num_heads`, `num_kv_heads`, `head_dim`, `qkv_bias` (True, False
or "optional"), `out_bias`, `window` (0: all earlier positions), `position` (a PartSpec).
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE, PackedMatrix
from .base import CacheBinding, CacheSpec, Mixer, PrecedingNorm, TensorDecl, build_part, register_mixer


class AttentionPlan:
    """How the matrix-core kernels split a step: prompt portions (2 tokens or more) go to the
    prompt kernel in tiles of up to 128 tokens, single tokens to the decoding kernel.  Made
    once per step and window, shared by all layers."""

    def __init__(self, ctx, window: int, n_heads: int, head_dim: int):
        dev = ctx.rt.device
        self.tiles = None
        self.partial = None
        self.decode_work = None
        if ctx.decode_only:
            # every span is one token, in order: no index list; the engine has counted the chunks
            # and brought the list of them to the device (what a captured graph replays must not
            # come from the host)
            self.decode_tokens = ctx.n_tokens
            self.max_chunks = ctx.decode_shapes[("attention_chunks", window)]
            self.decode_work = ctx.decode_inputs[("attention_work", window)]
            n_single = ctx.n_tokens
        else:
            tiles, seen, singles, chunks = [], [], [], 1
            tile = ctx.rt.k.attention_prefill_tile          # tokens of one request a tile of the prompt kernel holds
            for s in ctx.spans:
                if s.q_len == 1:
                    singles.append(s.q_start)
                    chunks = max(chunks, decode_chunks_of(s.start_pos, window, ctx.rt.k.attention_decode_chunk))
                else:
                    for at in range(0, s.q_len, tile):
                        n = min(tile, s.q_len - at)
                        tiles.append((s.q_start + at, n))
                        last = s.start_pos + at + n                 # positions the tile's last token sees
                        seen.append(min(last, window + n) if window > 0 else last)
            # the kernels trust these indices: check them here, on the host
            if (any(a < 0 or n < 1 or a + n > ctx.n_tokens for a, n in tiles)
                    or any(not 0 <= t < ctx.n_tokens for t in singles)):
                raise ValueError("attention plan: a span lies outside the tokens of the step")
            self.tiles = torch.tensor(pair_tiles(tiles, seen), dtype=torch.int32).to(dev) if tiles else None
            self.decode_tokens = torch.tensor(singles, dtype=torch.int32).to(dev) if singles else None
            self.max_chunks = chunks
            n_single = len(singles)
            if singles:
                at = {s.q_start: s.start_pos for s in ctx.spans if s.q_len == 1}
                work = ctx.rt.k.attention_decode_work([at[t] for t in singles], window)
                self.decode_work = torch.tensor(work, dtype=torch.int32).to(dev)
        if n_single:
            n = ctx.rt.k.attention_decode_workspace(n_single, n_heads, head_dim, self.max_chunks)
            lasting = ctx.decode_scratch.get(("attention_partial", window, n_heads, head_dim)) if ctx.decode_only else None
            if lasting is not None and lasting.numel() >= n:
                self.partial = lasting           # one workspace for every decoding step and graph
            else:
                self.partial = torch.empty(n, dtype=torch.float32, device=dev)


def pair_tiles(tiles, seen):
    """Two tiles a block, one that sees many positions with one that sees few: the tiles of a
    causal prompt see 1, 2, 3 ... blocks of positions, and blocks of equal work finish together.
    tiles: (first token, count); seen: positions each looks at.  Rows of (first, count, first,
    count), the second count 0 where a tile is left alone."""
    order = sorted(range(len(tiles)), key=lambda i: -seen[i])
    rows = []
    for k in range((len(order) + 1) // 2):
        a, b = order[k], order[len(order) - 1 - k]
        rows.append(tiles[a] + (tiles[b] if b != a else (0, 0)))
    return rows


def round_up_by_eighths(n: int) -> int:
    """n rounded up to a multiple of a power of two that is at most an eighth of it."""
    step = 1 << max(0, n.bit_length() - 4)
    return -(-n // step) * step


def decode_chunks_of(pos: int, window: int, chunk: int) -> int:
    """Chunks (of `chunk` positions, the kernel's constant) the decoding kernel cuts a token's range into."""
    lo = max(0, pos + 1 - window) if window > 0 else 0
    return (pos - lo // chunk * chunk) // chunk + 1


def attention_plan(ctx, window: int, n_heads: int, head_dim: int) -> AttentionPlan:
    key = ("attention_plan", window, n_heads, head_dim)
    plan = ctx.shared.get(key)
    if plan is None:
        plan = ctx.shared[key] = AttentionPlan(ctx, window, n_heads, head_dim)
    return plan


class GQAttention(Mixer):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden = int(p["hidden_size"])
        self.nh = int(p["num_heads"])
        self.nkv = int(p["num_kv_heads"])
        self.hd = int(p["head_dim"])
        self.window = int(p.get("window", 0))
        self.qkv_bias = p.get("qkv_bias", False)
        self.out_bias = bool(p.get("out_bias", False))
        if self.nh % self.nkv:
            raise ConfigError(f"{self.nh} query heads are not a multiple of {self.nkv} kv heads")
        if self.hd % 16 or not 16 <= self.hd <= 256:
            raise ConfigError(f"head_dim {self.hd} is not a multiple of 16 between 16 and 256: no kernel takes it")
        self.q_dim, self.kv_dim = self.nh * self.hd, self.nkv * self.hd
        self.scale = 1.0 / math.sqrt(self.hd)
        self.position = build_part("position", p["position"]) if p.get("position") is not None else None
        names = p.get("names", {})
        base = prefix + names.get("scope", "self_attn.")
        self.n = {k: base + names.get(k, k + "_proj") for k in ("q", "k", "v", "o")}
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None
        self._max_context = None
        self._workspace = None
        self.decode_chunk = 1 << 30          # until `load` has asked the kernels: one chunk
        self._work_list = lambda positions, window: list(range(len(positions)))

    # ------------------------------------------------------------------ declarations
    def tensors(self) -> List[TensorDecl]:
        t = [TensorDecl(self.n["q"] + ".weight", (self.q_dim, self.hidden)),
             TensorDecl(self.n["k"] + ".weight", (self.kv_dim, self.hidden)),
             TensorDecl(self.n["v"] + ".weight", (self.kv_dim, self.hidden)),
             TensorDecl(self.n["o"] + ".weight", (self.hidden, self.q_dim))]
        if self.qkv_bias:
            opt = self.qkv_bias == "optional"
            t += [TensorDecl(self.n["q"] + ".bias", (self.q_dim,), "bias", opt),
                  TensorDecl(self.n["k"] + ".bias", (self.kv_dim,), "bias", opt),
                  TensorDecl(self.n["v"] + ".bias", (self.kv_dim,), "bias", opt)]
        if self.out_bias:
            t.append(TensorDecl(self.n["o"] + ".bias", (self.hidden,), "bias"))
        return t

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(entries=2, heads=self.nkv, head_dim=self.hd, window=self.window)

    def max_context(self):
        return self._max_context

    def decode_shape(self, positions):
        """The decoding kernel's workspace is laid out by the longest context of the step, in
        chunks of the kernel's size, rounded up to a power of two so that few shapes exist (the
        blocks that are launched are those of `decode_input`, whatever this number)."""
        most = max(decode_chunks_of(p, self.window, self.decode_chunk) for p in positions)
        return ("attention_chunks", self.window), 1 << (most - 1).bit_length()

    def decode_input(self, positions):
        """The list of the chunks the decoding kernel computes, a block each: blocks are launched
        for the chunks that exist, not for the longest context times the tokens.  Padded in
        steps of an eighth or less."""
        work = self._work_list(positions, self.window)
        return ("attention_work", self.window), work + [-1] * (round_up_by_eighths(len(work)) - len(work))

    def decode_input_capacity(self, max_seqs: int, max_seq_len: int) -> int:
        return round_up_by_eighths(max_seqs * decode_chunks_of(max(0, max_seq_len - 1), 0, self.decode_chunk))

    def decode_scratch(self, max_seqs: int, max_seq_len: int):
        """The blocks' partial results of the decoding kernel, laid out by the longest context in
        chunks rounded up to a power of two (see `decode_shape`)."""
        if self._workspace is None:              # no kernel of this build and these sizes wants one
            return None
        most = decode_chunks_of(max(0, max_seq_len - 1), self.window, self.decode_chunk)
        chunks = 1 << (most - 1).bit_length()
        return ("attention_partial", self.window, self.nh, self.hd), self._workspace(max_seqs, self.nh, self.hd, chunks)

    def load(self, store, rt) -> None:
        self.decode_chunk = rt.k.attention_decode_chunk
        self._work_list = rt.k.attention_decode_work
        self._max_context = rt.k.attention_decode_max_context
        if rt.k.attention_fast_ok(self.hd, 64, self.nh, self.nkv):
            self._workspace = rt.k.attention_decode_workspace
        self.w_qkv = rt.k.prepare_weight(store.fused_matrix([self.n[k] + ".weight" for k in ("q", "k", "v")]))
        biases = [store.vector(self.n[k] + ".bias", optional=True) for k in ("q", "k", "v")] if self.qkv_bias else []
        present = [b is not None for b in biases]
        if any(present):
            if not all(present):
                raise ConfigError(f"{self.prefix}: q, k and v biases must all be present or all absent")
            dt = torch.float32 if any(b.dtype == torch.float32 for b in biases) else biases[0].dtype
            self.b_qkv = torch.cat([b.to(dt) for b in biases]).contiguous()
        self.w_o = rt.k.prepare_weight(store.matrix(self.n["o"] + ".weight"))
        store.forget(self.n["o"] + ".weight")
        self.b_o = store.vector(self.n["o"] + ".bias") if self.out_bias else None
        if self.position is not None:
            self.position.load(store, rt)

    # ------------------------------------------------------------------ the step
    def finishes_following_norm(self, ctx) -> bool:
        return isinstance(self.w_o, PackedMatrix) and ctx.rt.k.gemm_then_norm_ok(ctx.n_tokens, self.hidden, self.q_dim)

    def applies_preceding_norm(self, ctx) -> bool:
        k = ctx.rt.k
        rows = self.q_dim + 2 * self.kv_dim
        return (isinstance(self.w_qkv, PackedMatrix) and self.position is not None
                and k.gemm_qkv_rope_ok(ctx.n_tokens, rows, self.hidden, self.hd, self.position.rotary_dim)
                and k.gemm_normed_ok(ctx.n_tokens, rows, self.hidden))

    def forward(self, ctx, binding: CacheBinding, h, residual, following=None) -> None:
        k = ctx.rt.k
        T = h.shape[0]
        group = ctx.cache.group(binding.group)
        k_cache, v_cache = group.layer(binding.index)
        # values are kept position-contiguous: a page of them is [heads, head_dim, page_size]
        v_cache = v_cache.view(v_cache.shape[0], self.nkv, self.hd, group.page_size)
        qkv = ctx.ws.take((T, self.q_dim + 2 * self.kv_dim), ctx.rt.dtype)
        if self.position is not None:
            table, rotary = self.position.tables(ctx), self.position.rotary_dim
        else:
            table, rotary = ctx.no_rotation(), 0
        if binding.writes:
            w, bias = self.w_qkv, self.b_qkv
        else:
            # reading another run's cache: only the queries are needed
            w, bias = self.w_qkv[:self.q_dim], None if self.b_qkv is None else self.b_qkv[:self.q_dim]
        in_one = isinstance(w, PackedMatrix) and k.gemm_qkv_rope_ok(T, w.shape[0], self.hidden, self.hd, rotary)
        cache = (group.block_table, k_cache, v_cache, self.nh, self.nkv, self.hd)
        if isinstance(h, PrecedingNorm) and not (in_one and k.gemm_normed_ok(T, w.shape[0], self.hidden, gain=h.gain)):
            h = h.apply(ctx)
        if isinstance(h, PrecedingNorm):
            # few rows: the norm, the product, the rotation and the store into the pages in one launch
            k.gemm_normed_qkv_rope(h.rows, h.gain, h.eps, w, bias, qkv, table, ctx.positions, ctx.seq_rows, *cache,
                                   group.page_size, binding.writes)
        elif in_one:
            # product, rotation and the store into the pages in one launch (a short step) or with the
            # rotation and the store done by the kernel that adds the sums of the product's segments
            k.gemm_qkv_rope(h, w, bias, qkv, table, ctx.positions, ctx.seq_rows, *cache, group.page_size, binding.writes)
        else:
            k.gemm(h, w, qkv[:, :w.shape[0]], bias, MODE_STORE)
            k.rope_kv_write(qkv, table, ctx.positions, ctx.seq_rows, *cache, rotary, group.page_size, binding.writes)
        att = ctx.ws.take((T, self.q_dim), ctx.rt.dtype)
        if k.attention_fast_ok(self.hd, group.page_size, self.nh, self.nkv):
            plan = attention_plan(ctx, self.window, self.nh, self.hd)
            common = (k_cache, v_cache, group.block_table, ctx.positions, ctx.seq_rows, att)
            sizes = (self.nh, self.nkv, self.hd, group.page_size, self.window, self.scale)
            if plan.tiles is not None:
                k.attention_prefill(qkv, qkv.stride(0), *common, plan.tiles, *sizes)
            if plan.decode_tokens is not None:
                k.attention_decode(qkv, qkv.stride(0), *common, plan.decode_tokens, plan.partial, plan.max_chunks, *sizes,
                                   work=plan.decode_work)
        else:
            k.attention(qkv, qkv.stride(0), k_cache, v_cache, group.block_table, ctx.positions, ctx.seq_rows, att,
                        self.nh, self.nkv, self.hd, group.page_size, self.window, self.scale)
        k.gemm(att, self.w_o, residual, self.b_o, MODE_ADD_F32,
               following_norm=None if following is None else following.as_argument())


register_mixer("gqa_attention", GQAttention)
