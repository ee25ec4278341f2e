"""The dense SwiGLU feed-forward: down(silu(gate h) * up h), added to the residual stream.

act = (g / (1 + exp(-g))) * u (src/vmath.rs:128-132), no biases (src/model.rs:3043-3055).
gate and up run as one product over a fused [2 ffn, hidden] matrix whose epilogue applies the
activation, so the two halves never travel through memory.  Parameters:
`hidden_size`, `intermediate_size`.
"""
from __future__ import annotations

from typing import List

from ..kernels import MODE_ADD_F32, MODE_SWIGLU, PackedMatrix
from .base import FeedForward, PrecedingNorm, TensorDecl, register_feed_forward


class SwiGLUMLP(FeedForward):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden = int(params["hidden_size"])
        self.ffn = int(params["intermediate_size"])
        names = params.get("names", {})
        base = prefix + names.get("scope", "mlp.")
        self.n = {k: base + names.get(k, k + "_proj") + ".weight" for k in ("gate", "up", "down")}
        self.w_gate_up = self.w_down = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.n["gate"], (self.ffn, self.hidden)), TensorDecl(self.n["up"], (self.ffn, self.hidden)),
                TensorDecl(self.n["down"], (self.hidden, self.ffn))]

    def load(self, store, rt) -> None:
        self.w_gate_up = rt.k.prepare_weight(store.fused_matrix([self.n["gate"], self.n["up"]]), gated=True)
        self.w_down = rt.k.prepare_weight(store.matrix(self.n["down"]))
        store.forget(self.n["down"])

    def finishes_following_norm(self, ctx) -> bool:
        return isinstance(self.w_down, PackedMatrix) and ctx.rt.k.gemm_then_norm_ok(ctx.n_tokens, self.hidden, self.ffn)

    def applies_preceding_norm(self, ctx) -> bool:
        return (isinstance(self.w_gate_up, PackedMatrix)
                and ctx.rt.k.gemm_normed_ok(ctx.n_tokens, self.ffn, self.hidden, gated=True))

    def forward(self, ctx, h, residual, following=None) -> None:
        k = ctx.rt.k
        act = ctx.ws.take((h.shape[0], self.ffn), ctx.rt.dtype)
        if isinstance(h, PrecedingNorm) and not k.gemm_normed_ok(h.shape[0], self.ffn, self.hidden, gated=True, gain=h.gain):
            h = h.apply(ctx)
        if isinstance(h, PrecedingNorm):                        # few rows: the norm inside the product
            k.gemm_normed_glu(h.rows, h.gain, h.eps, self.w_gate_up, act)
        else:
            k.gemm(h, self.w_gate_up, act, None, MODE_SWIGLU)   # silu(gate h) * up h, in the product's epilogue
        k.gemm(act, self.w_down, residual, None, MODE_ADD_F32,
               following_norm=None if following is None else following.as_argument())


register_feed_forward("swiglu_mlp", SwiGLUMLP)
