"""The arrangement of a layer's parts around the residual stream.

"prenorm": x += mixer(norm1(x)); x += feed_forward(norm2(x)), the order of
src/model.rs:2980-3055.  The residual stream `x` is float32 and is updated in place: the
mixer and the feed-forward add their output to it in the epilogue of their last product.
"""
from __future__ import annotations

from typing import List

from .base import Block, CacheBinding, TensorDecl, register_block


class PreNormBlock(Block):
    graph_safe = True
    norm1_name = "input_layernorm.weight"
    norm2_name = "post_attention_layernorm.weight"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        super().__init__(norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)
        self.norm2 = norm_factory(self.norm2_name)

    def tensors(self) -> List[TensorDecl]:
        return self.norm1.tensors() + self.mixer.tensors() + self.norm2.tensors() + self.feed_forward.tensors()

    def load(self, store, rt) -> None:
        for part in (self.norm1, self.mixer, self.norm2, self.feed_forward):
            part.load(store, rt)

    def forward(self, ctx, binding: CacheBinding, x) -> None:
        mark = ctx.ws.mark()
        h = self.norm1.forward(ctx, x)
        self.mixer.forward(ctx, binding, h, x)
        ctx.ws.release(mark)
        h = self.norm2.forward(ctx, x)
        self.feed_forward.forward(ctx, h, x)
        ctx.ws.release(mark)


register_block("prenorm", PreNormBlock)
