"""The arrangement of a layer's parts around the residual stream.

"prenorm": x += mixer(norm1(x)); x += feed_forward(norm2(x)), the order of
src/model.rs:2980-3055.  The residual stream `x` is float32 and is updated in place: the
mixer and the feed-forward add their output to it in the epilogue of their last product.
"""
from __future__ import annotations

from typing import List

from .base import Block, CacheBinding, TensorDecl, register_block

# A norm behind a product whose kernel holds the finished rows anyway can be written by that
# kernel, and a norm before a product of few rows can be worked out inside that product (the same
# bits as the norm's own pass, both): the block asks its parts, step by step.


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

    def first_norm(self):
        return self.norm1

    def last_part(self):
        return self.feed_forward

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        h = normed
        if h is None:
            h = self.preceding_of(ctx, self.norm1, self.mixer, x)
        if h is None:
            h = self.norm1.forward(ctx, x)
        second = self.following_of(ctx, self.mixer, self.norm2, x.shape[0])
        if second is not None:
            self.mixer.forward(ctx, binding, h, x, second)
            h = second.values
        else:
            self.mixer.forward(ctx, binding, h, x)
            h = self.preceding_of(ctx, self.norm2, self.feed_forward, x)
            if h is None:
                h = self.norm2.forward(ctx, x)
        if following is not None:
            self.feed_forward.forward(ctx, h, x, following)
        else:
            self.feed_forward.forward(ctx, h, x)


register_block("prenorm", PreNormBlock)
