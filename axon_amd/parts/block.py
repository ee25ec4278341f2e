"""The arrangement of a layer's parts around the residual stream.

"prenorm": x += mixer(norm1(x)); x += feed_forward(norm2(x)), the order of
src/model.rs:2980-3055.  The residual stream `x` is float32 and is updated in place: the
mixer and the feed-forward add their output to it in the epilogue of their last product.
"""
from __future__ import annotations

from typing import List

from .base import Block, CacheBinding, TensorDecl, register_block

# A norm between two products can be folded into them where both offer it (short steps in
# bfloat16: the products then run in kernels that take it), or done whole by the product before
# it where that one offers it (steps whose products split K): the block asks its parts.


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

    def first_norm_fold(self, ctx, n_rows: int, whole: bool = False):
        if whole:
            return self.norm1.fold(ctx, n_rows, whole=True)
        return self.norm1.fold(ctx, n_rows) if self.mixer.takes_unscaled_rows(ctx) else None

    def folds_following_norm(self, ctx) -> bool:
        return self.feed_forward.folds_following_norm(ctx)

    def finishes_following_norm(self, ctx) -> bool:
        return self.feed_forward.finishes_following_norm(ctx)

    def forward(self, ctx, binding: CacheBinding, x, unscaled=None, fold_next=None) -> None:
        mark = ctx.ws.mark()
        h = unscaled if unscaled is not None else self.norm1.forward(ctx, x)
        fold = None
        if self.mixer.finishes_following_norm(ctx):
            fold = self.norm2.fold(ctx, x.shape[0], whole=True)
        elif self.mixer.folds_following_norm(ctx) and self.feed_forward.takes_unscaled_rows(ctx):
            fold = self.norm2.fold(ctx, x.shape[0])
        if fold is not None:
            self.mixer.forward(ctx, binding, h, x, fold)
            h = fold.rows()
        else:
            self.mixer.forward(ctx, binding, h, x)
            h = self.norm2.forward(ctx, x)
        if fold_next is not None:
            self.feed_forward.forward(ctx, h, x, fold_next)
        else:
            self.feed_forward.forward(ctx, h, x)
        ctx.ws.release(mark)


register_block("prenorm", PreNormBlock)
