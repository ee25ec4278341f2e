"""Token embedding and the language-model head.

The embedding row is the token's starting vector as it is (src/model.rs:2657-2675).  The head
is `lm_head.weight` if the tensor exists, else the embedding matrix; a model that is not tied
must have it (src/model.rs:1800-1803, src/safetensors.rs:1608-1614).  Logits are float32 and
are computed only at the rows asked for (src/model.rs:2647-2654).
"""
from __future__ import annotations

from typing import List

import torch

from ..kernels import MODE_STORE_F32, PackedMatrix
from .base import Part, TensorDecl, register_embedding, register_head


class TokenEmbedding(Part):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.name = prefix + params["tensor"]
        self.table = None            # row-major, or a head's packed matrix (see LMHead.load)

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.vocab, self.hidden), "matrix")]

    def load(self, store, rt) -> None:
        self.table = store.matrix(self.name)

    def read_from(self, head, store) -> None:
        """Read the rows out of `head`'s copy of this matrix (a head that `shares_with` this
        embedding); the copy loaded here is dropped."""
        self.table = head.weight
        store.forget(self.name)

    def forward(self, ctx, out=None):
        if out is None:
            out = ctx.ws.take((ctx.n_tokens, self.hidden), torch.float32)
        return ctx.rt.k.embed(ctx.tokens, self.table, out)


class LMHead(Part):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.name = prefix + params["tensor"]
        self.tied_to = params.get("tied_to")
        self.tied = bool(params.get("tied", False))
        self.weight = None
        self.source_name = None      # the tensor the head was loaded from

    def tensors(self) -> List[TensorDecl]:
        # tied: the head's own tensor is used if the checkpoint has one
        return [TensorDecl(self.name, (self.vocab, self.hidden), "matrix", optional=self.tied)]

    def load(self, store, rt) -> None:
        self.source_name = self.name
        weight = store.matrix(self.name, optional=self.tied)
        if weight is None:
            self.source_name = self.tied_to
            weight = store.matrix(self.tied_to)
        # packed for the matrix-core products where it can be; a tied embedding then reads the
        # packed matrix too (the model hands it over), so that the matrix is in memory once
        self.weight = rt.k.prepare_weight(weight)

    def shares_with(self, embedding) -> bool:
        """Whether this head was loaded from `embedding`'s tensor and keeps it in a form that the
        embedding kernel reads as well (packed): the matrix then need be in memory only once."""
        return (self.source_name is not None and self.source_name == getattr(embedding, "name", None)
                and isinstance(self.weight, PackedMatrix))

    def forward(self, ctx, h, out=None):
        """h: [rows, hidden] in the compute dtype -> float32 logits [rows, vocab]."""
        if out is None:
            out = torch.empty((h.shape[0], self.vocab), dtype=torch.float32, device=h.device)
        return ctx.rt.k.gemm(h, self.weight, out, None, MODE_STORE_F32)


register_embedding("token_embedding", TokenEmbedding)
register_head("lm_head", LMHead)
