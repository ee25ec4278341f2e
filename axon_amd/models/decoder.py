"""A decoder model put together from a `ModelSpec`: embedding, blocks in their execution
order, final norm and head.  It knows no architecture: the configuration decided the parts.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch

from ..cache.manager import GroupPlan
from ..config.base import ConfigError, ModelConfig
from ..parts.base import CacheBinding, TensorDecl, build_block, build_part


@dataclass
class CachePlan:
    """What the model's runs need from the cache manager: for each group its need and number
    of storing runs; for each run its binding; the sizes of the state arenas."""
    group_specs: List
    group_layers: List[int]
    bindings: List[CacheBinding]
    state_elems: List[int]


class DecoderModel:
    def __init__(self, config: ModelConfig):
        self.config = config
        spec = config.model_spec()
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.vocab_size = spec.vocab_size
        self.max_positions = spec.max_positions
        self.embedding = build_part("embedding", spec.embedding)
        self.blocks = []
        for layer in spec.layers:
            mixer = build_part("mixer", layer.mixer, layer.prefix)
            ffn = build_part("feed_forward", layer.feed_forward, layer.prefix)
            self.blocks.append(build_block(layer.block, layer.norm, mixer, ffn, layer.prefix))
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.order = list(spec.order)
        for run in self.order:
            if not 0 <= run.layer < len(self.blocks):
                raise ConfigError(f"the execution order names layer {run.layer}, the model has {len(self.blocks)}")
        self.cache_plan = self._plan_cache()

    # ------------------------------------------------------------------ declarations
    def tensors(self) -> List[TensorDecl]:
        out = list(self.embedding.tensors())
        for b in self.blocks:
            out += b.tensors()
        return out + self.final_norm.tensors() + self.head.tensors()

    def _plan_cache(self) -> CachePlan:
        group_of_key: Dict[Tuple, int] = {}
        specs, counts = [], []
        where: Dict[int, Tuple[int, int]] = {}      # cache id -> (group, index in group)
        writer_spec: Dict[int, object] = {}
        for run in self.order:                      # first the runs that store
            cs = self.blocks[run.layer].mixer.cache_spec()
            if cs is None or not run.writes_cache:
                continue
            if run.cache in where:
                raise ConfigError(f"two runs store into cache {run.cache}")
            g = group_of_key.setdefault(cs.group_key(), len(specs))
            if g == len(specs):
                specs.append(cs)
                counts.append(0)
            where[run.cache] = (g, counts[g])
            writer_spec[run.cache] = cs
            counts[g] += 1
        bindings, state_elems = [], []
        for run in self.order:
            mixer = self.blocks[run.layer].mixer
            cs, ss = mixer.cache_spec(), mixer.state_spec()
            b = CacheBinding(writes=run.writes_cache)
            if cs is not None:
                if run.cache not in where:
                    raise ConfigError(f"a run of layer {run.layer} reads cache {run.cache}, which no run stores")
                if writer_spec[run.cache].group_key() != cs.group_key():
                    raise ConfigError(f"layer {run.layer} cannot read cache {run.cache}: its shape differs")
                b.group, b.index = where[run.cache]
            if ss is not None:
                b.state_index = len(state_elems)
                state_elems.append((ss.elems, ss.dtype))
            bindings.append(b)
        return CachePlan(specs, counts, bindings, state_elems)

    def group_plans(self, page_size: int, pages_of_group) -> List[GroupPlan]:
        """`pages_of_group(spec, n_layers, page_size)` decides each pool's size."""
        return [GroupPlan(s, n, page_size, pages_of_group(s, n, page_size))
                for s, n in zip(self.cache_plan.group_specs, self.cache_plan.group_layers)]

    # ------------------------------------------------------------------ weights
    def load(self, store, rt) -> None:
        self.embedding.load(store, rt)
        for b in self.blocks:
            b.load(store, rt)
        self.final_norm.load(store, rt)
        self.head.load(store, rt)
        # a head tied to the embedding may keep the matrix in a form of its own (repacked for its
        # product): the head says so, the embedding then reads that copy and the other is dropped
        if self.head.shares_with(self.embedding):
            self.embedding.read_from(self.head, store)

    # ------------------------------------------------------------------ the step
    def embed(self, ctx, out=None) -> torch.Tensor:
        """The residual stream before the first run: float32 [T, hidden] (into `out` if given)."""
        return self.embedding.forward(ctx, out=out)

    def forward(self, ctx) -> torch.Tensor:
        """The residual stream after every run: float32 [T, hidden]."""
        x = self.embed(ctx)
        self.forward_runs(ctx, x, 0, len(self.order))
        return x

    def forward_runs(self, ctx, x: torch.Tensor, first: int, end: int) -> None:
        """Runs first .. end - 1 of the execution order on the residual stream x, in place."""
        normed = None        # the next block's first norm, where the block before it did its work
        for i in range(first, end):
            run, binding = self.order[i], self.cache_plan.bindings[i]
            block = self.blocks[run.layer]
            following = None
            if i + 1 < end:
                after = self.blocks[self.order[i + 1].layer]
                following = block.following_of(ctx, block.last_part(), after.first_norm(), x.shape[0])
            if normed is None and following is None:
                block.forward(ctx, binding, x)          # a block that knows nothing of this is called plainly
            else:
                block.forward(ctx, binding, x, normed, following)
            normed = None if following is None else following.values

    def run_is_graph_safe(self, i: int) -> bool:
        """Whether run i's block and its parts are all fixed launch sequences (see Part.graph_safe)."""
        block = self.blocks[self.order[i].layer]
        return all(getattr(p, "graph_safe", False) for p in (block, block.mixer, block.feed_forward))

    def ends_are_graph_safe(self) -> bool:
        """Whether what runs before the first run and behind the last (`embed`, `logits`) is a fixed
        launch sequence too, so that it can be captured with the runs beside it."""
        return all(getattr(p, "graph_safe", False) for p in (self.embedding, self.final_norm, self.head))

    def logits(self, ctx, x: torch.Tensor, rows: torch.Tensor, out=None) -> torch.Tensor:
        """Final norm and head at the rows asked for: float32 [len(rows), vocab]."""
        h = self.final_norm.forward(ctx, x, rows=rows)
        return self.head.forward(ctx, h, out)
