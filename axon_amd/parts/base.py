"""The interfaces of a layer's parts, and the registries they are found in.

A model is put together from parts that know nothing of the model they are in: each takes its
sizes and constants as parameters (a `PartSpec`'s `params`), declares the checkpoint tensors
it needs, says what cache or per-request state it wants, and runs on the tokens of a step.

* `Norm.forward(ctx, x, out)`: normalise rows of the 32-bit residual stream into the compute
  dtype.
* `PositionEncoding.tables(ctx)`: whatever the mixer's kernels need for the positions of
  this step, computed once per step and shared by all layers with equal parameters.
* `Mixer.forward(ctx, binding, h, residual)`: mix the tokens of each request (attention here),
  reading and writing the cache `binding` names, and ADD the result to `residual` (32-bit).
* `FeedForward.forward(ctx, h, residual)`: the same shape of call, without a cache.
* `Block.forward(ctx, binding, x)`: the arrangement of norm, mixer and feed-forward around
  the residual stream `x`.

Another part is a subclass registered under a new name (`register_mixer`, ...); a
configuration then names it in a `PartSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

from ..config.base import ConfigError, PartSpec


@dataclass(frozen=True)
class TensorDecl:
    """A checkpoint tensor a part needs.  `role` decides storage and random initialisation:
    "matrix" (compute dtype; normal), "bias" (vector; normal), "gain" (vector; 1 + normal),
    "table" (integers, kept as int32).  An `optional` tensor may be absent."""
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    optional: bool = False


@dataclass(frozen=True)
class CacheSpec:
    """Paged per-token storage a mixer wants for one run: `entries` arrays (keys and values:
    2) of `heads` x `head_dim` elements per position.  `window` > 0: only the last `window`
    positions are ever read, so earlier pages can be given back.  `dtype`: the element type of
    the pages ("float32", "bfloat16", "int8", ...); None: the engine's compute dtype."""
    entries: int
    heads: int
    head_dim: int
    window: int = 0
    dtype: Optional[str] = None

    def group_key(self):
        return (self.entries, self.heads, self.head_dim, self.window, self.dtype)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state a mixer wants for one run: `elems` elements of `dtype`
    (32-bit floats unless it says otherwise), zeroed when a request starts."""
    elems: int
    dtype: str = "float32"


@dataclass
class CacheBinding:
    """What a run of a layer is given by the cache manager: its cache group and its index in
    that group's storage, whether it stores what it computes, and its state arena."""
    group: int = -1
    index: int = -1
    writes: bool = True
    state_index: int = -1


class Part:
    """Common to all parts: tensors in, then bound to device memory.

    `graph_safe`: the part's work in a step is a fixed sequence of kernel launches that read
    everything that changes between steps (tokens, positions, block tables) from device memory,
    so a decoding step can be captured once into a HIP graph and replayed.  A part that
    branches on host values or keeps per-request state must leave it False."""
    graph_safe = False

    def __init__(self, params: Dict[str, Any], prefix: str = ""):
        self.params = dict(params)
        self.prefix = prefix

    def tensors(self) -> List[TensorDecl]:
        return []

    def load(self, store, rt) -> None:
        """Take the declared tensors from `store` (a `WeightStore`); `rt` is the runtime
        (device, dtype, kernels)."""


class FollowingNorm:
    """A norm handed to the part that runs before it (an option, never a duty: a part that does
    not offer it is followed by the norm's own pass).  Where the last product of a part adds into
    the residual stream through a kernel that holds the finished rows anyway, that kernel can
    write the norm of the new rows as well: `values` [T, size] in the compute dtype, the same
    bits as the norm's own pass would give.  The part after the norm then reads `values`."""

    def __init__(self, gain, eps: float, values):
        self.gain, self.eps, self.values = gain, eps, values

    def as_argument(self):
        return (self.gain, self.values, self.eps)


class PrecedingNorm:
    """A norm handed to the part that runs after it (an option, never a duty: a part that does
    not say `applies_preceding_norm` gets the normed rows as always).  Where the first product of a
    part can norm its operand on the way, the norm is no pass of its own: the part gets this
    object in place of the normed rows, with the float32 `rows` [T, size], the `gain` and `eps`,
    and gives the same bits as the norm's own pass followed by its product.  `apply(ctx)` is that
    pass, for a part that finds in the middle of a step that it cannot after all."""

    def __init__(self, norm, rows):
        self.norm, self.rows, self.gain, self.eps = norm, rows, norm.gain, norm.eps

    @property
    def shape(self):
        return self.rows.shape

    def apply(self, ctx):
        return self.norm.forward(ctx, self.rows)


class Norm(Part):
    def forward(self, ctx, x, out=None):
        raise NotImplementedError

    def preceding(self, ctx, x) -> Optional[PrecedingNorm]:
        """This norm of the rows x as work for the first product of the part after it, or None if
        it always runs on its own (the default).  What is handed over is (gain, eps): the RMS
        norm's arithmetic.  A norm of another kind does not offer itself, runs as a pass of its
        own, and is right, only a launch slower."""
        return None

    def following(self, ctx, n_rows: int) -> Optional[FollowingNorm]:
        """This norm as work for the product before it (with a buffer for `n_rows` rows), or None
        if it always runs on its own (the default)."""
        return None


class PositionEncoding(Part):
    def tables(self, ctx):
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def max_context(self) -> Optional[int]:
        """The most positions of a request this mixer's kernels take (None: no limit of its own).
        The engine refuses a longer `max_seq_len` when it is built, not in the middle of a step."""
        return None

    def decode_shape(self, positions) -> Optional[Tuple[Any, Any]]:
        """For a step of single tokens at `positions`: (name, value) if the launches of this
        mixer depend on more than the number of tokens (say, on how long the contexts are), so
        that a captured graph is replayed only for steps of the same shape.  The pair is handed
        back in `ctx.decode_shapes[name]`.  None: nothing else matters."""
        return None

    def decode_input(self, positions) -> Optional[Tuple[Any, Sequence[int]]]:
        """For a step of single tokens at `positions`: (name, int32 values) that this mixer's
        kernels read from the device (say, a list of the work to launch), or None.  The engine
        copies the values into a buffer that stays where it is (a captured graph reads it again
        at every replay) and hands it back as `ctx.decode_inputs[name]`; how many values there
        are is part of the step's shape, so pad them to few different lengths."""
        return None

    def decode_input_capacity(self, max_seqs: int, max_seq_len: int) -> int:
        """The most values `decode_input` ever returns with this many live requests of up to
        this many positions each."""
        return 0

    def decode_scratch(self, max_seqs: int, max_seq_len: int) -> Optional[Tuple[Any, int]]:
        """(name, float32 elements) of a workspace this mixer's kernels want in steps of single
        tokens, sized for this many live requests of up to this many positions each, or None.  The
        engine allocates one per name, once, and hands it back as `ctx.decode_scratch[name]`: every
        decoding step and every captured graph then uses the same memory, whatever its shape."""
        return None

    def finishes_following_norm(self, ctx) -> bool:
        """Whether `forward` takes a FollowingNorm as a further argument in this step: its last
        product also writes the finished norm of the rows it has added into.  Optional."""
        return False

    def applies_preceding_norm(self, ctx) -> bool:
        """Whether `forward` takes `h` as a PrecedingNorm in this step: its first product norms
        its operand itself.  Optional."""
        return False

    def forward(self, ctx, binding: CacheBinding, h, residual) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def finishes_following_norm(self, ctx) -> bool:
        """As for a mixer: optional."""
        return False

    def applies_preceding_norm(self, ctx) -> bool:
        """As for a mixer: optional."""
        return False

    def forward(self, ctx, h, residual) -> None:
        raise NotImplementedError


class Block(Part):
    """An arrangement: built from the layer's parts, not from a spec of its own.

    A block that wants the speed of norms finished by the product before them calls
    `run_part` for its mixer and feed-forward and `normed` for its norms (below); one that does
    not calls the parts plainly, and everything still works."""

    def __init__(self, norm_factory: Callable[[str], Norm], mixer: Mixer, feed_forward: FeedForward, prefix: str):
        super().__init__({}, prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward

    def first_norm(self) -> Optional[Norm]:
        """The norm this block starts with, if the block before may do its work; None: it may not."""
        return None

    def last_part(self):
        """The part whose product ends this block (it may finish the next block's first norm)."""
        return None

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following: Optional[FollowingNorm] = None) -> None:
        """Update the residual stream x in place.  `normed`: the first norm's rows, already left by
        the block before; `following`: the next block's first norm, to be finished by this block's
        last product (both only if this block offered it through `first_norm` / `last_part`)."""
        raise NotImplementedError

    # what a block's `forward` is put together from
    @staticmethod
    def following_of(ctx, part, norm: Optional[Norm], n_rows: int) -> Optional[FollowingNorm]:
        """`norm` as work for `part`'s last product in this step, or None."""
        if norm is None or part is None or not part.finishes_following_norm(ctx):
            return None
        return norm.following(ctx, n_rows)


    @staticmethod
    def preceding_of(ctx, norm: Optional[Norm], part, x) -> Optional[PrecedingNorm]:
        """`norm` of the rows x as work for `part`'s first product in this step, or None."""
        if norm is None or part is None or not part.applies_preceding_norm(ctx):
            return None
        return norm.preceding(ctx, x)


# --------------------------------------------------------------------------- registries

_REGISTRIES: Dict[str, Dict[str, Any]] = {k: {} for k in
                                          ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")}


def _register(kind: str, name: str, cls) -> None:
    _REGISTRIES[kind][name] = cls


def _lookup(kind: str, name: str):
    try:
        return _REGISTRIES[kind][name]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES[kind])) or "none"
        raise ConfigError(f"no {kind.replace('_', '-')} part is registered as '{name}' (known: {known})") from None


def register_norm(name, cls): _register("norm", name, cls)
def register_position(name, cls): _register("position", name, cls)
def register_mixer(name, cls): _register("mixer", name, cls)
def register_feed_forward(name, cls): _register("feed_forward", name, cls)
def register_block(name, cls): _register("block", name, cls)
def register_embedding(name, cls): _register("embedding", name, cls)
def register_head(name, cls): _register("head", name, cls)


def build_part(kind: str, spec: PartSpec, prefix: str = "") -> Part:
    return _lookup(kind, spec.kind)(spec.params, prefix)


def build_block(name: str, norm_spec: PartSpec, mixer: Mixer, feed_forward: FeedForward, prefix: str) -> Block:
    def norm_factory(tensor_name: str) -> Norm:
        return build_part("norm", PartSpec(norm_spec.kind, {**norm_spec.params, "tensor": tensor_name}), prefix)
    return _lookup("block", name)(norm_factory, mixer, feed_forward, prefix)
