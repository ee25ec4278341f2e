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
    positions are ever read, so earlier pages can be given back."""
    entries: int
    heads: int
    head_dim: int
    window: int = 0

    def group_key(self):
        return (self.entries, self.heads, self.head_dim, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state a mixer wants for one run: `elems` 32-bit floats, zeroed
    when a request starts."""
    elems: int


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


class UnscaledRows:
    """Rows of a norm that still lack their scale: `values` [T, size] in the compute dtype hold
    x * gain, `squares` float32 [T, size / 16] the sums of x^2 over the 16-column parts of each
    row, `eps` the norm's constant.  The product that reads them multiplies its result by
    1 / sqrt(sum(squares) / size + eps): the scale is common to a row, so it commutes with the
    product, and the norm needs no pass of its own over the rows."""

    def __init__(self, values, squares, eps: float):
        self.values, self.squares, self.eps = values, squares, eps

    @property
    def shape(self):
        return self.values.shape


class NormFold:
    """A norm handed to the part that runs before it: that part's last product, which adds into
    the residual stream, does the norm's work in its epilogue, and `rows()` is then what the
    part after the norm reads.  In parts (`squares` given): the product writes `values` =
    residual * gain and `squares` (see UnscaledRows), and the next product applies the rows'
    scale.  Whole (`squares` None): the product writes the finished norm into `values`."""

    def __init__(self, gain, eps: float, values, squares):
        self.gain, self.eps, self.values, self.squares = gain, eps, values, squares

    def following_norm(self):
        return (self.gain, self.values, self.squares, self.eps)

    def rows(self):
        return self.values if self.squares is None else UnscaledRows(self.values, self.squares, self.eps)


class Norm(Part):
    def forward(self, ctx, x, out=None):
        raise NotImplementedError

    def fold(self, ctx, n_rows: int, whole: bool = False) -> Optional[NormFold]:
        """This norm as work for the neighbouring products (with buffers for `n_rows` rows), or
        None if it has to run on its own.  `whole`: for a product that finishes the norm itself."""
        return None


class PositionEncoding(Part):
    def tables(self, ctx):
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
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

    def takes_unscaled_rows(self, ctx) -> bool:
        """Whether `h` may be UnscaledRows in this step (the first product applies the scale)."""
        return False

    def folds_following_norm(self, ctx) -> bool:
        """Whether `forward` takes a NormFold (in parts) as a further argument in this step and fills it."""
        return False

    def finishes_following_norm(self, ctx) -> bool:
        """Whether `forward` takes a whole NormFold in this step: its last product also writes the
        finished norm of the rows it has added into."""
        return False

    def forward(self, ctx, binding: CacheBinding, h, residual) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def takes_unscaled_rows(self, ctx) -> bool:
        return False

    def folds_following_norm(self, ctx) -> bool:
        return False

    def finishes_following_norm(self, ctx) -> bool:
        return False

    def forward(self, ctx, h, residual) -> None:
        raise NotImplementedError


class Block(Part):
    """An arrangement: built from the layer's parts, not from a spec of its own."""

    def __init__(self, norm_factory: Callable[[str], Norm], mixer: Mixer, feed_forward: FeedForward, prefix: str):
        super().__init__({}, prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward

    def first_norm_fold(self, ctx, n_rows: int, whole: bool = False) -> Optional[NormFold]:
        """The block's first norm as work for the block before it (see NormFold; `whole` if that
        block finishes the norm itself), or None: then `forward` is called without `unscaled`."""
        return None

    def folds_following_norm(self, ctx) -> bool:
        """Whether `forward` takes the next block's first norm (in parts) as `fold_next` in this step."""
        return False

    def finishes_following_norm(self, ctx) -> bool:
        """Whether `forward` takes the next block's first norm whole as `fold_next` in this step."""
        return False

    def forward(self, ctx, binding: CacheBinding, x, unscaled: Optional[UnscaledRows] = None,
                fold_next: Optional[NormFold] = None) -> None:
        """Update the residual stream x in place.  `unscaled`: the first norm's rows, already left
        by the block before; `fold_next`: to be filled for the block after (both only if this
        block offered it)."""
        raise NotImplementedError


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
