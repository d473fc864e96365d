"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from its spec (``shrike_amd.config.specs``) and the model's
width; it never sees which model it is in.  It declares the tensors it needs
(`params`), takes them (`load`), and runs on a step's flat token batch
(`forward`).  Kinds of parts:

* Norm:              forward(ctx, hidden) -> normed [N, width] in the compute dtype;
                     folds hidden.pending into hidden.resid first.
* PositionEncoding:  tells a mixer how queries and keys depend on position.
* Mixer:             forward(ctx, x, cache) -> [N, width]; mixes information
                     between the tokens of a sequence, through `cache`
                     (pages of keys/values, or a state slot per request).
* FeedForward:       forward(ctx, x) -> [N, width]; token by token.
* Block:             forward(ctx, hidden, cache) ; arranges norms, mixer and
                     feed-forward around the residual stream.
* Embedding:         forward(ctx) -> float32 [N, width], the residual stream's
                     first value, from ctx.token_ids (and ctx.positions).
* Head:              forward(ctx, x) -> float32 [R, vocab] from the normed rows.
* SideInput:         forward(ctx, hidden, x) ; something else that a layer adds to
                     the stream from the step's tokens (a per-layer token input).

Any part may implement prepare(shape): it is called once per step, before the
step's metadata goes to the device, with the host-side StepShape; there a part
decides how its kernels will be launched and adds the index arrays they need.

To add a part: write its spec dataclass with a unique ``kind``, write the
class, and register it with the matching ``register_*`` function.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part needs from the weight file.

    init: how the random-weights mode draws it: "matrix", "embedding" and
        "bias" are N(0, 0.02), "norm" is 1 + N(0, 0.1); the "unit" mode scales
        a "matrix" by its fan-in and leaves an "embedding" at N(0, 1).
    keep_float32: held in float32 whatever the compute dtype (vectors that
        enter float32 arithmetic); others are held in the compute dtype.
    shape: a size may be None where the file's tensor decides it (the rows of a
        table that config.json does not count); random weights then take
        `free_size` for it.
    """

    name: str
    shape: tuple
    init: str = "matrix"
    keep_float32: bool = False
    optional: bool = False
    free_size: int = 1

    def matches(self, shape) -> bool:
        """Whether a file's tensor of this shape is what the part declared."""
        shape = tuple(shape)
        return len(shape) == len(self.shape) and all(
            (want is None and got >= 1) or want == got for want, got in zip(self.shape, shape))

    def drawn_shape(self) -> tuple[int, ...]:
        """The shape that random weights take."""
        return tuple(self.free_size if d is None else int(d) for d in self.shape)


PAGE = "page"  # in a PageTensor's dims: the place of the page size


@dataclass(frozen=True)
class PageTensor:
    """One tensor that a mixer keeps for every page of a sequence.  `dims` is the
    shape of one page's part of it, ints and PAGE (the page size, which only the
    engine's options fix); the layout within a page is the mixer's own business
    and that of its kernels.  `dtype` None: the compute dtype."""

    name: str
    dims: tuple
    dtype: str | None = None

    def shape(self, page_size: int) -> tuple[int, ...]:
        return tuple(page_size if d == PAGE else int(d) for d in self.dims)

    def numel(self, page_size: int) -> int:
        n = 1
        for d in self.shape(page_size):
            n *= d
        return n


@dataclass(frozen=True)
class PagedSpec:
    """Cache need of a mixer: something per token, kept in pages, for all earlier
    tokens (window None) or for the last `window` of them; with `chunk`, only for
    the tokens of the current block of `chunk` positions (blocks counted from
    position 0).  The cache manager allocates every listed tensor as [layers,
    pages + 1, *dims] and hands a layer its slice under the tensor's name; it
    knows nothing else about them."""

    tensors: tuple[PageTensor, ...]
    window: int | None = None
    chunk: int | None = None

    def first_needed(self, position: int) -> int:
        """The oldest position that a query at `position` (or any later one) still reads."""
        lo = 0
        if self.window is not None:
            lo = max(lo, position - self.window + 1)
        if self.chunk is not None:
            lo = max(lo, position // self.chunk * self.chunk)
        return lo

    @property
    def bounded(self) -> bool:
        """Whether old pages fall out of reach as a sequence grows."""
        return self.window is not None or self.chunk is not None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged cache needs tensors with distinct names, got {names}")


@dataclass(frozen=True)
class StateSpec:
    """Cache need of a mixer: one tensor of fixed shape per request."""

    shape: tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class CompositeSpec:
    """Cache need of a mixer that is made of several mixers: ((sub-name, PagedSpec |
    StateSpec), ...), one entry for each of them that keeps something.  The mixer gets a
    LayerCache whose `parts[sub-name]` is the LayerCache of that entry."""

    parts: tuple

    def __post_init__(self):
        names = [name for name, _ in self.parts]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a composite cache needs entries with distinct names, got {names}")
        if any(not isinstance(spec, (PagedSpec, StateSpec)) for _, spec in self.parts):
            raise TypeError("the entries of a composite cache are PagedSpec or StateSpec")


class HiddenState:
    """The residual stream of a step: `resid` float32 [N, width], plus a part's
    output `pending` (compute dtype, or the partial sums of a split product) that
    has not been added yet.  The next norm adds it while it reads the row anyway.
    `pending_norm` = (weight float32 [width], eps) says that `pending` joins the
    stream as pending * rsqrt(mean(pending^2) + eps) * weight, row by row;
    (weight, bias, eps) that it joins as its layer norm, (pending - mean) /
    sqrt(var + eps) * weight + bias.  `cast`: the stream as it stands (nothing pending) in the
    compute dtype, where the kernel that wrote `resid` last left such a copy."""

    __slots__ = ("resid", "pending", "pending_norm", "cast")

    def __init__(self, resid: torch.Tensor, pending: torch.Tensor | None = None, pending_norm=None):
        self.resid = resid
        self.pending = pending
        self.pending_norm = pending_norm
        self.cast = None

    def settle(self, ctx) -> None:
        """Adds what is pending to `resid` now (for a reader that is no norm)."""
        from ..kernels import ops

        if self.pending is None:
            return
        self.cast = None
        if self.pending_norm is not None and len(self.pending_norm) == 3:
            ops.add_layernorm(self.resid, self.pending, dnorm=self.pending_norm, dtype=ctx.dtype)
        elif self.pending_norm is not None:
            weight, eps = self.pending_norm
            ops.add_normed_rmsnorm(self.resid, self.pending, weight, eps, dtype=ctx.dtype)
        else:
            ops.add_deltas(self.resid, self.pending, dtype=ctx.dtype)
        self.pending = self.pending_norm = None


class Part:
    """Common face of every part."""

    # False for a part whose forward cannot be recorded into a HIP graph (it reads
    # device data on the host, or launches work whose shape depends on the data);
    # a model with such a part runs every step kernel by kernel.
    graph_safe = True
    # True for a part whose launches (kernels, their scalar arguments, the buffers
    # they name) follow from the step's shape alone: the numbers of tokens, sequences,
    # single tokens and wanted rows, the widths of the block tables, the sizes of the
    # arrays that parts added, and the step's launch key.  Steps of equal shape then
    # run such a model's forward from a recorded list of launches.  A part that
    # decides anything else on the host per step must put it into the launch key.
    launches_follow_shape = False

    def __init__(self, spec, width: int, name: str):
        self.spec = spec
        self.width = width
        self.name = name

    def tensor_name(self, role: str, default: str | None = None) -> str:
        """Full name of the tensor that plays `role` for this part: the part's name plus
        the sub-name that the spec's `names` gives the role, else plus `default`
        (the role itself when none is given); an empty sub-name is the part's own name."""
        sub = dict(getattr(self.spec, "names", ()) or ()).get(role, role if default is None else default)
        return f"{self.name}.{sub}" if sub else self.name

    def params(self) -> list[ParamSpec]:
        return []

    def load(self, tensors: dict[str, torch.Tensor], runtime) -> None:
        """`tensors` maps each declared name to a device tensor."""

    def check(self, runtime) -> None:
        """Raise if the kernels cannot take this part's sizes."""

    def prepare(self, shape) -> None:
        """Called once per step with the host-side StepShape, before anything is
        copied to the device: decide launches, `shape.add` index arrays,
        leave `shape.notes` for forward, extend `shape.launch_key`."""


class Norm(Part):
    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def rotary_table(self):
        """(inv_freq float32 [rot_dim/2], rot_dim) when the encoding is a
        half-split rotation that the cache-write kernel applies; else None."""
        return None

    def apply(self, ctx, qkv: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> None:
        """Encode queries and keys of qkv in place (for encodings without a fused kernel)."""
        raise NotImplementedError


class Mixer(Part):
    # A mixer whose cache is a StateSpec is recorded into HIP graphs only if it
    # says that its forward finds its state through ctx.state_slots and
    # ctx.fresh on the device (nothing read on the host, no launch that depends
    # on which slots the step uses).
    state_graph_safe = False

    def cache_spec(self):
        """PagedSpec, StateSpec or None."""
        return None

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        raise NotImplementedError


class SideInput(Part):
    """Adds to the stream from the step's tokens, after a block's sublayers.  `x` is
    the stream in the compute dtype as it stands (nothing pending); the part leaves
    its contribution in hidden.pending (and hidden.pending_norm)."""

    def forward(self, ctx, hidden: HiddenState, x: torch.Tensor) -> None:
        raise NotImplementedError


class Embedding(Part):
    """Built from a spec with `vocab_size`; `table` is what a tied head may share."""

    table: torch.Tensor | None = None

    def forward(self, ctx) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Logits from the normed rows.  `tie(embedding)` is called before load when
    the model ties its output matrix to the embedding."""

    def tie(self, embedding: Embedding) -> None:
        raise NotImplementedError

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


_REGISTRIES: dict[str, dict[str, Callable]] = {
    "norm": {},
    "position": {},
    "mixer": {},
    "ffn": {},
    "block": {},
    "embedding": {},
    "head": {},
    "side": {},
}


def _register(family: str, kind: str, cls) -> None:
    _REGISTRIES[family][kind] = cls


def register_norm(kind: str, cls) -> None:
    _register("norm", kind, cls)


def register_position(kind: str, cls) -> None:
    _register("position", kind, cls)


def register_mixer(kind: str, cls) -> None:
    _register("mixer", kind, cls)


def register_ffn(kind: str, cls) -> None:
    _register("ffn", kind, cls)


def register_block(kind: str, cls) -> None:
    _register("block", kind, cls)


def register_embedding(kind: str, cls) -> None:
    _register("embedding", kind, cls)


def register_head(kind: str, cls) -> None:
    _register("head", kind, cls)


def register_side(kind: str, cls) -> None:
    _register("side", kind, cls)


def build_part(family: str, spec, width: int, name: str):
    """The part registered for ``spec.kind`` in `family`, built for `width`."""
    kind = getattr(spec, "kind", None)
    try:
        cls = _REGISTRIES[family][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES[family])) or "none"
        raise ValueError(f"no {family} part of kind {kind!r} is registered (known: {known})") from None
    return cls(spec, width, name)
