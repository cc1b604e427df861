"""Interfaces of the parts a model is put together from, and their registries.

A model is data: a ``ModelSpec`` lists layers, each layer names its parts by kind with
their sizes and constants as plain arguments, and a schedule lists the order in which
layers run.  The kinds are looked up here, so a new mixer, feed-forward, norm,
position encoding or block arrangement is one class and one ``register_*`` call; no
part knows which model it is in.

The reference composes fixed classes instead (kvcore/model/models/llama3.py:107-142);
its parts take their constants partly as parameters (layer/attention.py:19-31,
layer/rmsnorm.py:8) and partly from the config object (layer/rotary_embedding.py:53).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any, Callable

import torch

if TYPE_CHECKING:
    from kvcore_amd.engine.context import LayerCall, StepContext


# ------------------------------------------------------------------------ parameters
@dataclass(frozen=True)
class ParamSource:
    """One checkpoint tensor that fills rows ``[row, row + rows)`` of a parameter.
    ``name`` is relative to the part's checkpoint prefix."""

    name: str
    row: int
    rows: int


@dataclass(frozen=True)
class ParamSpec:
    """A parameter a part owns.

    ``kind``: ``"matrix"`` is kept in the model dtype; ``"vector"`` is always float32
    (norm gains and the like, whatever the file stores); ``"table"`` is int32.
    ``init`` names the rule of the random-weights mode: ``"normal"`` N(0, 0.02),
    ``"gain"`` 1 + N(0, 0.1), ``"zeros"``.
    ``sources`` empty means one checkpoint tensor of the same name and shape.
    ``alias_of`` names another parameter (by full name) whose storage this one shares;
    a checkpoint tensor for an alias is optional.
    """

    name: str
    shape: tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    sources: tuple[ParamSource, ...] = ()

    def resolved_sources(self) -> tuple[ParamSource, ...]:
        return self.sources or (ParamSource(self.name, 0, self.shape[0]),)


@dataclass(frozen=True)
class CacheNeed:
    """Paged memory that grows with the sequence.  ``planes`` lists what the mixer keeps per
    token, a shape for each plane: keys and values of 8 heads of 128 are ``((8, 128), (8,
    128))`` (:meth:`keys_and_values`), one compressed vector of 512 is ``((512,),)``, keys and
    values of different widths are two shapes that differ.  A page of a plane holds
    ``page_size`` tokens' worth of that shape in one contiguous piece; how the tokens lie
    inside the page is the mixer's own business (``CacheGroupView.plane`` hands out pages as
    flat rows, the mixer views them).  ``window`` 0 keeps every token, ``w > 0`` only the last
    ``w`` (pages wholly behind the window are given back during the request).
    ``page_size``: tokens per page if the mixer's kernels want a size of their own (None: the
    engine's ``block_size``); ``dtype``: the cache's element type (None: the model's).  Mixers
    with equal needs share a cache group; a group has its own page size, page count, pool,
    storage and block table."""

    planes: tuple[tuple[int, ...], ...]
    window: int = 0
    page_size: int | None = None
    dtype: torch.dtype | None = None

    def __post_init__(self) -> None:
        planes = tuple(tuple(int(n) for n in shape) for shape in self.planes)
        if not planes or any(not shape or min(shape) <= 0 for shape in planes):
            raise ValueError(f"a cache need names at least one plane of positive sizes, got {self.planes!r}")
        object.__setattr__(self, "planes", planes)

    @classmethod
    def keys_and_values(cls, num_kv_heads: int, head_dim: int, window: int = 0,
                        page_size: int | None = None, dtype: torch.dtype | None = None) -> "CacheNeed":
        """Two planes of ``num_kv_heads`` heads of ``head_dim``: what attention keeps."""
        shape = (num_kv_heads, head_dim)
        return cls((shape, shape), window, page_size, dtype)

    def token_elems(self) -> tuple[int, ...]:
        """Elements that one token takes in each plane."""
        out = []
        for shape in self.planes:
            n = 1
            for size in shape:
                n *= size
            out.append(n)
        return tuple(out)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size, kept in a slot array ``[max_seqs, *shape]``."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class RunLimits:
    """The sizes a runner runs a part at.  ``page_size`` and ``max_pages_per_seq`` are those
    of the part's cache group (0 if it has none)."""

    max_num_seqs: int
    max_num_tokens: int
    max_model_len: int
    page_size: int = 0
    max_pages_per_seq: int = 0


@dataclass(frozen=True)
class Runtime:
    """What a part needs to know about where it runs."""

    dtype: torch.dtype
    device: torch.device


class Part:
    """Base of all parts: declares parameters, receives them bound to device tensors.

    ``graph_safe``: the part's forward only launches work on the current stream with
    arguments fixed by the batch's size, so a step may be captured into a HIP graph and
    replayed.  A part that reads device data on the host or loops over requests in Python
    sets it to False, and the engine then runs every step launch by launch."""

    graph_safe = True

    def param_specs(self) -> list[ParamSpec]:
        return []

    def product_weights(self) -> tuple[str, ...]:
        """Local names of the parameters that this part hands to ``ops.linear`` and its
        kin as weight matrices: the model may keep a second copy of them in the order in
        which decode steps stream them (``ops.pack_weight``)."""
        return ()

    def setup(self, runtime: Runtime) -> None:
        """Called once after construction, before parameters are bound."""
        self.runtime = runtime

    def check_limits(self, limits: "RunLimits") -> None:
        """Called when a runner is built around the model, with the sizes it will run at:
        raise here, with a message that names the option to change, if a kernel of this part
        cannot serve them (so that nothing is refused in the middle of a generation)."""

    def bind(self, params: dict[str, torch.Tensor]) -> None:
        """``params`` maps the local names of ``param_specs`` to device tensors."""
        self.params = params


class Norm(Part):
    """``forward_fused`` adds ``delta`` (may be None) into the float32 ``residual`` in
    place and writes the normalised rows into ``out`` (model dtype).

    ``as_gain`` returns ``(gain [H] float32, eps)`` if the norm is ``x * rsqrt(mean(x^2) +
    eps) * gain``, so that the products around it may do its work (a product's epilogue adds
    into the residual and keeps the sums of squares, the next product applies the scale
    factor); None keeps the norm a step of its own."""

    def forward_fused(self, out: torch.Tensor, residual: torch.Tensor,
                      delta: torch.Tensor | None) -> None:
        raise NotImplementedError

    def as_gain(self) -> "tuple[torch.Tensor, float] | None":
        return None


class PositionEncoding(Part):
    """Position information.  ``prepare`` runs once per step before any layer.
    ``rotary`` returns what a mixer needs to rotate queries and keys, or None if this
    encoding does not rotate; ``embed`` may change the embedded rows in place."""

    def prepare(self, ctx: "StepContext") -> None:
        pass

    def rotary(self, ctx: "StepContext") -> "RotaryTables | None":
        return None

    def embed(self, residual: torch.Tensor, ctx: "StepContext") -> None:
        pass


@dataclass
class RotaryTables:
    cos: torch.Tensor  # [>= T, rot_dim / 2] float32
    sin: torch.Tensor
    rot_dim: int
    interleaved: bool


class Embedding(Part):
    """Token ids to rows of the residual stream: ``forward`` writes ``residual [T, H]``
    (float32) for ``token_ids [T]`` (int32 on the device).  A parameter named ``weight`` of
    shape ``[vocab, hidden]`` is what a tied head shares."""

    def forward(self, residual: torch.Tensor, token_ids: torch.Tensor) -> None:
        raise NotImplementedError


class Head(Part):
    """Normalised hidden rows to logits: ``forward`` writes float32 ``logits [S, V]`` from
    ``hidden_rows [S, H]`` in the model dtype.  ``tied``: the head owns no matrix; the model
    binds the embedding's ``weight`` to it under the same name."""

    tied = False

    def forward(self, logits: torch.Tensor, hidden_rows: torch.Tensor, ctx: "StepContext") -> None:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information across the tokens of a request.  ``x`` is ``[T, hidden]`` in
    the model dtype; the result has the same shape and may live in a step buffer.

    ``takes_scaled_rows``: ``x`` may also be an ``ops.ScaledRows`` (rows whose norm the first
    product finishes), because the part only hands ``x`` to ``ops.linear``.  ``takes_sink``:
    ``forward`` has a keyword ``sink`` (an ``ops.ResidualSink`` or None); given one, the last
    product goes into it through ``ops.linear`` and what that returns (``ops.ScaledRows`` or
    ``ops.NormedRows``) is returned instead of a tensor."""

    takes_scaled_rows = False
    takes_sink = False

    def cache_need(self) -> CacheNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x: torch.Tensor, ctx: "StepContext", call: "LayerCall") -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """``takes_scaled_rows`` and ``takes_sink`` as for :class:`Mixer`."""

    takes_scaled_rows = False
    takes_sink = False

    def forward(self, x: torch.Tensor, ctx: "StepContext", call: "LayerCall") -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, mixer and feed-forward around the residual stream.
    ``forward`` takes the pending ``delta`` (output of the previous block not yet added,
    or None) and the float32 ``residual``, and returns the new pending delta."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm]) -> None:
        self.mixer = mixer
        self.ffn = ffn
        self.norms = norms

    def children(self) -> dict[str, Part]:
        """Checkpoint sub-prefix -> part."""
        raise NotImplementedError

    # ---- what any arrangement needs to let the products around a norm do the norm's work
    # (see ``ops.ResidualSink``): which of the two ways a step of this size takes, and the
    # sink itself.  A block that does not use them gets ordinary tensors and separate norms.
    @staticmethod
    def norm_folding(ctx: "StepContext", width: int) -> tuple[bool, bool]:
        """``(fold, sums)`` for this step: ``fold``, up to 16 rows of bfloat16: the product
        before a norm adds into the residual and keeps sums of squares, the product after it
        applies the scale factor (``ops.ScaledRows``); ``sums``, a few dozen rows: the product
        before a norm leaves partial sums of slices along K and one kernel adds them into the
        residual and normalises (``ops.NormedRows``).  Never both."""
        from kvcore_amd.ops import library as ops

        ok = width % 8 == 0
        return (ok and ops.rows_fusable(ctx.num_tokens, ctx.dtype),
                ok and ops.rows_sinkable(ctx.num_tokens, ctx.dtype))

    @staticmethod
    def residual_sink(ctx: "StepContext", residual: torch.Tensor, gain: "tuple[torch.Tensor, float]",
                      name: str, fold: bool):
        """The ``ops.ResidualSink`` that a part's last product goes into instead of a tensor:
        ``gain`` is the following norm's ``as_gain()``, ``name`` the step buffer that receives
        the rows for the part after the norm, ``fold`` as ``norm_folding`` says."""
        from kvcore_amd.ops import library as ops

        H = residual.shape[1]
        rows = ctx.buf(name, H)
        if fold:
            parts = ctx.buffers.get(name + "_ss", ops.SKINNY_PREFERRED_ROWS, -(-H // 16), torch.float32)
            return ops.ResidualSink(residual, gain[0], gain[1], rows, parts)
        slices = ctx.buffers.get("block_slices", ops.mid_slices_bound(H) * ops.MID_ROWS, H, torch.float32)
        return ops.ResidualSink(residual, gain[0], gain[1], rows, None, slices)

    def input_gain(self, scaled: bool = True) -> "tuple[torch.Tensor, float] | None":
        """``(gain, eps)`` of the block's first norm (see :meth:`Norm.as_gain`) if the block
        before may do that norm's work, else None: with ``scaled`` it hands over
        ``ops.ScaledRows`` that this block's mixer must finish, without it ``ops.NormedRows``
        that are already normalised."""
        return None

    def forward(self, delta: torch.Tensor | None, residual: torch.Tensor, ctx: "StepContext",
                call: "LayerCall", next_block: "Block | None" = None) -> torch.Tensor:
        """``next_block`` is the block that runs after this one (None after the last); the
        result may be ``ops.ScaledRows`` or ``ops.NormedRows`` only if
        ``next_block.input_gain()`` allowed it."""
        raise NotImplementedError


# -------------------------------------------------------------------------- registry
@dataclass(frozen=True)
class PartSpec:
    """A part chosen by kind, with its sizes and constants."""

    kind: str
    args: dict[str, Any] = field(default_factory=dict)


class _Registry:
    def __init__(self, what: str) -> None:
        self.what = what
        self._items: dict[str, Callable[..., Any]] = {}

    def register(self, kind: str, factory: Callable[..., Any], *, replace: bool = False) -> None:
        if kind in self._items and not replace:
            raise ValueError(f"{self.what} kind {kind!r} is already registered")
        self._items[kind] = factory

    def build(self, spec: PartSpec, **extra: Any) -> Any:
        try:
            factory = self._items[spec.kind]
        except KeyError:
            raise ValueError(
                f"Unknown {self.what} kind {spec.kind!r}. Registered: {sorted(self._items)}"
            ) from None
        return factory(**spec.args, **extra)

    def kinds(self) -> list[str]:
        return sorted(self._items)

    def unregister(self, kind: str) -> None:
        self._items.pop(kind, None)


MIXERS = _Registry("mixer")
FEED_FORWARDS = _Registry("feed-forward")
NORMS = _Registry("norm")
POSITION_ENCODINGS = _Registry("position encoding")
BLOCKS = _Registry("block")
EMBEDDINGS = _Registry("embedding")
HEADS = _Registry("head")


def register_mixer(kind: str, factory: Callable[..., Mixer], **kw: Any) -> None:
    MIXERS.register(kind, factory, **kw)


def register_feed_forward(kind: str, factory: Callable[..., FeedForward], **kw: Any) -> None:
    FEED_FORWARDS.register(kind, factory, **kw)


def register_norm(kind: str, factory: Callable[..., Norm], **kw: Any) -> None:
    NORMS.register(kind, factory, **kw)


def register_position_encoding(kind: str, factory: Callable[..., PositionEncoding], **kw: Any) -> None:
    POSITION_ENCODINGS.register(kind, factory, **kw)


def register_block(kind: str, factory: Callable[..., Block], **kw: Any) -> None:
    BLOCKS.register(kind, factory, **kw)


def register_embedding(kind: str, factory: Callable[..., Embedding], **kw: Any) -> None:
    EMBEDDINGS.register(kind, factory, **kw)


def register_head(kind: str, factory: Callable[..., Head], **kw: Any) -> None:
    HEADS.register(kind, factory, **kw)
