"""Interfaces of the parts a model is put together from, and their registries.

A part takes its sizes and constants as constructor parameters and never learns which
model it sits in.  Five kinds exist:

* ``Mixer``: mixes information across the positions of a sequence (attention here).
  It may need cache: pages of keys and values (all of them or a window), and/or a
  fixed-size state per request.
* ``FeedForward``: per-token transformation (dense SwiGLU here; routed experts later).
* ``Norm``: normalisation, fused with the residual add in front of it.
* ``PositionEncoding``: what a mixer consults to encode positions (rotation tables here).
* ``Block``: the arrangement of mixer, feed-forward and norms around the residual stream.
* ``Embedding`` and ``OutputProjection``: the two ends of the model, token ids to the
  residual stream and the last hidden rows to logits.

Every part declares its tensors as :class:`ParamSpec` (``param_specs``), receives them
loaded (``bind``), and runs on a flat batch of tokens described by a
:class:`~rapid_llm_amd.engine.step.StepContext` (``forward``).  The reference reaches the
same seams by constructor injection (rapid_llm/models/base.py:188-216: ``mlp=`` and
``attention=`` arguments of ``DecoderLayer``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any, Callable

if TYPE_CHECKING:  # pragma: no cover
    import torch

    from ..engine.step import StepContext


# --------------------------------------------------------------------------- #
# tensors a part needs
# --------------------------------------------------------------------------- #


@dataclass(frozen=True)
class Source:
    """One checkpoint tensor feeding ``rows`` rows (dim 0) of a parameter."""

    name: str
    rows: int


@dataclass(frozen=True)
class ParamSpec:
    """One tensor of the model as the engine holds it.

    ``sources`` are concatenated along dim 0 in order: a fused matrix such as the packed
    query/key/value projection lists its three checkpoint tensors
    (rapid_llm/modules/linear.py:253-271 writes the same row blocks).

    ``role`` decides the storage type:
      * ``"matrix"``: the engine's compute type; in a bfloat16 engine a tensor the
        checkpoint stores in 32-bit stays 32-bit.
      * ``"vector"``: small per-channel weights (norms); always held in float32, which
        represents a bfloat16 checkpoint value exactly.
      * ``"table"``: integer lookup tables, held as int32.
    ``fallback`` names another parameter whose tensor is shared when the checkpoint has
    none of this one's sources (a tied output projection).
    ``init`` is the distribution the random-weights mode draws the sources from.
    """

    name: str
    shape: tuple[int, ...]
    role: str
    sources: tuple[Source, ...]
    init: str = "normal"  # "normal" | "norm" | "zeros" | "table"
    fallback: str | None = None


@dataclass(frozen=True)
class StateSpec:
    """One fixed-size per-request tensor: ``[slots, *shape]`` on the device."""

    name: str
    shape: tuple[int, ...]
    dtype: str | None = None  # torch dtype name; None: the engine's compute type


@dataclass(frozen=True)
class PagedSpec:
    """One paged tensor of a mixer: what it keeps per position, and where the positions of a
    page lie among that array's axes.

    Per position the mixer keeps an array of ``shape``; the cache holds it as
    ``[pages, *shape[:slot_axis], page_size, *shape[slot_axis:]]``.  Keys of ``h`` heads of ``d``
    channels with ``slot_axis=1`` are ``[pages, h, page_size, d]`` (a key is one contiguous row);
    the same shape with ``slot_axis=2`` is ``[pages, h, d, page_size]`` (stored transposed: the
    positions of a page are contiguous for one channel); one latent row of ``r`` channels per
    token, ``shape=(r,)`` with ``slot_axis=0``, is ``[pages, page_size, r]``
    (rapid_llm/engine/kv_cache_spec.py:171-188 is such a row).
    """

    name: str
    shape: tuple[int, ...]
    slot_axis: int = 0
    dtype: str | None = None  # torch dtype name; None: the engine's compute type

    def __post_init__(self) -> None:
        if not self.shape or any(int(n) < 1 for n in self.shape):
            raise ValueError(f"paged tensor {self.name!r} needs a per-position shape of positive sizes, got {self.shape}")
        if not 0 <= self.slot_axis <= len(self.shape):
            raise ValueError(f"paged tensor {self.name!r}: slot_axis {self.slot_axis} is outside its shape {self.shape}")

    def page_shape(self, pages: int, page_size: int) -> tuple[int, ...]:
        return (pages, *self.shape[: self.slot_axis], page_size, *self.shape[self.slot_axis :])

    def elements(self) -> int:
        """Elements one position costs."""
        count = 1
        for n in self.shape:
            count *= int(n)
        return count


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the cache manager.

    ``kind == "paged"``: tensors that grow with the request, in pages, each named and laid out
    by a :class:`PagedSpec` (keys and values here; a mixer may name one latent row, or keys and
    values of different widths).  ``window`` 0 keeps every position, otherwise only the last
    ``window`` positions of a request are kept and older pages are given back.
    ``kind == "state"``: nothing paged.  Fixed-size per-request tensors the mixer owns, zeroed
    when a request takes the slot, may accompany either kind: one as ``state_shape`` (and
    ``state_dtype``), or several, each under a name, as ``states`` (a mixer with a short
    convolution's tail beside a recurrent state names both).
    ``share_with`` names the place in the run order whose cache this one reads instead of
    writing its own.
    """

    kind: str  # "paged" | "state" | "none"
    window: int = 0
    paged: tuple[PagedSpec, ...] = ()
    state_shape: tuple[int, ...] | None = None
    state_dtype: str | None = None  # torch dtype name; None: the engine's compute type
    share_with: int | None = None
    states: tuple[StateSpec, ...] = ()

    def __post_init__(self) -> None:
        if self.kind not in ("paged", "state", "none"):
            raise ValueError(f"a cache need is 'paged', 'state' or 'none', not {self.kind!r}")
        if (self.kind == "paged") != bool(self.paged):
            raise ValueError(f"a {self.kind!r} cache need names {len(self.paged)} paged tensors")
        names = [p.name for p in self.paged]
        if len(names) != len(set(names)):
            raise ValueError(f"a mixer names two paged tensors alike: {names}")

    @classmethod
    def keys_and_values(cls, num_kv_heads: int, head_dim: int, window: int = 0, **more) -> "CacheNeed":
        """The layout the attention kernels of this package read: keys ``[pages, heads,
        page_size, head_dim]`` under ``"k"``, values transposed ``[pages, heads, head_dim,
        page_size]`` under ``"v"``."""
        shape = (num_kv_heads, head_dim)
        return cls("paged", window=window, paged=(PagedSpec("k", shape, 1), PagedSpec("v", shape, 2)), **more)

    def state_specs(self) -> tuple[StateSpec, ...]:
        """Every per-request tensor asked for; the one given as ``state_shape`` is named ``"state"``."""
        single = (StateSpec("state", self.state_shape, self.state_dtype),) if self.state_shape is not None else ()
        specs = single + tuple(self.states)
        names = [s.name for s in specs]
        if len(names) != len(set(names)):
            raise ValueError(f"a mixer names two state tensors alike: {names}")
        return specs


class Part:
    """Common protocol: declare tensors, receive them, run."""

    #: A part whose ``forward`` may be recorded once into a HIP graph and replayed for later
    #: steps declares ``replayable = True``.  It promises that everything ``forward`` does on
    #: the host depends only on what is fixed for a recorded step (the number of rows, that
    #: every request brings one token, the context bound in ``ctx.static["context_bound"]``),
    #: that every per-step value (ids, positions, slots, block tables, state) is read on the
    #: device from the tensors of ``ctx`` and of the cache, and that nothing waits for the
    #: device or copies from the host while the step is recorded.  Launch data that depends
    #: only on what a recorded step fixes (index lists, tile tables) is kept in ``ctx.static``:
    #: the step runs once eagerly before it is recorded, what that run left in ``ctx.static`` is
    #: there again during the recording and lives as long as the graph, whereas ``ctx.extra`` is
    #: emptied between the two.  A model with a part that does not declare it runs every step
    #: eagerly.
    replayable = False

    def param_specs(self) -> list[ParamSpec]:
        return []

    def bind(self, params: dict[str, "torch.Tensor"], runtime: Any) -> None:
        """Receive the loaded tensors (keyed by ``ParamSpec.name``) and the runtime
        (device, compute type, kernel library, largest sequence length)."""

    def recorded_step_bytes(self, rows: int, context_bound: int, page_size: int) -> int:
        """Bytes of device memory, beyond a few rows of activations, that one run of this part
        keeps alive inside a recorded step of ``rows`` single tokens over contexts of at most
        ``context_bound`` positions (partial results between two of its kernels, work lists).
        The engine reserves them when it sizes the page pool from what is free."""
        return 0


class PositionEncoding(Part):
    """Supplies what a mixer needs to encode a token's absolute position, and says how it is
    applied; the mixer's kernels do the applying, or refuse what they cannot do.

    A rotary encoding exposes, after ``bind``: ``cos`` and ``sin``, float32
    ``[positions, rotary_dim // 2]``; ``rotary_dim``, the leading channels of a head that
    rotate (the rest pass unrotated); and ``pairing``, which channels form a rotated pair:
    ``"half_split"`` pairs channel ``i`` with ``i + rotary_dim // 2``, ``"interleaved"`` channel
    ``2i`` with ``2i + 1``.  An encoding that rotates nothing leaves ``cos`` and ``sin`` ``None``.
    """

    kind = "none"
    pairing = "half_split"
    rotary_dim = 0
    cos = None
    sin = None


class Mixer(Part):
    def cache_need(self) -> CacheNeed:
        return CacheNeed("none")

    def forward(self, x: "torch.Tensor", ctx: "StepContext", cache: Any) -> "torch.Tensor":
        """``x [T, hidden]`` (normalised) -> the mixer's contribution ``[T, hidden]``.
        ``cache`` is the :class:`~rapid_llm_amd.cache.storage.LayerCache` of this place in
        the run order: a layer that runs twice has a cache for each run."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: "torch.Tensor", ctx: "StepContext") -> "torch.Tensor":
        raise NotImplementedError


class Norm(Part):
    def forward(
        self,
        residual: "torch.Tensor",
        delta: "torch.Tensor | None",
        ctx: "StepContext",
        rows: "torch.Tensor | None" = None,
    ) -> "torch.Tensor":
        """``residual += delta`` (in place, float32) and return ``norm(residual)`` in the
        compute type.  With ``rows`` (int32 indices) only those rows are produced, packed."""
        raise NotImplementedError


class Block(Part):
    def forward(self, residual: "torch.Tensor", delta, ctx: "StepContext", cache: Any):
        """Advance the residual stream through one layer; returns the pending ``delta``
        (the last sub-layer's output, to be added by whoever normalises next)."""
        raise NotImplementedError


class Embedding(Part):
    """Token ids to the float32 residual stream."""

    def forward(self, token_ids: "torch.Tensor", ctx: "StepContext") -> "torch.Tensor":
        """``token_ids [T]`` int32 -> ``[T, hidden]`` float32.  An id ``-(r + 1)`` stands for
        ``ctx.fed_tokens[r]``, the token that row ``r`` of the latest sampling chose on the
        device (:func:`~rapid_llm_amd.engine.feed.fed_token`)."""
        raise NotImplementedError


class OutputProjection(Part):
    """The normalised hidden rows that were asked for to float32 logits ``[rows, vocab]``."""

    def forward(self, h: "torch.Tensor", ctx: "StepContext") -> "torch.Tensor":
        raise NotImplementedError


# --------------------------------------------------------------------------- #
# registries: kind name -> constructor
# --------------------------------------------------------------------------- #


@dataclass
class PartRegistry:
    what: str
    _table: dict[str, Callable[..., Any]] = field(default_factory=dict)

    def register(self, kind: str, ctor: Callable[..., Any] | None = None, *, replace=False):
        def _do(c):
            if kind in self._table and not replace:
                raise ValueError(f"{self.what} kind {kind!r} is already registered")
            self._table[kind] = c
            return c

        return _do if ctor is None else _do(ctor)

    def unregister(self, kind: str) -> None:
        self._table.pop(kind, None)

    def create(self, kind: str, /, **params: Any) -> Any:
        try:
            ctor = self._table[kind]
        except KeyError:
            raise ValueError(
                f"unknown {self.what} kind {kind!r}; known: {', '.join(sorted(self._table))}"
            ) from None
        return ctor(**params)

    def kinds(self) -> list[str]:
        return sorted(self._table)


MIXERS = PartRegistry("mixer")
FEED_FORWARDS = PartRegistry("feed-forward")
NORMS = PartRegistry("norm")
POSITION_ENCODINGS = PartRegistry("position encoding")
BLOCKS = PartRegistry("block")
EMBEDDINGS = PartRegistry("embedding")
OUTPUT_PROJECTIONS = PartRegistry("output projection")
