"""What a model is made of: the kinds of parts, what each must provide, and the
table that maps a part's description to the class that runs it.

A model is described by data (:class:`ModelSpec`): an embedding, a list of layer
descriptions (each naming its mixer, feed-forward, norms and their arrangement),
the order in which layers run, a final norm and an output head. Each description
is a small dataclass with a ``kind``; ``register_part(role, kind, cls)`` says which
class runs it. No part knows which model it is in: it sees its own description,
its own tensors and the step's :class:`~pyre_amd.engine.context.StepContext`.

Interfaces (duck-typed; the base classes document them):

``Part``          ``tensor_specs()`` names the checkpoint tensors it needs;
                  ``bind(tensors, runtime)`` takes them (already on the device).
``Mixer``         ``cache_spec()`` says what it keeps per token (tensors in pages, in a
                  layout of its own choice, all tokens or a window) or per request
                  (fixed-size state), or nothing; ``step_arrays()`` names the work
                  lists its kernels want of every step; ``forward(ctx, h, cache) -> Partials`` turns the normed
                  hidden rows into the term to be added to the residual stream.
``FeedForward``   ``forward(ctx, h) -> Partials``.
``Norm``          ``forward(ctx, resid, delta, out, rows=None)``: adds ``delta`` to the
                  fp32 residual stream and writes the normed rows to ``out``.
``PositionEncoding``  ``rotary(runtime) -> (cos, sin, rotary_dim)`` tables indexed by
                  absolute position for mixers that rotate queries and keys, or
                  ``rotary_dim = 0`` for none.
``Block``         ``forward(ctx, state, caches)`` arranges the four above around the
                  residual stream; ``cache_specs()`` lists what the block keeps (one
                  description per cache: a block with one mixer has its mixer's, a block
                  with two has two, in the order in which ``forward`` receives their
                  views) and ``step_arrays()`` what its parts want of every step. The
                  model asks the block, never the parts inside it.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar

# --------------------------------------------------------------------------- tensors


@dataclass(frozen=True)
class TensorSpec:
    """One checkpoint tensor a part needs.

    ``init`` tells the random-weights mode how to draw it: ``"normal"`` (matrices,
    embeddings, biases: N(0, std)), ``"gain"`` (norm gains: 1 + N(0, gain_std)),
    ``"zeros"``, ``"int"`` (integer tables: zeros).
    ``alias_of`` names a tensor that stands in when this one is absent from the
    file (a tied output head).
    """

    name: str
    shape: tuple[int, ...]
    init: str = "normal"
    alias_of: str | None = None


# --------------------------------------------------------------------------- cache needs


@dataclass(frozen=True)
class PagedTensorSpec:
    """One tensor that a mixer keeps per token, in pages.

    ``token_shape`` is what one token owns, for instance ``(kv_heads, head_dim)`` for a
    key. A page of ``page_size`` tokens has the token axis inserted at ``token_axis``:
    ``token_axis = 1`` on ``(kv_heads, head_dim)`` gives pages of ``(kv_heads, page_size,
    head_dim)`` (every head's keys of a page lie together), ``token_axis = 2`` gives
    ``(kv_heads, head_dim, page_size)`` (transposed: runs of tokens), ``token_axis = 0``
    gives ``(page_size, ...)`` (one record per token). The layout is the mixer's choice,
    made for its kernels; the cache manager only allocates what it is told.
    ``dtype`` is "model" (the engine's element type) or "float32".
    """

    name: str
    token_shape: tuple[int, ...]
    token_axis: int = 0
    dtype: str = "model"

    def __post_init__(self) -> None:
        if not (0 <= self.token_axis <= len(self.token_shape)):
            raise ValueError(f"paged tensor {self.name!r}: token_axis {self.token_axis} does not fit "
                             f"token_shape {self.token_shape}")
        if self.dtype not in ("model", "float32"):
            raise ValueError(f"paged tensor {self.name!r}: dtype must be 'model' or 'float32'")

    def page_shape(self, page_size: int) -> tuple[int, ...]:
        s = list(self.token_shape)
        s.insert(self.token_axis, page_size)
        return tuple(s)

    def elements_per_token(self) -> int:
        n = 1
        for d in self.token_shape:
            n *= d
        return n


@dataclass(frozen=True)
class PagedCacheSpec:
    """What a mixer keeps per token: one or more tensors in pages that share a block
    table. ``window`` = 0 keeps every token; ``window`` = W keeps the last W (a query at
    position p sees p-W+1 .. p), and pages that no later query can see are given back."""

    tensors: tuple[PagedTensorSpec, ...]
    window: int = 0
    #: tokens per page that this mixer's kernels need, if they need a particular number; None:
    #: whatever the engine is set to. All page groups of an engine share one page size, so an
    #: engine set to another size refuses the model when it is built.
    page_size: int | None = None

    kind: ClassVar[str] = "paged"

    def __post_init__(self) -> None:
        names = [t.name for t in self.tensors]
        if not names or len(names) != len(set(names)):
            raise ValueError("a paged cache needs at least one tensor, each with a name of its own")
        if self.window < 0:
            raise ValueError("window must not be negative")
        if self.page_size is not None and self.page_size <= 0:
            raise ValueError("page_size must be positive")


@dataclass(frozen=True)
class StateCacheSpec:
    """A fixed-size state per request: ``shape`` elements of ``dtype`` ("float32" or
    "model" for the engine's element type), zeroed when a request starts."""

    shape: tuple[int, ...]
    dtype: str = "float32"

    kind: ClassVar[str] = "state"


# --------------------------------------------------------------------------- the checkpoint's tensors at bind time


class TensorBag(dict):
    """The checkpoint's tensors while the parts take theirs. ``uses[name]`` counts the parts
    that named the tensor in their ``tensor_specs``; :func:`take` hands a tensor out and, when
    the last of them has come for it, drops it from the bag, so that a part which copies its
    tensors (a fused weight) does not keep the originals alive until the whole model is bound."""

    def __init__(self, tensors: dict, uses: dict[str, int]):
        super().__init__(tensors)
        self.uses = dict(uses)


def take(tensors: dict, name: str):
    """``tensors[name]``; out of the bag with it if nobody else is going to ask. With a plain
    dictionary this is ``tensors[name]`` and nothing more."""
    uses = getattr(tensors, "uses", None)
    if uses is None or name not in uses:
        return tensors[name]
    uses[name] -= 1
    return tensors.pop(name) if uses[name] <= 0 else tensors[name]


# --------------------------------------------------------------------------- part classes


@dataclass(frozen=True)
class StepArraySpec:
    """An int32 array that a part's kernels need of every step beside the common ones
    (tokens, positions, block tables, ...): work lists, tiles, anything that follows from
    the step's batch. ``build(host_batch)`` returns it (numpy int32, any shape);
    ``capacity(max_tokens, max_seqs)`` bounds its number of elements
    (``max_seqs`` as ``HostBatch.decode_shape`` rounds the number of single-token requests). The engine builds it
    on the host, uploads it in the step's one copy and hands it to the parts as
    ``ctx.arrays[name]`` (device) and ``ctx.host.arrays[name]`` (host). Parts that name the
    same array share it."""

    name: str
    capacity: Any = field(compare=False)
    build: Any = field(compare=False)


class Part:
    """Base of everything that owns tensors."""

    def tensor_specs(self) -> list[TensorSpec]:
        return []

    def linears(self) -> list:
        """The matrix products (:class:`~pyre_amd.parts.linear.Linear`) this part owns,
        for whoever wants to prepare them (the engine lets the BLAS library time its
        kernels for their shapes)."""
        return []

    def bind(self, tensors: dict[str, Any], runtime: Any) -> None:
        """Take the tensors named by ``tensor_specs`` out of ``tensors``."""


class Mixer(Part):
    def cache_spec(self) -> PagedCacheSpec | StateCacheSpec | None:
        return None

    def step_arrays(self) -> list[StepArraySpec]:
        """Arrays that this mixer's kernels want of every step beside the common ones."""
        return []

    def forward(self, ctx, h, cache):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, h):
        raise NotImplementedError


class Norm(Part):
    def forward(self, ctx, resid, delta, out, rows=None):
        raise NotImplementedError


class PositionEncoding(Part):
    def rotary(self, runtime):
        return None, None, 0


class Block(Part):
    """A layer: parts arranged around the residual stream. ``forward`` receives one cache view
    per description of ``cache_specs()``, in that order (or the views of the entry whose caches
    this call reads, ``LayerCall.cache_from``)."""

    def cache_specs(self) -> list:
        return []

    def step_arrays(self) -> list[StepArraySpec]:
        return []

    def forward(self, ctx, state, caches: list) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registry of parts

_PARTS: dict[tuple[str, str], type] = {}
ROLES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")


def register_part(role: str, kind: str, cls: type) -> None:
    if role not in ROLES:
        raise ValueError(f"unknown role {role!r}; roles are {ROLES}")
    _PARTS[(role, kind)] = cls


def make_part(role: str, spec: Any, **kw: Any):
    """Build the part that ``spec`` (a dataclass with a ``kind``) describes."""
    _load_builtin_parts()
    kind = getattr(spec, "kind", None)
    try:
        cls = _PARTS[(role, kind)]
    except KeyError:
        known = sorted(k for r, k in _PARTS if r == role)
        raise ValueError(f"no {role} of kind {kind!r} is registered; known: {known}") from None
    return cls(spec, **kw)


def _load_builtin_parts() -> None:
    import pyre_amd.parts.builtin  # noqa: F401


# --------------------------------------------------------------------------- descriptions


@dataclass(frozen=True)
class RMSNormSpec:
    hidden_size: int
    eps: float
    prefix: str                      #: tensor name is ``prefix + ".weight"``
    kind: ClassVar[str] = "rmsnorm"


@dataclass(frozen=True)
class RotarySpec:
    """Half-split rotary positions: element j pairs with j + rotary_dim/2."""

    head_dim: int
    theta: float
    max_positions: int
    rotary_dim: int | None = None    #: None: the whole head
    kind: ClassVar[str] = "rotary"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: ClassVar[str] = "none"


@dataclass(frozen=True)
class AttentionSpec:
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    position: Any                    #: a position-encoding description
    prefix: str                      #: e.g. "model.layers.0.self_attn"
    qkv_bias: bool = True
    out_bias: bool = False
    window: int = 0                  #: 0: every earlier key is visible
    scale: float | None = None       #: None: head_dim ** -0.5
    kind: ClassVar[str] = "attention"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden_size: int
    intermediate_size: int
    prefix: str                      #: e.g. "model.layers.0.mlp"
    kind: ClassVar[str] = "swiglu"


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(norm(x)); x += feed_forward(norm(x))   (pre-norm residual block)."""

    mixer: Any
    mixer_norm: Any
    feed_forward: Any
    feed_forward_norm: Any
    kind: ClassVar[str] = "pre_norm"


@dataclass(frozen=True)
class EmbeddingSpec:
    vocab_size: int
    hidden_size: int
    name: str = "model.embed_tokens.weight"
    kind: ClassVar[str] = "embedding"


@dataclass(frozen=True)
class LMHeadSpec:
    vocab_size: int
    hidden_size: int
    name: str = "lm_head.weight"
    tied_to: str | None = None       #: embedding tensor used when the head is tied
    kind: ClassVar[str] = "lm_head"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the order in which layers run.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named more than once).
    ``cache_from`` = j lets this call's mixer read the cache that the j-th entry
    of the order wrote, instead of keeping one of its own.
    """

    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: Any
    layers: tuple[Any, ...]
    schedule: tuple[LayerCall, ...]
    final_norm: Any
    head: Any
    extra: dict = field(default_factory=dict, compare=False)
