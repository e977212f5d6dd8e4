"""Architecture-neutral description of a decoder: what the parts and the cache are built from.

An architecture module (``clockwork_amd.models.*``) reads its own ``config.json``
keys into a typed configuration and turns that into a :class:`ModelSpec`. Nothing
below this line knows a model's name: parts see only their own spec, the cache
manager sees only :class:`KVPagesSpec` / :class:`StateSpec`, and the order in which
layers run is the ``run`` list.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional, Sequence


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part owns.

    ``precision``:
      * ``"compute"`` - cast to the engine's dtype (bfloat16 or float32);
      * ``"stored"``  - like ``"compute"``, but a tensor the checkpoint holds in
        float32 stays float32 (small vectors: norm weights, biases);
      * ``"float32"`` / ``"int32"`` - always that type.
    ``init`` names the random-weights distribution: ``("normal", std)``,
    ``("one_plus_uniform", half_width)`` or ``("zeros",)``.
    """

    shape: tuple[int, ...]
    precision: str = "compute"
    init: tuple = ("normal", 0.02)


@dataclass(frozen=True)
class KVPagesSpec:
    """A mixer that keeps keys and values of earlier tokens in pages.

    ``window`` None: every earlier token is read, pages live as long as the
    request. ``window`` W: a token reads itself and the W-1 tokens before it;
    pages wholly behind the window are given back while the request runs.
    Mixers whose (kv_heads, head_dim, window) agree share a layer group and
    therefore a block table.
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def group_key(self) -> tuple:
        return ("kv", self.num_kv_heads, self.head_dim, self.window)

    @property
    def planes(self) -> tuple:
        """What a page holds per token, as (name, row shape) pairs: a key row and a value row."""
        row = (self.num_kv_heads, self.head_dim)
        return (("k", row), ("v", row))


@dataclass(frozen=True)
class PagedRowsSpec:
    """A mixer that keeps rows of its own making for earlier tokens in pages: ``planes`` names
    each kind of row and gives its shape, e.g. ``(("latent", (24,)),)`` for one 24-wide vector a
    token and no values, or keys and values of different widths. Pages, block tables, windows
    and sharing work as for :class:`KVPagesSpec` (which is the case of two equal planes named
    ``k`` and ``v``); the mixer finds its planes in ``EntryCache.planes`` by name, each a flat
    [num_blocks * block_size, *row shape] view, and addresses them through the step's block
    tables and slots of its group.
    """

    planes: tuple
    window: Optional[int] = None

    def __post_init__(self):
        names = [name for name, _ in self.planes]
        if not self.planes or len(set(names)) != len(names):
            raise ValueError(f"a paged cache needs planes with names of their own, got {self.planes!r}")
        for name, shape in self.planes:
            if not shape or any(int(d) < 1 for d in shape):
                raise ValueError(f"plane {name!r} has no valid row shape: {shape!r}")

    def group_key(self) -> tuple:
        return ("rows", tuple((name, tuple(shape)) for name, shape in self.planes), self.window)


@dataclass(frozen=True)
class StateSpec:
    """A mixer that keeps a fixed-size state per request (a recurrence, a convolution tail).

    One slot of ``shape``/``dtype`` per live request and per run entry; when a request's first
    token arrives its slot is set to the fresh state: ``init`` says which, ``("zeros",)`` or
    ``("fill", value)`` (a part with another beginning, learned say, writes it into the pool's
    template row at ``bind`` time: ``CachePools.set_fresh_state``).
    """

    shape: tuple[int, ...]
    dtype: str = "float32"
    init: tuple = ("zeros",)

    def __post_init__(self):
        if self.init[0] not in ("zeros", "fill") or (self.init[0] == "fill" and len(self.init) != 2):
            raise ValueError(f"a fresh state is ('zeros',) or ('fill', value), got {self.init!r}")

    def group_key(self) -> tuple:
        return ("state", self.shape, self.dtype, self.init)


@dataclass(frozen=True)
class LayerSpec:
    """One block: which parts it is made of and how they are wired.

    ``arrangement`` names an entry of the arrangement registry ("prenorm":
    x + mixer(norm(x)), then x + ffn(norm(x))). The parts are specs of registered
    part kinds under the names the arrangement expects: the four that most blocks
    have can be given by keyword (any of them may be left out), others in
    ``extra`` as (name, spec) pairs; the arrangement's factory receives them all
    as keyword arguments. Different layers of one model may hold different kinds.
    The part named ``mixer`` is the one that owns the block's cache.
    """

    arrangement: str
    mixer: Any = None
    feed_forward: Any = None
    mixer_norm: Any = None
    ffn_norm: Any = None
    extra: tuple = ()

    def named_parts(self) -> dict:
        """{name: spec} of every part of the block, in a fixed order."""
        parts = {}
        for name in ("mixer", "feed_forward", "mixer_norm", "ffn_norm"):
            if getattr(self, name) is not None:
                parts[name] = getattr(self, name)
        for name, spec in self.extra:
            if name in parts:
                raise ValueError(f"a block has two parts named {name!r}")
            parts[name] = spec
        return parts


@dataclass(frozen=True)
class RunEntry:
    """One step of the forward pass: run ``layer`` (an index into ``ModelSpec.layers``).

    A layer may appear in several entries (its weights are then shared; each
    entry still has a cache of its own). ``cache_from`` names an *earlier entry*
    whose cache this entry reads instead of writing its own.
    """

    layer: int
    cache_from: Optional[int] = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Sequence[LayerSpec]
    run: Sequence[RunEntry]
    final_norm: Any
    tie_embeddings: bool = False
    eos_token_ids: tuple[int, ...] = ()
    # specs of the part that turns token ids into the residual stream and of the part that turns
    # the final norm's rows into logits; None: a plain table lookup and a plain product with a
    # [vocab, hidden] matrix (the embedding table itself when ``tie_embeddings`` is set)
    embedding: Any = None
    head: Any = None
    # free-form facts for reporting (bench config lines and the like), never read by parts
    info: dict = field(default_factory=dict)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        if not self.run:
            raise ValueError("the run list is empty")
        for i, entry in enumerate(self.run):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"run[{i}] names layer {entry.layer}, model has {len(self.layers)}")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < i:
                    raise ValueError(f"run[{i}].cache_from={entry.cache_from} must name an earlier entry")
                if self.run[entry.cache_from].cache_from is not None:
                    raise ValueError(f"run[{i}].cache_from names an entry that itself borrows a cache")


@dataclass(frozen=True)
class WeightTarget:
    """How one parameter of the model is filled from checkpoint tensors.

    ``sources`` are tensor names in the checkpoint with their expected shapes (as the file holds
    them); several sources are concatenated along dim 0 (fused projections).
    ``optional`` sources may be absent (a tied output head). ``transform`` reshapes every source
    after it is read and before it is put in its place: one step or a tuple of steps, each a tuple
    of a name from ``clockwork_amd.weights.transforms`` and its arguments, e.g. ``("transpose",)``
    for a matrix the checkpoint stores the other way round, ``("split_rows", 1, 3)`` for the second
    third of a tensor that holds three projections, or both in a row.
    """

    param: str
    sources: tuple[str, ...]
    source_shapes: tuple[tuple[int, ...], ...]
    optional: bool = False
    transform: Optional[tuple] = None
