"""A model as data: which parts make each layer, and the order layers run in.

An architecture (see ``registry.py``) turns its typed configuration into a
``ModelPlan``. The plan names, layer by layer, a mixer, a feed-forward, the
norms and the block arrangement, each as a ``PartSpec`` (a registered kind, its
sizes and constants, and the names of its tensors in the model file). The plan
also lists the caches the layers own and ``order``: the sequence of
``RunStep``s one forward pass executes. A layer may appear in ``order`` more
than once, and a step may read the cache another step writes.

Parts never see the plan or the configuration; they see only their own
``PartSpec.args``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Sequence


@dataclass(frozen=True)
class PartSpec:
    """One part to build: ``kind`` picks the class from the registry of its role."""

    kind: str
    args: Mapping[str, Any] = field(default_factory=dict)
    # logical tensor name of the part -> tensor name in the model file
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class TensorDecl:
    """One tensor a part reads from the model file.

    ``init`` tells the random-weights mode how to draw it: ``"matrix"`` and
    ``"embedding"`` are zero-mean normal, ``"norm"`` is a scale around one.
    ``storage`` is ``"float"`` (stored as bfloat16, float32 or float16) or ``"int"``
    (an integer table, held as int32; drawn as zeros in the random-weights mode unless
    ``init`` is ``"index:<n>"``, uniform in ``[0, n)``).
    """

    file_name: str
    shape: tuple[int, ...]
    init: str = "matrix"
    storage: str = "float"


@dataclass(frozen=True)
class PagedStream:
    """One tensor a paged cache keeps for every token: ``heads`` x ``width`` elements.

    Within a page the tensor is ``[head, offset, width]``, or, ``transposed``,
    ``[head, width, offset]`` (the tokens of a page contiguous for one element: what a kernel
    wants that multiplies probabilities over keys with values)."""

    name: str
    heads: int
    width: int
    transposed: bool = False

    def page_shape(self, page_size: int) -> tuple[int, int, int]:
        return (self.heads, self.width, page_size) if self.transposed else (self.heads, page_size, self.width)

    def elements_per_token(self) -> int:
        return self.heads * self.width


@dataclass(frozen=True)
class CacheSpec:
    """What one cache owner keeps between steps.

    ``kind == "paged_kv"``: keys and values for every token (or the last
    ``window`` tokens), ``heads`` x ``head_dim`` keys and ``heads`` x ``value_dim``
    values (``head_dim`` when None), held in pages; the values transposed within a
    page. ``kind == "paged"``: any other set of per-token tensors, named by
    ``streams`` (one latent vector per token, say), with the same pages, tables and
    window. ``kind == "state"``: a fixed-size tensor of ``shape`` per request, held
    in a slot; ``dtype`` is a torch dtype name or ``"model"`` for the model's dtype.
    """

    kind: str
    heads: int = 0
    head_dim: int = 0
    window: int | None = None
    shape: tuple[int, ...] = ()
    dtype: str = "model"
    value_dim: int | None = None
    streams: tuple[PagedStream, ...] = ()

    @property
    def paged(self) -> bool:
        return self.kind in ("paged_kv", "paged")

    def page_streams(self) -> tuple[PagedStream, ...]:
        """The per-token tensors of a paged cache; a ``CacheView`` holds one device tensor for each,
        under the stream's name."""
        if self.kind == "paged_kv":
            return (PagedStream("k", self.heads, self.head_dim),
                    PagedStream("v", self.heads, self.head_dim if self.value_dim is None else self.value_dim, True))
        if self.kind == "paged":
            if not self.streams:
                raise ValueError("a cache of kind 'paged' names its streams")
            return tuple(self.streams)
        return ()

    def elements_per_token(self) -> int:
        return sum(s.elements_per_token() for s in self.page_streams())

    def group_key(self) -> tuple:
        """Caches with equal keys share pages' geometry and lifetime, hence a pool."""
        if self.paged:
            return ("paged", self.page_streams(), self.window)
        return ("state", tuple(self.shape), self.dtype)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement over a mixer, a feed-forward and norms."""

    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]


@dataclass(frozen=True)
class RunStep:
    """One entry of the execution order.

    ``layer`` indexes ``ModelPlan.layers``. ``cache`` indexes ``ModelPlan.caches``
    (or is None for a mixer without cache). ``writes_cache`` is False when the
    step only reads a cache that an earlier step of the same pass wrote.
    """

    layer: int
    cache: int | None = None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelPlan:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: Sequence[LayerSpec]
    caches: Sequence[CacheSpec]
    order: Sequence[RunStep]
    final_norm: PartSpec
    head: PartSpec
    # tensors a model file may hold although the plan reads them from elsewhere
    ignorable: Sequence[str] = ()
    eos_token_id: int | None = None

    def __post_init__(self) -> None:
        writers: set[int] = set()
        for i, step in enumerate(self.order):
            if not 0 <= step.layer < len(self.layers):
                raise ValueError(f"order[{i}] names layer {step.layer}; the plan has {len(self.layers)}")
            if step.cache is None:
                continue
            if not 0 <= step.cache < len(self.caches):
                raise ValueError(f"order[{i}] names cache {step.cache}; the plan has {len(self.caches)}")
            if step.writes_cache:
                if step.cache in writers:
                    raise ValueError(f"cache {step.cache} is written by two steps of the order")
                writers.add(step.cache)
            elif step.cache not in writers:
                raise ValueError(f"order[{i}] reads cache {step.cache} before any step writes it")
