"""Interfaces every part implements, and the per-step context they receive.

A part is built from numbers (``PartSpec.args``), says which tensors it reads
(``tensor_decls``), takes them from a ``WeightFetcher`` (``load``) and then runs
on packed tokens. A part knows neither the model it is in nor the
configuration the numbers came from.

Roles and the call each must answer (``T`` tokens of this step, ``H`` width):

* embedding      ``forward(ctx, ids[T] int32) -> residual[T, H] float32``
* norm           ``forward(ctx, residual[T, H] float32, delta[T, H] | None, rows=None) -> [T|R, H]``
                 adds ``delta`` into ``residual`` in place, then normalises
* mixer          ``forward(ctx, x[T, H], cache: CacheView | None) -> [T, H]``
* feed_forward   ``forward(ctx, x[T, H]) -> [T, H]``
* position       ``rotate(ctx, q[T, nq, D], k[T, nkv, D]) -> (q, k)``
* block          ``forward(ctx, residual, delta, cache) -> (residual, delta)``
* head           ``forward(ctx, x[R, H]) -> logits[R, V] float32``

The residual stream is float32 in every mode; ``delta`` is the output of the
previous sub-layer that has not been added yet, so that the add fuses with the
next norm. A sub-layer may hand its output over in planes ``[P, T, H]`` whose
sum it is (``ops.linear_for_residual``); only a norm ever looks into ``delta``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Protocol, Sequence

import torch

from .plan import CacheSpec, TensorDecl


class WeightFetcher(Protocol):
    """What ``load`` may ask for; implemented by ``weights.loader.WeightLoader``."""

    def matrix(self, file_name: str) -> torch.Tensor: ...

    def fused(self, file_names: Sequence[str], dim: int = 0) -> torch.Tensor: ...

    def vector_f32(self, file_name: str) -> torch.Tensor: ...

    def table_i32(self, file_name: str) -> torch.Tensor: ...

    def constant(self, tensor: torch.Tensor) -> torch.Tensor: ...


@dataclass
class StepCost:
    """What a step asks of the device, for rooflines: bytes of each tensor it reads (by file
    name: a tensor two parts share, or a layer that runs twice, is read once) and
    floating-point operations."""

    weight_bytes: dict[str, int] = field(default_factory=dict)
    flop: float = 0.0

    def add(self, other: "StepCost") -> None:
        for name, n in other.weight_bytes.items():
            self.weight_bytes[name] = max(self.weight_bytes.get(name, 0), n)
        self.flop += other.flop

    @property
    def total_weight_bytes(self) -> int:
        return sum(self.weight_bytes.values())


class Part:
    """Base of all parts: holds the tensor-name map, declares and loads tensors."""

    role = ""
    # What the step function and the scheduler must know of a part, declared by its class:
    # ``graph_capturable``: False for a part whose ``forward`` reads device memory on the host,
    # or does anything else a captured HIP graph cannot replay; steps of a model with such a
    # part run eagerly. ``portion_multiple``: a part that works on blocks of this many tokens
    # wants every portion of a prompt but the last to be a multiple of it.
    graph_capturable = True
    portion_multiple = 1

    def __init__(self, tensors: Mapping[str, str] | None = None):
        self.tensor_names: dict[str, str] = dict(tensors or {})

    def tensor_decls(self) -> list[TensorDecl]:
        return []

    def load(self, fetch: WeightFetcher) -> None:
        return None

    def children(self) -> Sequence["Part"]:
        return ()

    def step_cost(self, spans: Sequence[tuple[int, int]], rows: int, elem_bytes: int) -> StepCost:
        """Bytes and operations of one run of this part (children not included) over a step whose
        sequences are ``spans`` = (tokens of the step, tokens in the cache after it), with logits
        wanted at ``rows`` places. The default fits a part whose tensors are all read whole and
        whose matrices each multiply every token once; a part for which that is wrong (a table
        that is only looked up, experts of which few run, attention's own products) says so."""
        tokens = sum(q for q, _ in spans)
        cost = StepCost()
        for decl in self.tensor_decls():
            n = 1
            for dim in decl.shape:
                n *= dim
            cost.weight_bytes[decl.file_name] = n * elem_bytes
            if decl.init == "matrix" and len(decl.shape) == 2:
                cost.flop += 2.0 * tokens * n
        return cost

    def _name(self, logical: str) -> str:
        try:
            return self.tensor_names[logical]
        except KeyError:
            raise KeyError(
                f"{type(self).__name__} needs a file name for its tensor {logical!r}; "
                f"the plan gave {sorted(self.tensor_names)}"
            ) from None


class Mixer(Part):
    role = "mixer"

    def cache_spec(self) -> CacheSpec | None:
        return None


class FeedForward(Part):
    role = "feed_forward"


class Norm(Part):
    role = "norm"


class PositionEncoding(Part):
    role = "position"
    # An encoding that the fused q/k kernel can apply itself says which of the kernel's forms
    # it is; the attention mixer then never calls ``rotate``. The one form there is:
    # ``"neox_full"``, the rotation of all ``head_dim`` elements, first half against second
    # half, by the angles ``position * self.inv_freq[j]`` (float32 [head_dim / 2] on the device).
    # None (the default) means the mixer norms, calls ``rotate`` and stores, as three steps.
    fused_form: str | None = None
    # Encodings with equal keys rotate by equal angles: the layers of a step then share one table
    # of its tokens' cosines and sines. None: the encoding's own ``inv_freq`` tensor is the key.
    angles_key: Any = None


class Block(Part):
    role = "block"


@dataclass
class GroupView:
    """One cache group's view of this step's batch (device tensors).

    ``block_table[s, i]`` is the physical page of sequence ``s`` that holds
    positions ``[i*page_size, (i+1)*page_size)``, or -1 where the page has been
    given back or not been taken yet. ``slots[t]`` is
    ``page * page_size + offset`` for packed token ``t``.
    """

    page_size: int
    window: int | None
    block_table: torch.Tensor
    slots: torch.Tensor


@dataclass
class CacheView:
    """What one ``RunStep`` sees of its cache."""

    spec: CacheSpec
    writes: bool = True
    group: GroupView | None = None
    # paged_kv: keys [pages, heads, page_size, D]; values [pages, heads, Dv, page_size]
    k: torch.Tensor | None = None
    v: torch.Tensor | None = None
    # state: [slots, *shape]
    state: torch.Tensor | None = None
    # any paged cache: stream name -> [pages, *PagedStream.page_shape(page_size)]; for
    # "paged_kv" the entries "k" and "v" are the tensors above
    pages: dict[str, torch.Tensor] = field(default_factory=dict)


@dataclass
class StepContext:
    """Everything about one step's batch that parts may read.

    Sequences are packed: tokens of sequence ``s`` are rows
    ``cu_q[s] : cu_q[s+1]``, at positions ``kv_lens[s] - q_len .. kv_lens[s] - 1``.
    The ``*_host`` fields hold the same numbers as Python lists so that launch
    shapes need no device read.
    """

    ops: Any
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_seqs: int
    positions: torch.Tensor          # int32 [T]
    cu_q: torch.Tensor               # int32 [S+1]
    kv_lens: torch.Tensor            # int32 [S]   lengths after this step
    seq_of_token: torch.Tensor       # int32 [T]
    state_slots: torch.Tensor        # int32 [S]   slot of each sequence's fixed-size state
    first_span: torch.Tensor         # int32 [S]   1 where the span starts at position 0
    q_lens_host: list[int] = field(default_factory=list)
    kv_lens_host: list[int] = field(default_factory=list)
    max_q_len: int = 0
    max_kv_len: int = 0
    groups: list[GroupView] = field(default_factory=list)
    scratch: dict[str, Any] = field(default_factory=dict)
    # values computed from the step's own data (positions, lengths) that several layers share: the
    # model empties this at the start of every pass, also of one that reuses the context (a
    # captured graph keeps its context, and what is computed here must be part of the capture)
    per_pass: dict[Any, Any] = field(default_factory=dict)
