"""A decoder built from a ``ModelPlan``: embedding, ordered blocks, norm, head.

``forward`` runs the packed tokens of one step through ``plan.order`` and
returns float32 logits at the requested rows (reference, for the equivalent
fixed loop: qwen3_runtime/models/qwen3.py:222-266).
"""

from __future__ import annotations

import math
from typing import Sequence

from ..registry import part_class
from .base import CacheView, Part, StepContext, StepCost
from .plan import ModelPlan, PartSpec, TensorDecl


def build_part(role: str, spec: PartSpec) -> Part:
    return part_class(role, spec.kind)(**spec.args, tensors=spec.tensors)


def walk(part: Part):
    yield part
    for child in part.children():
        if child is not None:
            yield from walk(child)


class DecoderModel:
    def __init__(self, plan: ModelPlan):
        self.plan = plan
        self.embedding = build_part("embedding", plan.embedding)
        self.blocks = []
        for layer in plan.layers:
            mixer = build_part("mixer", layer.mixer)
            ff = build_part("feed_forward", layer.feed_forward)
            norms = {name: build_part("norm", spec) for name, spec in layer.norms.items()}
            block_cls = part_class("block", layer.block.kind)
            self.blocks.append(
                block_cls(mixer, ff, norms, **layer.block.args, tensors=layer.block.tensors)
            )
        self.final_norm = build_part("norm", plan.final_norm)
        self.head = build_part("head", plan.head)
        self._check_caches()

    def _check_caches(self) -> None:
        for i, step in enumerate(self.plan.order):
            spec = self.blocks[step.layer].mixer.cache_spec()
            if spec is None:
                if step.cache is not None:
                    raise ValueError(f"order[{i}]: layer {step.layer}'s mixer keeps no cache")
                continue
            if step.cache is None:
                raise ValueError(f"order[{i}]: layer {step.layer}'s mixer needs a cache")
            have = self.plan.caches[step.cache]
            if have.group_key() != spec.group_key():
                raise ValueError(
                    f"order[{i}]: layer {step.layer} needs cache {spec}, the plan gives {have}"
                )

    def parts(self):
        yield from walk(self.embedding)
        for block in self.blocks:
            yield from walk(block)
        yield from walk(self.final_norm)
        yield from walk(self.head)

    @property
    def graph_capturable(self) -> bool:
        """Whether a step of this model may be captured into a HIP graph: every part says so."""
        return all(part.graph_capturable for part in self.parts())

    @property
    def portion_multiple(self) -> int:
        """Least common multiple of what the parts ask of a prompt's portions."""
        return math.lcm(*(max(1, int(part.portion_multiple)) for part in self.parts()))

    def step_cost(self, spans, rows: int, elem_bytes: int) -> StepCost:
        """Bytes of weights and floating-point operations of one step (``Part.step_cost``), summed
        over the parts in the order they run: a layer named twice computes twice and is read once."""
        cost = StepCost()
        runs = [self.embedding] + [self.blocks[step.layer] for step in self.plan.order] + [self.final_norm, self.head]
        for top in runs:
            for part in walk(top):
                cost.add(part.step_cost(spans, rows, elem_bytes))
        return cost

    def tensor_decls(self) -> list[TensorDecl]:
        """Every tensor the model reads, once per file name."""
        seen: dict[str, TensorDecl] = {}
        for part in self.parts():
            for decl in part.tensor_decls():
                prior = seen.get(decl.file_name)
                if prior is not None and prior.shape != decl.shape:
                    raise ValueError(
                        f"tensor {decl.file_name} is declared with shapes {prior.shape} and {decl.shape}"
                    )
                seen.setdefault(decl.file_name, decl)
        return list(seen.values())

    def load(self, fetch) -> None:
        for part in self.parts():
            part.load(fetch)

    def forward(self, ctx: StepContext, ids, caches: Sequence[CacheView | None], rows=None):
        """``ids`` int32 [T]; ``caches[i]`` is the view for ``plan.order[i]``.

        Returns logits ``[R, V]`` float32 for the packed row indices ``rows``
        (int32 tensor), or None when ``rows`` is None: the pass then only fills
        the caches.
        """
        ctx.per_pass.clear()
        residual = self.embedding.forward(ctx, ids)
        delta = None
        for step, cache in zip(self.plan.order, caches):
            residual, delta = self.blocks[step.layer].forward(ctx, residual, delta, cache)
        if rows is None:
            return None
        x = self.final_norm.forward(ctx, residual, delta, rows)
        return self.head.forward(ctx, x)
