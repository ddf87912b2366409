"""Rotary position encoding, NeoX pairing.

``inv_j = theta^(-2j/D)``, angle ``pos * inv_j``; the head vector is split
into its first and second half ``x1 | x2`` and rotated pairwise:
``y1 = x1 cos - x2 sin``, ``y2 = x2 cos + x1 sin``
(reference: qwen3_runtime/layers/rope.py:7-21). Angles, sine and cosine are
float32. The same angles serve every head; values are not rotated.
"""

from __future__ import annotations

import torch

from ..registry import register_part
from .base import PositionEncoding


@register_part("position", "rope_neox")
class RotaryNeox(PositionEncoding):
    fused_form = "neox_full"

    def __init__(self, head_dim: int, theta: float, tensors=None):
        super().__init__(tensors)
        if head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        # float32 throughout, as the table of the reference is built
        # (reference: qwen3_runtime/layers/rope.py:18)
        self.inv_freq_cpu = 1.0 / (
            self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim)
        )
        self.inv_freq = None
        # layers whose encodings have equal keys rotate by equal angles and share a step's table
        self.angles_key = ("rope_neox", self.head_dim, self.theta)

    def load(self, fetch):
        self.inv_freq = fetch.constant(self.inv_freq_cpu)

    def rotate(self, ctx, q, k):
        """Unfused form: rotate already-normed q ``[T, nq, D]`` and k ``[T, nkv, D]``."""
        return ctx.ops.rope_neox(q, k, ctx.positions, self.inv_freq)
