"""Arrangement of a layer's parts: the pre-norm residual block.

``x += mixer(norm_in(x)); x += feed_forward(norm_post(x))``: the form the
reference's oracle writes (tests/cpu/reference_qwen3.py:79-110) and its model
computes as a chain of fused add-norms (qwen3_runtime/models/qwen3.py:165-187).
Here the block receives the residual stream and the previous sub-layer's
output that is still to be added, and hands both on, so that each add fuses
with the norm that follows it without a block knowing its neighbour.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Block


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    norm_names = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms, tensors=None):
        super().__init__(tensors)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]

    def children(self):
        return (self.norm_in, self.mixer, self.norm_post, self.feed_forward)

    def forward(self, ctx, residual, delta, cache):
        x = self.norm_in.forward(ctx, residual, delta)
        mixed = self.mixer.forward(ctx, x, cache)
        x = self.norm_post.forward(ctx, residual, mixed)
        return residual, self.feed_forward.forward(ctx, x)
