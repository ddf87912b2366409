"""Dense gated feed-forward (SwiGLU).

``down( silu(gate(x)) * up(x) )`` with gate and up as one fused matrix whose
rows are gate's followed by up's (reference: qwen3_runtime/models/qwen3.py:130-138,
qwen3_runtime/utils/loader.py:51-53); ``silu(g) = g * sigmoid(g)``
(reference: qwen3_runtime/layers/ops.py:23-25), evaluated in float32 here.
"""

from __future__ import annotations

from ..registry import register_part
from .base import FeedForward
from .plan import TensorDecl


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int, tensors=None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up = None
        self.down = None

    def tensor_decls(self):
        h, i = self.hidden_size, self.intermediate_size
        return [
            TensorDecl(self._name("gate"), (i, h)),
            TensorDecl(self._name("up"), (i, h)),
            TensorDecl(self._name("down"), (h, i)),
        ]

    def load(self, fetch):
        self.gate_up = fetch.fused([self._name("gate"), self._name("up")], dim=0)
        self.down = fetch.matrix(self._name("down"))

    def forward(self, ctx, x):
        act = ctx.ops.gated_linear(x, self.gate_up)
        return ctx.ops.linear_for_residual(act, self.down)
