"""RMSNorm with the residual add fused in front of it.

``y = x * rsqrt(mean(x^2) + eps) * w`` over the last dimension, all in
float32, the weight multiplying after normalisation, no offset, no bias
(reference: qwen3_runtime/layers/ops.py:17-20). The fused form first adds the
pending sub-layer output into the residual stream
(reference: qwen3_runtime/layers/ops.py:28-37), here in float32.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Norm
from .plan import TensorDecl


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, tensors=None):
        super().__init__(tensors)
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def tensor_decls(self):
        return [TensorDecl(self._name("weight"), (self.size,), init="norm")]

    def load(self, fetch):
        self.weight = fetch.vector_f32(self._name("weight"))

    def forward(self, ctx, residual, delta=None, rows=None):
        """Add ``delta`` into ``residual`` (in place), return its normalised rows.

        With ``rows`` (int32 indices) only those rows are normalised and
        returned, packed; ``residual`` is then left as it is.
        """
        return ctx.ops.add_rmsnorm(residual, delta, self.weight, self.eps, ctx.dtype, rows)
