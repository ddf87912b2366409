"""Token embedding and output head.

``h0[t] = E[ids[t]]`` without scaling (reference: qwen3_runtime/models/qwen3.py:243);
``logits = x W^T`` where ``W`` is the embedding table when the head is tied,
no bias and no scaling of logits (reference: qwen3_runtime/models/qwen3.py:265-266).
The embedding starts the float32 residual stream; logits come out in float32.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Part, StepCost
from .plan import TensorDecl


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    role = "embedding"

    def __init__(self, vocab_size: int, hidden_size: int, tensors=None):
        super().__init__(tensors)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight = None

    def tensor_decls(self):
        return [TensorDecl(self._name("weight"), (self.vocab_size, self.hidden_size), init="embedding")]

    def load(self, fetch):
        self.weight = fetch.matrix(self._name("weight"))

    def forward(self, ctx, ids):
        return ctx.ops.embed(ids, self.weight)

    def step_cost(self, spans, rows, elem_bytes):
        # a lookup: one row of the table per token, no arithmetic
        tokens = sum(q for q, _ in spans)
        return StepCost({self._name("weight"): min(tokens, self.vocab_size) * self.hidden_size * elem_bytes}, 0.0)


@register_part("head", "linear_head")
class LinearHead(Part):
    """Projection to the vocabulary. A tied head names the embedding's tensor."""

    role = "head"

    def __init__(self, vocab_size: int, hidden_size: int, tensors=None):
        super().__init__(tensors)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight = None

    def tensor_decls(self):
        return [TensorDecl(self._name("weight"), (self.vocab_size, self.hidden_size), init="embedding")]

    def load(self, fetch):
        self.weight = fetch.matrix(self._name("weight"))

    def forward(self, ctx, x):
        return ctx.ops.linear(x, self.weight, out_f32=True)

    def step_cost(self, spans, rows, elem_bytes):
        # the whole matrix, multiplied with the wanted rows only
        n = self.vocab_size * self.hidden_size
        return StepCost({self._name("weight"): n * elem_bytes}, 2.0 * rows * n)
