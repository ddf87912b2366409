"""Grouped-query attention over a paged cache, with optional per-head q/k norm.

Order of operations (reference: qwen3_runtime/models/qwen3.py:96-117):
one fused projection to q | k | v, reshape to heads, RMSNorm of every q head and
every k head over the head dimension with one weight per layer, position
encoding of q and k, keys (normed, rotated) and values (raw) written to the
cache before anything reads it, attention of every query over its sequence's
cache, output projection. Query head ``h`` reads key/value head ``h // g``,
``g = heads / kv_heads``; scores are ``q.k / sqrt(D)``, key ``j`` is visible
to the query at position ``i`` iff ``j <= i`` (and ``j > i - window`` when the
mixer has a window); softmax in float32
(reference: qwen3_runtime/attention/pytorch.py:12-47).
"""

from __future__ import annotations

import math

from ..registry import part_class, register_part
from .base import Mixer
from .plan import CacheSpec, PartSpec, TensorDecl


@register_part("mixer", "gqa_attention")
class GroupedQueryAttention(Mixer):
    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        qk_norm_eps: float | None = None,
        position: PartSpec | None = None,
        window: int | None = None,
        scale: float | None = None,
        tensors=None,
    ):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} key/value heads")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = None
        if position is not None:
            self.position = part_class("position", position.kind)(**position.args, tensors=position.tensors)
        self.qkv = self.o = self.q_norm = self.k_norm = None

    def children(self):
        return (self.position,) if self.position is not None else ()

    def cache_spec(self):
        return CacheSpec("paged_kv", heads=self.num_kv_heads, head_dim=self.head_dim, window=self.window)

    def tensor_decls(self):
        h, d = self.hidden_size, self.head_dim
        decls = [
            TensorDecl(self._name("q"), (self.num_heads * d, h)),
            TensorDecl(self._name("k"), (self.num_kv_heads * d, h)),
            TensorDecl(self._name("v"), (self.num_kv_heads * d, h)),
            TensorDecl(self._name("o"), (h, self.num_heads * d)),
        ]
        if self.qk_norm_eps is not None:
            decls += [
                TensorDecl(self._name("q_norm"), (d,), init="norm"),
                TensorDecl(self._name("k_norm"), (d,), init="norm"),
            ]
        return decls

    def load(self, fetch):
        self.qkv = fetch.fused([self._name("q"), self._name("k"), self._name("v")], dim=0)
        self.o = fetch.matrix(self._name("o"))
        if self.qk_norm_eps is not None:
            self.q_norm = fetch.vector_f32(self._name("q_norm"))
            self.k_norm = fetch.vector_f32(self._name("k_norm"))

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)  # the four projections
        for q, kv in spans:  # scores and weighted values: 4 D operations per (query head, visible key)
            first = kv - q
            pairs = sum(min(first + i + 1, self.window or kv) for i in range(q)) if self.window else \
                q * first + q * (q + 1) // 2
            cost.flop += 4.0 * self.num_heads * self.head_dim * pairs
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        qkv = ops.linear(x, self.qkv)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        fused = self.position is None or self.position.fused_form == "neox_full"
        inv_freq = None if self.position is None or not fused else self.position.inv_freq
        if fused and ops.fuses_decode_attention(ctx, qkv, nq, nkv, d, cache):
            # a step of single tokens: all of it inside the attention kernel
            attn = ops.decode_attention(qkv, cache, ctx, nq, nkv, d, self.scale, self.window,
                                        self.q_norm, self.k_norm, eps, inv_freq,
                                        None if self.position is None else self.position.angles_key)
            return ops.linear_for_residual(attn, self.o)
        if fused:
            # norm, rotation and the cache write in one pass over qkv
            q = ops.qk_norm_rope_store(
                qkv, nq, nkv, d, self.q_norm, self.k_norm, eps, inv_freq, ctx.positions,
                cache if cache.writes else None, ctx=ctx,
                angles_key=None if self.position is None else self.position.angles_key,
            )
        else:
            # an encoding the fused kernel has no form for: norm, let it rotate, then store
            q, k, v = ops.qk_norm_split(qkv, nq, nkv, d, self.q_norm, self.k_norm, eps)
            q, k = self.position.rotate(ctx, q, k)
            if cache.writes:
                ops.kv_store(k, v, cache)
            q = q.reshape(ctx.num_tokens, nq * d)
        attn = ops.paged_attention(q, cache, ctx, nq, nkv, d, self.scale, self.window)
        return ops.linear_for_residual(attn, self.o)
