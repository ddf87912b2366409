"""Plain torch version of every device op, one function per kernel.

Two uses: the GPU tests compare each HIP kernel alone with its function here,
and ``TorchOps`` lets the host-side tests drive the engine (cache manager,
step function, scheduler) on the CPU, where no kernel can run. The engine
itself never imports this file: its only ops are the HIP ones.

Arithmetic inside each op is float32 (or ``compute``), results are cast to the
output type, as the kernels do. The cache layout is the engine's: keys
``[page, head, offset, D]``, values ``[page, head, D, offset]``.
"""

from __future__ import annotations

import math

import torch


def embed(ids, table):
    return table[ids.long()].to(torch.float32)


def add_rmsnorm(residual, delta, weight, eps, out_dtype, rows=None, compute=torch.float32):
    if delta is not None and delta.dim() == 3:
        delta = delta.to(residual.dtype).sum(0)
    if delta is not None:
        if rows is None:
            residual += delta.to(residual.dtype)
            x = residual
        else:
            x = residual[rows.long()] + delta[rows.long()].to(residual.dtype)
    else:
        x = residual if rows is None else residual[rows.long()]
    x = x.to(compute)
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return (x * torch.rsqrt(var + eps) * weight.to(compute)).to(out_dtype)


def linear(x, w, out_f32=False, compute=torch.float32):
    y = x.to(compute) @ w.to(compute).T
    return y.to(torch.float32 if out_f32 else x.dtype)


def head_rmsnorm(x, weight, eps, compute=torch.float32):
    x = x.to(compute)
    if weight is None:
        return x
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.to(compute)


def rope_rotate(x, positions, inv_freq, compute=torch.float32):
    """x [T, heads, D] (compute dtype); angles = float32(pos) * inv_freq in float32."""
    d = x.shape[-1]
    ang = (positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]).to(compute)
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def qk_norm_split(qkv, nq, nkv, d, q_w, k_w, eps, compute=torch.float32):
    t = qkv.shape[0]
    q = qkv[:, : nq * d].reshape(t, nq, d)
    k = qkv[:, nq * d: (nq + nkv) * d].reshape(t, nkv, d)
    v = qkv[:, (nq + nkv) * d:].reshape(t, nkv, d)
    q = head_rmsnorm(q, q_w, eps, compute).to(qkv.dtype)
    k = head_rmsnorm(k, k_w, eps, compute).to(qkv.dtype)
    return q, k, v.contiguous()


def kv_store(k, v, k_cache, v_cache, slots, page_size):
    """k, v: [T, heads, D]; slot = page * page_size + offset."""
    pages = (slots // page_size).long()
    offs = (slots % page_size).long()
    k_cache[pages, :, offs, :] = k.to(k_cache.dtype)
    v_cache[pages, :, :, offs] = v.to(v_cache.dtype)


def qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                       k_cache=None, v_cache=None, slots=None, page_size=None, compute=torch.float32):
    t = qkv.shape[0]
    q = qkv[:, : nq * d].reshape(t, nq, d)
    k = qkv[:, nq * d: (nq + nkv) * d].reshape(t, nkv, d)
    v = qkv[:, (nq + nkv) * d:].reshape(t, nkv, d)
    q = head_rmsnorm(q, q_w, eps, compute)
    k = head_rmsnorm(k, k_w, eps, compute)
    if inv_freq is not None:
        q = rope_rotate(q, positions, inv_freq, compute)
        k = rope_rotate(k, positions, inv_freq, compute)
    if k_cache is not None:
        kv_store(k, v, k_cache, v_cache, slots, page_size)
    return q.to(qkv.dtype).reshape(t, nq * d)


def gather_kv(k_cache, v_cache, table_row, lo, hi, page_size):
    """Keys and values of positions lo..hi-1 of one sequence: [hi-lo, heads, D] each."""
    pos = torch.arange(lo, hi, device=k_cache.device)
    pages = table_row.long()[pos // page_size]
    offs = pos % page_size
    if (pages < 0).any():
        raise AssertionError("attention reads a position whose page was given back")
    k = k_cache[pages, :, offs, :]
    v = v_cache[pages, :, :, offs]
    return k, v


def paged_attention(q, k_cache, v_cache, cu_q, kv_lens, block_table, page_size, nq, nkv, d,
                    scale, window=None, compute=torch.float32, round_probs=False):
    """q [T, nq*D] -> [T, nq*D]. Query row i of a sequence sits at position
    kv_len - q_len + i and sees keys j <= its position (and > position - window)."""
    out = torch.zeros_like(q)
    g = nq // nkv
    cu = [int(x) for x in cu_q]
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        q_len, kv_len = b - a, int(kv_lens[s])
        if q_len == 0 or kv_len == 0:
            continue
        first_pos = kv_len - q_len
        lo = 0 if window is None else max(0, first_pos - window + 1)
        k, v = gather_kv(k_cache, v_cache, block_table[s], lo, kv_len, page_size)
        k = k.to(compute).repeat_interleave(g, dim=1)
        v = v.to(compute).repeat_interleave(g, dim=1)
        qs = q[a:b].reshape(q_len, nq, d).to(compute)
        scores = torch.einsum("qhd,khd->hqk", qs, k) * scale
        qpos = torch.arange(first_pos, kv_len, device=q.device)[:, None]
        kpos = torch.arange(lo, kv_len, device=q.device)[None, :]
        ok = kpos <= qpos
        if window is not None:
            ok = ok & (kpos > qpos - window)
        scores = scores.masked_fill(~ok, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        if round_probs:
            probs = probs.to(q.dtype).to(compute)
        ctx = torch.einsum("hqk,khd->qhd", probs, v)
        out[a:b] = ctx.reshape(q_len, nq * d).to(q.dtype)
    return out


def swiglu(gate_up, compute=torch.float32):
    i = gate_up.shape[-1] // 2
    g, u = gate_up[..., :i].to(compute), gate_up[..., i:].to(compute)
    return (g * torch.sigmoid(g) * u).to(gate_up.dtype)


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)


class TorchOps:
    """The engine's op interface over the functions above (tests only)."""

    def __init__(self, compute=torch.float32):
        self.compute = compute

    def embed(self, ids, table):
        return embed(ids, table)

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None):
        return add_rmsnorm(residual, delta, weight, eps, out_dtype, rows, self.compute)

    def linear(self, x, w, out_f32=False):
        return linear(x, w, out_f32, self.compute)

    def linear_for_residual(self, x, w):
        return linear(x, w, False, self.compute)

    def qk_norm_rope_store(self, qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions, cache, ctx=None,
                           angles_key=None):
        if cache is None:
            return qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                                      compute=self.compute)
        return qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                                  cache.k, cache.v, cache.group.slots, cache.group.page_size, self.compute)

    def fuses_decode_attention(self, ctx, qkv, nq, nkv, d, cache):
        return False  # no one-kernel form of a decode step's attention here: the steps above, in order

    def qk_norm_split(self, qkv, nq, nkv, d, q_w, k_w, eps):
        return qk_norm_split(qkv, nq, nkv, d, q_w, k_w, eps, self.compute)

    def rope_neox(self, q, k, positions, inv_freq):
        return (rope_rotate(q.to(self.compute), positions, inv_freq, self.compute).to(q.dtype),
                rope_rotate(k.to(self.compute), positions, inv_freq, self.compute).to(k.dtype))

    def kv_store(self, k, v, cache):
        kv_store(k, v, cache.k, cache.v, cache.group.slots, cache.group.page_size)

    def paged_attention(self, q, cache, ctx, nq, nkv, d, scale, window):
        return paged_attention(q, cache.k, cache.v, ctx.cu_q, ctx.kv_lens, cache.group.block_table,
                               cache.group.page_size, nq, nkv, d, scale, window, self.compute)

    def swiglu(self, gate_up):
        return swiglu(gate_up, self.compute)

    def gated_linear(self, x, w_gate_up):
        return swiglu(linear(x, w_gate_up, False, self.compute), self.compute)

    def argmax(self, logits):
        return argmax(logits)
