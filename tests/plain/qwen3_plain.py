"""Plain, slow Qwen3 dense decoder: whole sequences, no cache, one function per part.

Written from the reference's formulas; every function cites the file and lines of
yuzheng310/qwen3-runtime where its formula stands. It shares no code with the engine: it parses
config.json and reads the safetensors file itself. Arithmetic runs in float64
unless ``dtype`` says otherwise, except rotation angles, which the reference
fixes to float32 (the table is built in float32).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def rms_norm(x, weight, eps):
    """qwen3_runtime/layers/ops.py:17-20: x * rsqrt(mean(x^2) + eps) * w, weight after normalising."""
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def rope_angles(positions, head_dim, theta):
    """qwen3_runtime/layers/rope.py:18-21: inv = 1/theta^(2j/D); freqs = pos x inv, in float32."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)).to(positions.device)
    return positions.to(torch.float32)[:, None] * inv[None, :]  # [T, D/2] float32


def rope_neox(x, positions, theta):
    """qwen3_runtime/layers/rope.py:7-11: halves (x1 | x2); y1 = x1 cos - x2 sin; y2 = x2 cos + x1 sin.

    x: [T, heads, D]; the same angles for all heads.
    """
    d = x.shape[-1]
    ang = rope_angles(positions, d, theta).to(x.dtype)
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def causal_attention(q, k, v, scale=None, window=None, q_offset=0):
    """qwen3_runtime/attention/pytorch.py:12-47 (and reference/dense_attention.py:26-46).

    q: [Tq, nq, D], k/v: [Tk, nkv, D]. Query head h reads kv head h // g
    (repeat_interleave). scores = (q k^T) * scale with scale = 1/sqrt(D) applied
    after the product; key j visible to query row i iff j <= q_offset + i
    (bottom-right aligned when q_offset = Tk - Tq); softmax over keys; ctx = P v.
    ``window`` (not in the reference) additionally hides keys j <= q_offset + i - window.
    Returns [Tq, nq * D].
    """
    tq, nq, d = q.shape
    tk, nkv, _ = k.shape
    g = nq // nkv
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    k = k.repeat_interleave(g, dim=1)
    v = v.repeat_interleave(g, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * scale
    qpos = torch.arange(tq, device=q.device)[:, None] + q_offset
    kpos = torch.arange(tk, device=q.device)[None, :]
    allowed = kpos <= qpos
    if window is not None:
        allowed = allowed & (kpos > qpos - window)
    scores = scores.masked_fill(~allowed, float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    ctx = torch.einsum("hqk,khd->qhd", probs, v)
    return ctx.reshape(tq, nq * d)


def swiglu(gate, up):
    """qwen3_runtime/layers/ops.py:23-25: silu(gate) * up, silu(x) = x * sigmoid(x)."""
    return gate * torch.sigmoid(gate) * up


def read_model(folder, dtype=torch.float64, device="cpu"):
    """config.json as a dict and every tensor of model.safetensors, upcast to ``dtype``. With a
    ``device`` the same torch routines run there (the tests of models too large for the host's
    patience do that); ``forward`` follows the weights' device."""
    from safetensors.torch import load_file

    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    tensors = {}
    for path in sorted(folder.glob("*.safetensors")):
        tensors.update(load_file(str(path)))
    return cfg, {k: v.to(device=device, dtype=dtype) for k, v in tensors.items()}


def attention_layer(x, w, prefix, cfg, positions):
    """qwen3_runtime/models/qwen3.py:96-117 with separate q/k/v matrices
    (tests/cpu/reference_qwen3.py:86-105): project, per-head q/k norm, rope, attend, o_proj."""
    t = x.shape[0]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    eps = cfg["rms_norm_eps"]
    q = (x @ w[f"{prefix}.q_proj.weight"].T).view(t, nq, d)
    k = (x @ w[f"{prefix}.k_proj.weight"].T).view(t, nkv, d)
    v = (x @ w[f"{prefix}.v_proj.weight"].T).view(t, nkv, d)
    q = rms_norm(q, w[f"{prefix}.q_norm.weight"], eps)
    k = rms_norm(k, w[f"{prefix}.k_norm.weight"], eps)
    q = rope_neox(q, positions, cfg["rope_theta"])
    k = rope_neox(k, positions, cfg["rope_theta"])
    ctx = causal_attention(q, k, v)
    return ctx @ w[f"{prefix}.o_proj.weight"].T


def feed_forward(x, w, prefix):
    """qwen3_runtime/models/qwen3.py:130-138: down(silu(gate x) * up x)."""
    act = swiglu(x @ w[f"{prefix}.gate_proj.weight"].T, x @ w[f"{prefix}.up_proj.weight"].T)
    return act @ w[f"{prefix}.down_proj.weight"].T


def forward(cfg, w, ids):
    """Logits [T, V] of one whole sequence from position 0.

    Pre-norm blocks h += attn(norm(h)); h += mlp(norm(h)); final norm; head tied
    to the embedding or not (tests/cpu/reference_qwen3.py:79-110,
    qwen3_runtime/models/qwen3.py:243-266).
    """
    dev = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(ids, dtype=torch.long, device=dev)
    positions = torch.arange(ids.numel(), device=dev)
    eps = cfg["rms_norm_eps"]
    h = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        n = rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
        h = h + attention_layer(n, w, f"{p}.self_attn", cfg, positions)
        n = rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
        h = h + feed_forward(n, w, f"{p}.mlp")
    h = rms_norm(h, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return h @ head.T


def greedy(logits):
    """qwen3_runtime/sampling.py:28-32: argmax, ties to the lowest id."""
    return int(torch.argmax(logits, dim=-1))


def greedy_generate(cfg, w, prompt, n):
    """Recompute from token 0 for every new token (qwen3_runtime/reference/hf_greedy.py:11-25)."""
    ids = list(prompt)
    out = []
    for _ in range(n):
        tok = greedy(forward(cfg, w, ids)[-1])
        out.append(tok)
        ids.append(tok)
    return out


def apply_penalties(logits, token_ids, repetition, presence, frequency):
    """qwen3_runtime/sampling.py:44-72: counts over prompt+generated ids; seen and >0 -> /r,
    seen and <=0 -> *r; minus presence * seen; minus frequency * count."""
    counts = torch.zeros(logits.numel(), dtype=torch.long)
    for t in token_ids:
        if 0 <= t < logits.numel():
            counts[t] += 1
    out = logits.clone()
    seen = counts > 0
    pos = out > 0
    out = torch.where(seen & pos, out / repetition, out)
    out = torch.where(seen & ~pos, out * repetition, out)
    out = out - presence * seen.to(out.dtype)
    out = out - frequency * counts.to(out.dtype)
    return out


def min_p_filter(logits, min_p):
    """qwen3_runtime/sampling.py:75-81: drop ids whose probability is below min_p * max prob."""
    probs = torch.softmax(logits, dim=-1)
    return torch.where(probs < min_p * probs.max(), torch.full_like(logits, float("-inf")), logits)


def top_k_filter(logits, k):
    """qwen3_runtime/sampling.py:98-101: keep values >= the k-th largest."""
    thresh = torch.topk(logits, min(k, logits.numel())).values[-1]
    return torch.where(logits < thresh, torch.full_like(logits, float("-inf")), logits)


def top_p_filter(logits, p):
    """qwen3_runtime/sampling.py:102-109: sort descending; drop an id when the mass before it
    already exceeds p (the first id past the mass is kept)."""
    sorted_logits, idx = torch.sort(logits, descending=True)
    cum = torch.softmax(sorted_logits, dim=-1).cumsum(dim=-1)
    remove_sorted = cum > p
    remove_sorted[1:] = remove_sorted[:-1].clone()
    remove_sorted[0] = False
    remove = torch.zeros_like(remove_sorted)
    remove[idx] = remove_sorted
    return torch.where(remove, torch.full_like(logits, float("-inf")), logits)


def inverse_cdf_draw(probs, u):
    """qwen3_runtime/sampling.py:208-227: first index whose cumulative mass exceeds u, clamped."""
    cdf = probs.cumsum(0)
    idx = int(torch.searchsorted(cdf, torch.tensor(u, dtype=cdf.dtype), right=True))
    return max(0, min(idx, probs.numel() - 1))
