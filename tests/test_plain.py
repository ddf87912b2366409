"""What fixes the plain implementation beside the reference's text: library routines it
must reduce to, vectors the reference's own tests hold, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain import ops_ref as R
from plain import qwen3_plain as P

torch.set_default_dtype(torch.float32)


# ---- RMSNorm ---------------------------------------------------------------------------------
def test_rms_norm_equals_the_library_routine_and_the_reference_vector():
    torch.manual_seed(0)
    x = torch.randn(4, 8)            # the reference's own vector: tests/cpu/test_rmsnorm.py:6-13
    w = torch.ones(8)
    var = x.float().pow(2).mean(dim=-1, keepdim=True)
    want = x.float() * torch.rsqrt(var + 1e-6) * w
    torch.testing.assert_close(P.rms_norm(x, w, 1e-6), want)
    w = 1 + 0.3 * torch.randn(8)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (8,), w, 1e-5))


def test_rms_norm_unit_rms_scale_invariance_and_weight_after_normalising():
    x = torch.randn(5, 64).double()
    y = P.rms_norm(x, torch.ones(64).double(), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5).double())
    torch.testing.assert_close(P.rms_norm(7.0 * x, torch.ones(64).double(), 1e-12), y)
    w = torch.rand(64).double() + 0.5
    torch.testing.assert_close(P.rms_norm(x, w, 1e-12), y * w)   # not (1 + w), not before the rsqrt


# ---- rotary -------------------------------------------------------------------------------------
def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    x = torch.randn(3, 2, 16).double()
    torch.testing.assert_close(P.rope_neox(x, torch.zeros(3, dtype=torch.long), 1e4), x)
    y = P.rope_neox(x, torch.tensor([5, 77, 1234]), 1e4)
    torch.testing.assert_close(y[..., :8] ** 2 + y[..., 8:] ** 2, x[..., :8] ** 2 + x[..., 8:] ** 2)


def test_rope_pairs_element_j_with_j_plus_half_not_with_its_neighbour():
    x = torch.zeros(1, 1, 8).double()
    x[0, 0, 1] = 1.0
    y = P.rope_neox(x, torch.tensor([3]), 100.0)[0, 0]
    ang = 3 * (100.0 ** (-2 / 8))
    assert y[1] == pytest.approx(math.cos(ang), abs=1e-6) and y[5] == pytest.approx(math.sin(ang), abs=1e-6)
    assert y[0] == 0 and y[2] == 0   # an interleaved pairing would have put the sine at index 0


def test_rope_is_a_complex_multiplication_and_depends_on_distance_only():
    torch.manual_seed(1)
    q, k = torch.randn(1, 1, 32).double(), torch.randn(1, 1, 32).double()
    inv = 1.0 / (1e6 ** (torch.arange(0, 32, 2, dtype=torch.float32) / 32))
    pos = torch.tensor([9])
    z = torch.complex(q[..., :16], q[..., 16:]) * torch.polar(torch.ones(16).double(), (pos.float() * inv).double())
    torch.testing.assert_close(P.rope_neox(q, pos, 1e6), torch.cat((z.real, z.imag), -1))

    def score(m, n):
        return (P.rope_neox(q, torch.tensor([m]), 1e4) * P.rope_neox(k, torch.tensor([n]), 1e4)).sum()

    # a wrong sign of the sine makes the score depend on m + n instead of m - n
    assert score(7, 3) == pytest.approx(float(score(40, 36)), abs=1e-4)
    assert abs(float(score(7, 3)) - float(score(3, 7))) > 1e-3


# ---- attention -------------------------------------------------------------------------------------
@pytest.mark.parametrize("nq,nkv,d,t", [(4, 2, 16, 9), (6, 2, 32, 17), (1, 1, 8, 5)])
def test_causal_attention_equals_the_library_routine(nq, nkv, d, t):
    torch.manual_seed(2)
    q, k, v = torch.randn(t, nq, d), torch.randn(t, nkv, d), torch.randn(t, nkv, d)
    g = nq // nkv
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat_interleave(g, 1).transpose(0, 1), v.repeat_interleave(g, 1).transpose(0, 1),
        is_causal=True).transpose(0, 1).reshape(t, nq * d)
    torch.testing.assert_close(P.causal_attention(q, k, v), want, atol=1e-5, rtol=1e-5)


def test_attention_special_cases():
    torch.manual_seed(3)
    q, k, v = torch.randn(1, 4, 8), torch.randn(1, 2, 8), torch.randn(1, 2, 8)
    # one token: the context is its own value, repeated over the group
    torch.testing.assert_close(P.causal_attention(q, k, v), v.repeat_interleave(2, 1).reshape(1, 32))
    # one query over a history without mask = plain softmax attention
    k, v = torch.randn(11, 2, 8), torch.randn(11, 2, 8)
    got = P.causal_attention(q, k, v, q_offset=10)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(2, 1).transpose(0, 1),
                                          v.repeat_interleave(2, 1).transpose(0, 1)).transpose(0, 1).reshape(1, 32)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    # query head h reads kv head h // g: changing kv head 1 leaves query heads 0 and 1 alone
    v2 = v.clone()
    v2[:, 1] += 1.0
    diff = (P.causal_attention(q, k, v2, q_offset=10) - got).reshape(4, 8).abs().sum(-1)
    assert diff[0] == 0 and diff[1] == 0 and diff[2] > 0 and diff[3] > 0


def test_a_portion_with_history_is_the_tail_of_the_whole():
    torch.manual_seed(4)
    q, k, v = torch.randn(20, 4, 8), torch.randn(20, 2, 8), torch.randn(20, 2, 8)
    whole = P.causal_attention(q, k, v)
    torch.testing.assert_close(P.causal_attention(q[13:], k, v, q_offset=13), whole[13:])
    # and the paged reference agrees with it, with pages in any physical order
    ps, pages = 4, [5, 2, 7, 0, 3]
    kc, vc = torch.zeros(8, 2, ps, 8), torch.zeros(8, 2, 8, ps)
    slots = torch.tensor([pages[p // ps] * ps + p % ps for p in range(20)])
    R.kv_store(k, v, kc, vc, slots, ps)
    got = R.paged_attention(q[13:].reshape(7, 32), kc, vc, [0, 7], [20], torch.tensor([pages]), ps, 4, 2, 8,
                            1 / math.sqrt(8))
    torch.testing.assert_close(got, whole[13:], atol=1e-6, rtol=1e-6)


def test_window_hides_keys_at_distance_window_and_beyond():
    torch.manual_seed(5)
    q, k, v = torch.randn(12, 2, 8), torch.randn(12, 2, 8), torch.randn(12, 2, 8)
    full = P.causal_attention(q, k, v)
    torch.testing.assert_close(P.causal_attention(q, k, v, window=12), full)
    w1 = P.causal_attention(q, k, v, window=1)
    torch.testing.assert_close(w1, v.reshape(12, 16))          # only itself
    w3 = P.causal_attention(q, k, v, window=3)
    torch.testing.assert_close(w3[:3], full[:3])
    assert (w3[5] - full[5]).abs().max() > 1e-4


# ---- feed-forward, embedding, head ----------------------------------------------------------------------
def test_swiglu_equals_library_silu_times_up():
    g, u = torch.randn(7, 33) * 3, torch.randn(7, 33)
    torch.testing.assert_close(P.swiglu(g, u), F.silu(g) * u)
    assert P.swiglu(torch.zeros(3), torch.randn(3)).abs().sum() == 0
    torch.testing.assert_close(R.swiglu(torch.cat((g, u), -1)), F.silu(g) * u)


# ---- the whole model ----------------------------------------------------------------------------------------
def test_whole_model_shift_of_positions_and_hand_computed_layer(model_folders):
    cfg, w = P.read_model(model_folders["tiny_b"])
    ids = torch.randint(0, cfg["vocab_size"], (12,))
    logits = P.forward(cfg, w, ids)
    assert logits.shape == (12, cfg["vocab_size"])
    # causal: a later token does not change earlier logits
    ids2 = ids.clone()
    ids2[-1] = (ids2[-1] + 1) % cfg["vocab_size"]
    torch.testing.assert_close(P.forward(cfg, w, ids2)[:-1], logits[:-1])
    # untied head is used (tiny_b), tied one for tiny_a
    assert not cfg["tie_word_embeddings"]
    h = P.rms_norm(w["model.embed_tokens.weight"][ids[:1]], w["model.layers.0.input_layernorm.weight"],
                   cfg["rms_norm_eps"])
    # position 0, one token: attention returns v; written out by hand for layer 0
    v = (h @ w["model.layers.0.self_attn.v_proj.weight"].T).view(1, 2, 32).repeat_interleave(3, 1).reshape(1, -1)
    want = v @ w["model.layers.0.self_attn.o_proj.weight"].T
    got = P.attention_layer(h, w, "model.layers.0.self_attn", cfg, torch.tensor([0]))
    torch.testing.assert_close(got, want)


def _library_attention_layer(x, wq, wk, pos, theta, eps):
    """One head, identity projections, written with library routines only: F.rms_norm, a complex
    multiplication for the rotation, F.scaled_dot_product_attention."""
    d = x.shape[-1]

    def rotate(v):
        inv = 1.0 / theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d)
        ang = (pos.float()[:, None] * inv[None, :]).double()
        z = torch.complex(v[:, : d // 2], v[:, d // 2:]) * torch.polar(torch.ones_like(ang), ang)
        return torch.cat((z.real, z.imag), -1)

    q = rotate(F.rms_norm(x, (d,), wq, eps))
    k = rotate(F.rms_norm(x, (d,), wk, eps))
    return F.scaled_dot_product_attention(q[None, None], k[None, None], x[None, None], is_causal=True)[0, 0]


def test_q_norm_comes_before_the_rotation():
    """With a non-uniform norm weight, norm-then-rotate differs from rotate-then-norm; the
    expected values come from library routines, not from the plain functions."""
    torch.manual_seed(6)
    d = 8
    cfg = dict(num_attention_heads=1, num_key_value_heads=1, head_dim=d, hidden_size=d, rms_norm_eps=1e-6,
               rope_theta=10.0)
    eye = torch.eye(d).double()
    wq = torch.tensor([0.1, 0.9, 0.2, 0.8, 0.3, 0.7, 0.4, 0.6]).double()
    wk = torch.tensor([1.0, 0.5, 1.5, 0.7, 0.9, 1.1, 0.6, 1.3]).double()
    w = {"a.q_proj.weight": eye, "a.k_proj.weight": eye, "a.v_proj.weight": eye, "a.o_proj.weight": eye,
         "a.q_norm.weight": wq, "a.k_norm.weight": wk}
    x = torch.randn(4, d).double()
    pos = torch.tensor([0, 3, 4, 9])
    got = P.attention_layer(x, w, "a", cfg, pos)
    torch.testing.assert_close(got, _library_attention_layer(x, wq, wk, pos, 10.0, 1e-6))
    # the plausible mistake: rotate first, then norm
    q_wrong = P.rms_norm(P.rope_neox(x.view(4, 1, d), pos, 10.0), wq, 1e-6)
    k_right = P.rope_neox(P.rms_norm(x.view(4, 1, d), wk, 1e-6), pos, 10.0)
    assert (P.causal_attention(q_wrong, k_right, x.view(4, 1, d)) - got).abs().max() > 1e-3


def _tiny_model(layers=2, tied=False, seed=0):
    """A hand-sized model with every norm weight different, in float64."""
    g = torch.Generator().manual_seed(seed)
    h, nq, nkv, d, i, v = 12, 2, 1, 4, 10, 17
    cfg = dict(num_hidden_layers=layers, hidden_size=h, num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d,
               intermediate_size=i, vocab_size=v, rms_norm_eps=1e-5, rope_theta=100.0, tie_word_embeddings=tied)
    rnd = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float64)
    w = {"model.embed_tokens.weight": rnd(v, h), "model.norm.weight": 1 + 0.5 * rnd(h), "lm_head.weight": rnd(v, h)}
    for l in range(layers):
        p = f"model.layers.{l}"
        w.update({f"{p}.input_layernorm.weight": 1 + 0.5 * rnd(h), f"{p}.post_attention_layernorm.weight": 1 + 0.5 * rnd(h),
                  f"{p}.self_attn.q_proj.weight": rnd(nq * d, h), f"{p}.self_attn.k_proj.weight": rnd(nkv * d, h),
                  f"{p}.self_attn.v_proj.weight": rnd(nkv * d, h), f"{p}.self_attn.o_proj.weight": rnd(h, nq * d),
                  f"{p}.self_attn.q_norm.weight": 1 + 0.5 * rnd(d), f"{p}.self_attn.k_norm.weight": 1 + 0.5 * rnd(d),
                  f"{p}.mlp.gate_proj.weight": rnd(i, h), f"{p}.mlp.up_proj.weight": rnd(i, h),
                  f"{p}.mlp.down_proj.weight": rnd(h, i)})
    return cfg, w


def test_the_order_of_the_layers_parts_by_special_cases_that_reduce_to_library_routines():
    """Where the norms stand, what the residual adds, the final norm and the head, each pinned by a
    model in which all but one sub-layer is switched off (its output matrix zeroed), so that the
    logits can be written with F.rms_norm, F.silu and F.linear alone. A post-norm block, a residual
    taken from the normed tensor, the feed-forward behind the wrong norm, a missing final norm or
    the embedding used where the model has a head of its own each fail one of these."""
    eps = 1e-5
    norm = lambda x, wt: F.rms_norm(x, (x.shape[-1],), wt, eps)
    ids = torch.tensor([3, 11, 5, 3, 16])

    # 1. every sub-layer off: logits = head(final_norm(embedding))
    cfg, w = _tiny_model(layers=2)
    for l in range(2):
        w[f"model.layers.{l}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{l}.mlp.down_proj.weight"].zero_()
    e = w["model.embed_tokens.weight"][ids]
    torch.testing.assert_close(P.forward(cfg, w, ids), F.linear(norm(e, w["model.norm.weight"]), w["lm_head.weight"]))
    cfg_tied = dict(cfg, tie_word_embeddings=True)
    torch.testing.assert_close(P.forward(cfg_tied, w, ids),
                               F.linear(norm(e, w["model.norm.weight"]), w["model.embed_tokens.weight"]))

    # 2. only the feed-forward of layer 1 on: h = e + down(silu(gate n) * up n), n = post-attention norm of e
    cfg, w = _tiny_model(layers=2, seed=1)
    for l in range(2):
        w[f"model.layers.{l}.self_attn.o_proj.weight"].zero_()
    w["model.layers.0.mlp.down_proj.weight"].zero_()
    e = w["model.embed_tokens.weight"][ids]
    p = "model.layers.1"
    n = norm(e, w[f"{p}.post_attention_layernorm.weight"])
    ff = F.linear(F.silu(F.linear(n, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(n, w[f"{p}.mlp.up_proj.weight"]),
                  w[f"{p}.mlp.down_proj.weight"])
    want = F.linear(norm(e + ff, w["model.norm.weight"]), w["lm_head.weight"])
    torch.testing.assert_close(P.forward(cfg, w, ids), want)
    for wrong in (F.linear(norm(n + ff, w["model.norm.weight"]), w["lm_head.weight"]),           # residual from the normed tensor
                  F.linear(norm(norm(e + ff, w[f"{p}.post_attention_layernorm.weight"]), w["model.norm.weight"]),
                           w["lm_head.weight"])):                                                 # post-norm
        assert (wrong - want).abs().max() > 1e-2

    # 3. only the attention of layer 0 on, one token (attention then returns its value):
    #    h = e + o(repeat(v(input norm of e)))
    cfg, w = _tiny_model(layers=2, seed=2)
    for l in range(2):
        w[f"model.layers.{l}.mlp.down_proj.weight"].zero_()
    w["model.layers.1.self_attn.o_proj.weight"].zero_()
    one = ids[:1]
    e = w["model.embed_tokens.weight"][one]
    p = "model.layers.0"
    n = norm(e, w[f"{p}.input_layernorm.weight"])
    v = F.linear(n, w[f"{p}.self_attn.v_proj.weight"]).view(1, 1, 4).repeat_interleave(2, 1).reshape(1, 8)
    want = F.linear(norm(e + F.linear(v, w[f"{p}.self_attn.o_proj.weight"]), w["model.norm.weight"]), w["lm_head.weight"])
    torch.testing.assert_close(P.forward(cfg, w, one), want)

    # 4. both sub-layers of one layer on, two tokens: the feed-forward sees the stream after the
    #    attention's add, through the post-attention norm (attention from library routines)
    cfg, w = _tiny_model(layers=1, seed=3)
    two = ids[:2]
    e = w["model.embed_tokens.weight"][two]
    n = norm(e, w[f"{p}.input_layernorm.weight"])
    d = 4
    def heads(x, k):
        return x.view(2, k, d)
    def rotate(x):
        inv = 1.0 / 100.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d)
        ang = (torch.arange(2).float()[:, None] * inv[None, :]).double()[:, None, :]
        z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * torch.polar(torch.ones_like(ang), ang)
        return torch.cat((z.real, z.imag), -1)
    q = rotate(F.rms_norm(heads(F.linear(n, w[f"{p}.self_attn.q_proj.weight"]), 2), (d,), w[f"{p}.self_attn.q_norm.weight"], eps))
    k = rotate(F.rms_norm(heads(F.linear(n, w[f"{p}.self_attn.k_proj.weight"]), 1), (d,), w[f"{p}.self_attn.k_norm.weight"], eps))
    v = heads(F.linear(n, w[f"{p}.self_attn.v_proj.weight"]), 1)
    attn = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(2, 1).transpose(0, 1)[None],
                                          v.repeat_interleave(2, 1).transpose(0, 1)[None], is_causal=True)[0]
    h1 = e + F.linear(attn.transpose(0, 1).reshape(2, 8), w[f"{p}.self_attn.o_proj.weight"])
    n2 = norm(h1, w[f"{p}.post_attention_layernorm.weight"])
    h2 = h1 + F.linear(F.silu(F.linear(n2, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(n2, w[f"{p}.mlp.up_proj.weight"]),
                       w[f"{p}.mlp.down_proj.weight"])
    torch.testing.assert_close(P.forward(cfg, w, two), F.linear(norm(h2, w["model.norm.weight"]), w["lm_head.weight"]))


def test_engine_formulation_equals_plain_on_cpu(model_folders):
    """The fused residual chain (pending add + norm) is algebraically the plain pre-norm block
    (reference asserts the same of its own two forms: tests/cpu/test_tiny_qwen3.py:23-37)."""
    import traces
    from test_engine_host import load_cpu

    cfg, w = P.read_model(model_folders["tiny_a"])
    reqs = {"x": torch.randint(0, cfg["vocab_size"], (5,)).tolist()}
    got = traces.replay(load_cpu(model_folders["tiny_a"], 16, 4), traces.whole(reqs))
    traces.compare(got, traces.plain_logits(model_folders["tiny_a"], reqs), atol=1e-5, rtol=1e-5)


# ---- sampling -----------------------------------------------------------------------------------------------------
def test_greedy_vectors():
    # reference: tests/cpu/test_sampling.py:95-118
    assert P.greedy(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1
    assert P.greedy(torch.zeros(8)) == 0
    assert [P.greedy(r) for r in torch.tensor([[0.1, 0.7, 0.2], [3.0, -1.0, 2.5]])] == [1, 0]


def test_filters_and_draw():
    logits = torch.tensor([0.0, 4.0, 1.0, 3.0])
    assert P.greedy(P.top_k_filter(logits, 1)) == 1 and torch.isinf(P.top_k_filter(logits, 1)).sum() == 3
    probs = torch.tensor([0.6, 0.3, 0.1])
    kept = P.top_p_filter(probs.log(), 0.7)
    assert torch.isinf(kept).tolist() == [False, False, True]      # the id that crosses the mass stays
    assert torch.isinf(P.min_p_filter(probs.log(), 0.4)).tolist() == [False, False, True]
    assert [P.inverse_cdf_draw(probs, u) for u in (0.0, 0.59, 0.61, 0.95, 0.9999999)] == [0, 0, 1, 2, 2]
    pen = P.apply_penalties(torch.tensor([2.0, -2.0, 1.0]), [0, 0, 1], 2.0, 0.5, 0.25)
    torch.testing.assert_close(pen, torch.tensor([2.0 / 2 - 0.5 - 0.5, -2.0 * 2 - 0.5 - 0.25, 1.0]))
