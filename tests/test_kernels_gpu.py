"""Each HIP kernel alone against its plain torch reference (tests/plain/ops_ref.py),
at sizes other than the engine's: odd widths, head sizes in steps of 16, group
sizes that do not divide a tile, pages of 8 to 64 tokens."""

import math

import pytest
import torch

from plain import ops_ref as R

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from qwen3_runtime_amd.ops.hip import HipOps

    return HipOps()


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, atol, rtol):
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("v,h,t", [(300, 100, 7), (64, 2560, 3)])
def test_embed(ops, dtype, v, h, t):
    table = rnd(v, h, dtype=dtype)
    ids = torch.randint(0, v, (t,), dtype=torch.int32, device=DEV)
    close(ops.embed(ids, table), R.embed(ids, table), 0, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,h,eps", [(5, 96, 1e-5), (3, 2560, 1e-6), (9, 1000, 1e-6)])
def test_add_rmsnorm(ops, dtype, t, h, eps):
    res = rnd(t, h, seed=1)
    delta = rnd(t, h, dtype=dtype, seed=2)
    w = (1 + 0.1 * rnd(h, seed=3)).contiguous()
    want_res = res.clone()
    want = R.add_rmsnorm(want_res, delta, w, eps, dtype)
    got_res = res.clone()
    got = ops.add_rmsnorm(got_res, delta, w, eps, dtype)
    close(got_res, want_res, 0, 0)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    close(got, want, tol, tol)
    # no delta; rows subset leaves the residual alone
    rows = torch.tensor([t - 1, 0], dtype=torch.int32, device=DEV)
    got_res = res.clone()
    got = ops.add_rmsnorm(got_res, delta, w, eps, dtype, rows)
    close(got_res, res, 0, 0)
    close(got, R.add_rmsnorm(res.clone(), delta, w, eps, dtype, rows), tol, tol)
    close(ops.add_rmsnorm(res.clone(), None, w, eps, dtype), R.add_rmsnorm(res.clone(), None, w, eps, dtype), tol, tol)


@pytest.mark.parametrize("planes", [1, 2, 3, 4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize("t,h", [(3, 2560), (2, 5000), (4, 4096), (5, 101), (1, 8)])
def test_add_rmsnorm_sums_planes_in_order(ops, planes, t, h):
    """The delta in planes [P, T, H] (float32): the residual becomes ((res + p0) + p1) + ..., bit
    for bit, for plane counts the kernel unrolls (1, 2, 4) and those it loops over, for rows held
    in registers, rows wider than that (5,000) and rows that cannot be read four at a time (101)."""
    res = rnd(t, h, seed=1)
    delta = rnd(planes, t, h, seed=2)
    w = (1 + 0.1 * rnd(h, seed=3)).contiguous()
    want_res = res.clone()
    for p in range(planes):
        want_res = want_res + delta[p]
    got_res = res.clone()
    got = ops.add_rmsnorm(got_res, delta, w, 1e-6, torch.bfloat16)
    close(got_res, want_res, 0, 0)
    close(got, R.add_rmsnorm(want_res.clone(), None, w, 1e-6, torch.bfloat16), 1e-2, 1e-2)
    rows = torch.tensor([t - 1, 0], dtype=torch.int32, device=DEV)
    untouched = res.clone()
    sel = ops.add_rmsnorm(untouched, delta, w, 1e-6, torch.bfloat16, rows)
    close(untouched, res, 0, 0)
    close(sel, got[rows.long()], 0, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(ops, dtype):
    gu = rnd(11, 2 * 272, dtype=dtype, scale=3.0)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    close(ops.swiglu(gu), R.swiglu(gu), tol, tol)
    zero_gate = gu.clone()
    zero_gate[:, :272] = 0
    assert ops.swiglu(zero_gate).abs().max().item() == 0.0


@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (7, 272, 96), (33, 100, 50), (130, 384, 192), (65, 1000, 2560)])
def test_gemm_f32(ops, m, n, k):
    x, w = rnd(m, k, seed=1), rnd(n, k, seed=2, scale=0.05)
    want = (x.double() @ w.double().T).float()
    close(ops.linear(x, w), want, 1e-4, 1e-4)


def test_gemm_f32_rows_do_not_depend_on_batch(ops):
    x, w = rnd(70, 200, seed=1), rnd(150, 200, seed=2)
    whole = ops.linear(x, w)
    alone = ops.linear(x[40:41].contiguous(), w)
    assert torch.equal(whole[40:41], alone)


@pytest.mark.parametrize("out_f32", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (8, 272, 96), (17, 100, 48), (40, 384, 272), (100, 1000, 2560),
                                   (3, 50, 20)])
def test_gemm_bf16(ops, m, n, k, out_f32):
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    want = x.double() @ w.double().T
    got = ops.linear(x, w, out_f32=out_f32)
    assert got.dtype == (torch.float32 if out_f32 else torch.bfloat16)
    if out_f32:
        close(got, want, 1e-3, 1e-3)
    else:
        close(got, want, 2e-2, 2e-2)


@pytest.mark.parametrize("m,i,k", [(1, 9728, 2560), (8, 288, 96), (33, 100, 64), (64, 272, 96), (70, 64, 64),
                                   (5, 64, 48), (16, 1000, 128)])
def test_gated_linear(ops, m, i, k, monkeypatch):
    """The fused form (few rows) and the two-kernel form agree with the plain one."""
    for dtype in (torch.bfloat16, torch.float32):
        x, w = rnd(m, k, dtype=dtype, seed=3), rnd(2 * i, k, dtype=dtype, seed=4, scale=0.05)
        gu = x.double() @ w.double().T
        if dtype == torch.bfloat16:
            gu = gu.to(torch.bfloat16).double()     # the unfused kernels round here
        want = R.swiglu(gu)
        tol = 3e-2 if dtype == torch.bfloat16 else 1e-4
        got = ops.gated_linear(x, w)
        assert got.shape == (m, i)
        close(got, want, tol, tol)


@pytest.mark.parametrize("m", [1, 8, 16, 17, 32, 40, 64, 65])
@pytest.mark.parametrize("n,k", [(6144, 2560), (2560, 4096), (1008, 9728), (272, 96), (272, 192)])
def test_gemm_bf16_few_rows_at_model_sizes(m, n, k):
    """Up to 16 rows the few-row kernel; 17 to 64 rows the kernel that shares the activations
    through LDS if K is a multiple of 64; otherwise, and beyond, the vendor library. All of them
    against a float64 product."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps()
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.02)
    want = x.double() @ w.double().T
    got = ops.linear(x, w, out_f32=True)
    assert got.dtype == torch.float32
    close(got, want, 2e-3, 2e-3)
    close(ops.linear(x, w), want, 3e-2, 3e-2)


@pytest.mark.parametrize("m", [1, 3, 8, 11, 12, 16, 17, 31, 33, 48, 64, 65, 96, 128])
@pytest.mark.parametrize("n,k,gated", [(6144, 2560, False), (2560, 4096, False), (608, 9728, False), (64, 64, False),
                                       (9728, 2560, True), (48, 96, True), (151936, 256, False), (80, 128, True),
                                       (4112, 640, True), (16, 64, False)])
def test_products_of_1_to_128_rows_whole_and_gated(m, n, k, gated):
    """Every number of rows that changes the kernel (few-row up to 16 rows or below the form's
    threshold, sharing the activations through LDS beyond, in accumulator blocks of 16 rows up to
    64 or 128) at shapes with one tile, with fewer tiles than a block takes, with more tiles than
    compute units, with very many; against a float64 product."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps()
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * n if gated else n, k, dtype=torch.bfloat16, seed=2, scale=0.03)
    if gated:
        want = R.swiglu((x.double() @ w.double().T).to(torch.bfloat16).double())
        close(ops.gated_linear(x, w), want, 3e-2, 3e-2)
    else:
        want = x.double() @ w.double().T
        close(ops.linear(x, w, out_f32=True), want, 2e-3, 2e-3)
        close(ops.linear(x, w), want, 3e-2, 3e-2)


@pytest.mark.parametrize("m", [1, 3, 8, 9, 16, 17, 40, 64, 70, 128, 129])
@pytest.mark.parametrize("n,k", [(2560, 4096), (2560, 9728), (96, 2048), (6144, 2560), (64, 64), (4096, 12288)])
def test_product_for_the_residual_may_come_in_planes(m, n, k):
    """linear_for_residual's planes sum to the product, and add_rmsnorm adds them like one delta."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps()
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.03)
    want = x.double() @ w.double().T
    got = ops.linear_for_residual(x, w)
    kernel = ops._own_kernel(m, n, k, "planes")
    parts = ops.choose_k_parts(n, k, m, kernel == 1) if kernel is not None and k % 64 == 0 else 1
    assert (kernel == 1) == (9 <= m <= 128 and k % 64 == 0 and k >= 128)
    assert (kernel == 0) == (m < 9 or (m <= 16 and k < 128))
    if parts > 1:
        assert got.dim() == 3 and got.shape[0] == parts and got.dtype == torch.float32
        close(got.sum(0), want, 2e-3, 2e-3)
    else:
        assert got.dim() == 2
        close(got, want, 3e-2, 3e-2)
    res = rnd(m, n, seed=4)
    weight = (1 + 0.1 * rnd(n, seed=5)).contiguous()
    one = got if got.dim() == 2 else got.sum(0).to(torch.bfloat16)
    res_a, res_b = res.clone(), res.clone()
    ya = ops.add_rmsnorm(res_a, got, weight, 1e-6, torch.bfloat16)
    yb = ops.add_rmsnorm(res_b, one, weight, 1e-6, torch.bfloat16)
    close(res_a, res_b, 2e-2, 2e-2)
    close(ya, yb, 3e-2, 3e-2)
    want_res = res.double() + want
    close(res_a, want_res, 3e-2, 3e-2)
    rows = torch.tensor([m - 1, 0], dtype=torch.int32, device=DEV)
    yc = ops.add_rmsnorm(res.clone(), got, weight, 1e-6, torch.bfloat16, rows)
    close(yc, ya[rows.long()], 0, 0)


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k,gated", [(1000, 320, False), (50, 64, False), (2560, 4096, False), (4112, 640, True),
                                       (16, 128, False), (40, 192, True), (6144, 2560, False), (33000, 128, False),
                                       (640, 5120, False), (9, 2048, True)])
def test_few_rows_on_weights_as_stored(m, n, k, gated):
    """The few-row kernel that brings row-major weights through LDS by direct loads, called as the
    library exports it: any number of weight rows (the last tile repeats the last row), K in pairs
    of k-steps that do not divide evenly among the waves or the parts, whole and in 2, 4 and 8
    planes (some of them empty), against a float64 product. A piece of a row in another row's
    place, or a pair read before it has landed, would show in every entry."""
    from ctypes import c_int

    from qwen3_runtime_amd.ops.hip import BF16, F32, HipOps, _ptr, _stream

    ops = HipOps()
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * n if gated else n, k, dtype=torch.bfloat16, seed=2, scale=0.03)
    if gated:
        want = R.swiglu((x.double() @ w.double().T).to(torch.bfloat16).double())
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops._check(ops.lib, ops.lib.qrt_gemm_bf16(_ptr(x), _ptr(w), _ptr(out), BF16, c_int(m), c_int(n), c_int(k),
                                                  c_int(1), c_int(0), c_int(1), _stream()))
        close(out, want, 3e-2, 3e-2)
        return
    want = x.double() @ w.double().T
    for parts in (1, 2, 4, 8):
        out = torch.full((parts, m, n), float("nan"), dtype=torch.float32, device=DEV)
        ops._check(ops.lib, ops.lib.qrt_gemm_bf16(_ptr(x), _ptr(w), _ptr(out), F32, c_int(m), c_int(n), c_int(k),
                                                  c_int(0), c_int(0), c_int(parts), _stream()))
        close(out.sum(0), want, 2e-3, 2e-3)
    # planes need the kernel that can cut K: more rows, or a K that is no multiple of 64, are refused
    with pytest.raises(Exception, match="K parts"):
        big = rnd(17, k, dtype=torch.bfloat16, seed=3)
        out = torch.empty((2, 17, n), dtype=torch.float32, device=DEV)
        ops._check(ops.lib, ops.lib.qrt_gemm_bf16(_ptr(big), _ptr(w), _ptr(out), F32, c_int(17), c_int(n), c_int(k),
                                                  c_int(0), c_int(0), c_int(2), _stream()))


@pytest.mark.parametrize("m", [1, 8, 64])
def test_vocabulary_head_at_its_real_size(m):
    """The head of the 4B and 8B models, 151,936 x 2,560, through the dispatch a decode step uses
    (the few-row kernel with two row tiles per block up to 16 rows; the kernel that shares
    activations, eight tiles per block, for 64),
    float32 out, against a float64 product of the same bfloat16 values computed on the device."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps()
    n, k = 151936, 2560
    x = rnd(m, k, dtype=torch.bfloat16, seed=5)
    g = torch.Generator(device=DEV).manual_seed(17)
    w = (0.02 * torch.randn(n, k, generator=g, device=DEV, dtype=torch.float32)).to(torch.bfloat16)
    assert ops._own_kernel(m, n, k, "whole") == (0 if m <= 16 else 1)
    got = ops.linear(x, w, out_f32=True)
    want = torch.empty((m, n), dtype=torch.float64, device=DEV)
    for lo in range(0, n, 16384):                       # in pieces: the float64 copy of W is 3 GB otherwise
        want[:, lo: lo + 16384] = x.double() @ w[lo: lo + 16384].double().T
    err = (got.double() - want).abs()
    # entries are sums of 2,560 products of size 0.02: about one in size; float32 sums err by 1e-5 or so
    assert 0.5 < float(want.abs().mean()) < 1.5 and float(err.max()) < 2e-4, float(err.max())
    assert torch.equal(got.argmax(-1), want.argmax(-1))


def test_gemm_bf16_large_uses_blas_and_agrees(ops):
    x, w = rnd(300, 512, dtype=torch.bfloat16, seed=1), rnd(640, 512, dtype=torch.bfloat16, seed=2, scale=0.05)
    close(ops.linear(x, w), x.double() @ w.double().T, 3e-2, 3e-2)
    close(ops.linear(x, w, out_f32=True), x.double() @ w.double().T, 1e-3, 1e-3)


def test_library_product_in_two_column_chunks():
    """Products with many rows go to the vendor library, whole or as two calls over column chunks
    of one result tensor; which, follows from the shape alone, so two processes give the same
    bits. Both ways give the float64 product."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps()
    m, n, k = 300, 33000, 64                       # two row tiles: 32,768 columns fill the chip once
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    want = x.double() @ w.double().T
    assert ops.library_split(m, n) == 32768
    chunked = ops.linear(x, w)
    assert chunked.is_contiguous() and chunked.shape == (m, n)
    close(chunked, want, 3e-2, 3e-2)
    assert torch.equal(chunked, HipOps().linear(x, w))   # nothing measured, nothing remembered
    ops.library_split_min_rows = 0                 # switched off: one call
    assert ops.library_split(m, n) == 0
    close(ops.linear(x, w), want, 3e-2, 3e-2)
    ops = HipOps()
    assert ops.library_split(200, n) == 0          # few rows: never split
    assert ops.library_split(m, 30000) == 0        # fewer columns than one round
    assert ops.library_split(2048, 19456) == 16384 and ops.library_split(2048, 24576) == 0   # 2.4 rounds; 3 whole ones


def test_float32_weight_with_bfloat16_activations_stays_float32(ops):
    x, w = rnd(5, 64, dtype=torch.bfloat16), rnd(48, 64, scale=0.1)
    close(ops.linear(x, w, out_f32=True), x.double() @ w.double().T, 1e-5, 1e-5)


def make_cache(pages, nkv, ps, d, dtype):
    from qwen3_runtime_amd.parts.base import CacheView, GroupView
    from qwen3_runtime_amd.parts.plan import CacheSpec

    k = torch.zeros(pages, nkv, ps, d, dtype=dtype, device=DEV)
    v = torch.zeros(pages, nkv, d, ps, dtype=dtype, device=DEV)
    view = CacheView(CacheSpec("paged_kv", heads=nkv, head_dim=d), group=GroupView(ps, None, None, None), k=k, v=v)
    return view


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,ps,theta", [(4, 2, 16, 16, 1e4), (6, 2, 32, 8, 1e6), (3, 1, 80, 4, 5e5),
                                               (8, 8, 128, 32, 1e6), (2, 1, 256, 16, 1e4)])
def test_qk_norm_rope_store(ops, dtype, nq, nkv, d, ps, theta):
    t, pages = 13, 12
    qkv = rnd(t, (nq + 2 * nkv) * d, dtype=dtype)
    qw, kw = 1 + 0.1 * rnd(d, seed=5), 1 + 0.1 * rnd(d, seed=6)
    inv = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    pos = torch.tensor([0, 1, 2, 3, 500, 501, 7, 8, 9, 4000, 4001, 30000, 5], dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * ps)[:t].to(torch.int32).to(DEV)
    cache = make_cache(pages, nkv, ps, d, dtype)
    cache.group.slots = slots
    want_cache = make_cache(pages, nkv, ps, d, dtype)
    want = R.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, want_cache.k, want_cache.v, slots, ps)
    got = ops.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, cache)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(got, want, tol, tol)
    close(cache.k, want_cache.k, tol, tol)
    close(cache.v, want_cache.v, 0, 0)
    # no norm, no rotation: a copy
    got = ops.qk_norm_rope_store(qkv, nq, nkv, d, None, None, 0.0, None, pos, None)
    close(got, qkv[:, : nq * d], 0, 0)
    # unfused pieces agree with the fused pass
    q, k, v = ops.qk_norm_split(qkv, nq, nkv, d, qw, kw, 1e-6)
    q, k = ops.rope_neox(q, k, pos, inv)
    cache2 = make_cache(pages, nkv, ps, d, dtype)
    cache2.group.slots = slots
    ops.kv_store(k, v, cache2)
    close(q.reshape(t, -1), want, tol, tol)
    close(cache2.k, want_cache.k, tol, tol)
    close(cache2.v, want_cache.v, 0, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,nq,nkv,d,ps", [(300, 8, 2, 128, 16), (257, 3, 1, 32, 8), (512, 4, 4, 256, 16)])
def test_qk_norm_rope_store_with_the_steps_table_of_angles(ops, dtype, t, nq, nkv, d, ps):
    """A long step computes its cosines and sines once (``rope_table``) and every layer's kernel
    looks them up: the same bits as the kernel that computes them itself, and the plain formulas."""
    from types import SimpleNamespace

    pages = (t + ps - 1) // ps + 2
    qkv = rnd(t, (nq + 2 * nkv) * d, dtype=dtype, seed=3)
    qw, kw = 1 + 0.1 * rnd(d, seed=5), 1 + 0.1 * rnd(d, seed=6)
    inv = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    pos = (torch.arange(t, dtype=torch.int32) + 4000).to(DEV)
    slots = torch.randperm(pages * ps)[:t].to(torch.int32).to(DEV)
    caches = [make_cache(pages, nkv, ps, d, dtype) for _ in range(3)]
    for c in caches:
        c.group.slots = slots
    ctx = SimpleNamespace(per_pass={}, positions=pos, num_tokens=t)
    looked_up = ops.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, caches[0], ctx=ctx)
    assert len(ctx.per_pass) == 1, "the step's table of angles was not made"
    computed = ops.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, caches[1])
    close(looked_up, computed, 0, 0)
    close(caches[0].k, caches[1].k, 0, 0)
    close(caches[0].v, caches[1].v, 0, 0)
    want = R.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, caches[2].k, caches[2].v, slots, ps)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(looked_up, want, tol, tol)
    close(caches[0].k, caches[2].k, tol, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,nq,nkv,d,ps,start", [(40, 6, 2, 32, 8, 16), (37, 4, 2, 64, 16, 8), (33, 4, 2, 16, 8, 3),
                                                 (700, 32, 8, 128, 16, 0), (9, 3, 1, 48, 8, 0)])
def test_qk_norm_rope_store_neighbouring_slots(ops, dtype, t, nq, nkv, d, ps, start):
    """A prompt portion: consecutive positions in consecutive slots, so that values go into their
    transposed pages eight tokens at a time (where the run starts on a multiple of eight) or one
    by one (start 3, and the tail of every run); with 700 tokens a wave makes all passes over the
    heads of its token."""
    pages = (start + t + ps - 1) // ps + 2
    qkv = rnd(t, (nq + 2 * nkv) * d, dtype=dtype)
    qw, kw = 1 + 0.1 * rnd(d, seed=5), 1 + 0.1 * rnd(d, seed=6)
    inv = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    pos = torch.arange(start, start + t, dtype=torch.int32, device=DEV)
    order = torch.randperm(pages)
    slots = torch.tensor([int(order[p // ps]) * ps + p % ps for p in range(start, start + t)], dtype=torch.int32, device=DEV)
    cache = make_cache(pages, nkv, ps, d, dtype)
    cache.group.slots = slots
    want_cache = make_cache(pages, nkv, ps, d, dtype)
    want = R.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, want_cache.k, want_cache.v, slots, ps)
    got = ops.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, pos, cache)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(got, want, tol, tol)
    close(cache.k, want_cache.k, tol, tol)
    close(cache.v, want_cache.v, 0, 0)


def build_attention_case(seqs, nq, nkv, d, ps, dtype, seed=0, window=None, shuffle=True, spare_pages=3,
                         poison=False):
    """seqs: list of (q_len, kv_len). Returns q, cache view with filled pages, ctx. ``poison``:
    every place no sequence has written (the rest of each sequence's last page, pages in no
    table) holds NaN or an infinity instead of noise, as a page's last holder may have left."""
    from qwen3_runtime_amd.parts.base import StepContext

    g = torch.Generator().manual_seed(seed)
    total_pages = sum((kv + ps - 1) // ps for _, kv in seqs) + spare_pages
    order = torch.randperm(total_pages, generator=g) if shuffle else torch.arange(total_pages)
    width = max((kv + ps - 1) // ps for _, kv in seqs)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    cache = make_cache(total_pages, nkv, ps, d, dtype)
    # stale content everywhere: a kernel that reads past kv_len or a foreign page shows
    cache.k.copy_((torch.randn(cache.k.shape, generator=g) * 3).to(dtype))
    cache.v.copy_((torch.randn(cache.v.shape, generator=g) * 3).to(dtype))
    nxt = 0
    for s, (_, kv) in enumerate(seqs):
        n = (kv + ps - 1) // ps
        table[s, :n] = order[nxt: nxt + n].to(torch.int32)
        nxt += n
    if poison:
        written = torch.zeros(total_pages, ps, dtype=torch.bool)
        for s, (_, kv) in enumerate(seqs):
            pos = torch.arange(kv)
            written[table[s, pos // ps].long(), pos % ps] = True
        bad = torch.tensor([float("nan"), float("inf"), float("-inf")])[torch.arange(total_pages * ps) % 3]
        bad = bad.view(total_pages, ps).to(dtype).to(DEV)
        unwritten = (~written).to(DEV)
        cache.k.copy_(torch.where(unwritten[:, None, :, None], bad[:, None, :, None], cache.k))
        cache.v.copy_(torch.where(unwritten[:, None, None, :], bad[:, None, None, :], cache.v))
    t = sum(q for q, _ in seqs)
    q = (torch.randn(t, nq * d, generator=g)).to(dtype).to(DEV)
    cu = [0]
    positions, seq_of = [], []
    for s, (ql, kv) in enumerate(seqs):
        cu.append(cu[-1] + ql)
        positions += list(range(kv - ql, kv))
        seq_of += [s] * ql
    cache.group.block_table = table.to(DEV)
    cache.group.window = window
    dev_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    ctx = StepContext(
        ops=None, dtype=dtype, device=torch.device(DEV), num_tokens=t, num_seqs=len(seqs),
        positions=dev_i32(positions), cu_q=dev_i32(cu), kv_lens=dev_i32([kv for _, kv in seqs]),
        seq_of_token=dev_i32(seq_of), state_slots=dev_i32([0] * len(seqs)), first_span=dev_i32([0] * len(seqs)),
        q_lens_host=[ql for ql, _ in seqs], kv_lens_host=[kv for _, kv in seqs],
        max_q_len=max(ql for ql, _ in seqs), max_kv_len=max(kv for _, kv in seqs), groups=[cache.group],
    )
    return q, cache, ctx


ATTN_CASES = [
    # (seqs, nq, nkv, d, page)
    ([(1, 1)], 4, 2, 16, 16),
    ([(7, 7), (1, 40), (33, 33)], 4, 2, 16, 16),
    ([(5, 37), (1, 17), (2, 95), (24, 24)], 6, 2, 32, 8),
    ([(1, 300), (1, 17), (1, 64), (1, 65)], 6, 2, 32, 8),
    ([(70, 70)], 5, 1, 48, 24),
    ([(3, 130), (64, 64)], 8, 2, 64, 64),
    ([(40, 200), (1, 1000)], 32, 8, 128, 16),
    ([(9, 50)], 3, 3, 80, 16),
    ([(1, 700)], 34, 2, 16, 32),
    ([(1, 100), (2, 61), (1, 24)], 4, 2, 32, 24),   # page sizes that are no power of two
    ([(20, 131), (300, 300)], 4, 1, 64, 40),
    ([(150, 210)], 2, 1, 256, 16),                  # a long portion at a head size whose LDS stages do not fit
    ([(1, 333), (1, 40), (2, 700)], 4, 1, 256, 16),  # the decode kernel at head size 256 (more LDS than the default)
    ([(1, 1500), (90, 90)], 4, 2, 256, 16),          # ... and beside a portion: two launches
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqs,nq,nkv,d,ps", ATTN_CASES)
def test_paged_attention(ops, dtype, seqs, nq, nkv, d, ps):
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, dtype)
    scale = 1.0 / math.sqrt(d)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale)
    got = ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, None)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(got, want, tol, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqs,nq,nkv,d,ps", [
    ([(7, 7), (1, 41), (33, 35), (1, 1)], 4, 2, 16, 16),     # general kernel; decode kernel for the single tokens alone
    ([(1, 300), (1, 17), (1, 61), (1, 67)], 8, 2, 64, 8),    # decode kernel, several key splits
    ([(150, 213), (70, 70)], 4, 1, 128, 16),                 # long portions through LDS
    ([(100, 1501)], 8, 2, 64, 32),                           # ... with the keys cut over blocks
    ([(1, 1203), (90, 91)], 32, 8, 128, 16),                 # two launches
    ([(150, 211)], 2, 1, 256, 16),                           # general kernel with two row tiles
])
def test_paged_attention_ignores_what_a_page_held_before(ops, dtype, seqs, nq, nkv, d, ps):
    """Every place of the cache that the sequences have not written holds NaN or an infinity: the
    rest of each last page (within the last group of 8 keys and after it) and every page in no
    table. A kernel that multiplies such a value, by a probability of zero too, shows it."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, dtype, poison=True)
    scale = 1.0 / math.sqrt(d)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale)
    assert torch.isfinite(want.float()).all()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, None), want, tol, tol)
    if dtype == torch.bfloat16:
        for splits in (2, 5):
            ctx.scratch["attn_splits"] = splits
            close(ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, None), want, tol, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 5, 32, 100])
def test_paged_attention_window(ops, dtype, window):
    seqs, nq, nkv, d, ps = [(6, 90), (1, 41), (50, 50)], 4, 2, 32, 8
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, dtype, window=window)
    # pages wholly below the window of the first query are gone
    table = cache.group.block_table.clone()
    for s, (ql, kv) in enumerate(seqs):
        first_needed = kv - ql - window + 1
        for p in range(table.shape[1]):
            if (p + 1) * ps <= first_needed:
                table[s, p] = -1
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 0.25, window)
    cache.group.block_table = table
    got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.25, window)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    close(got, want, tol, tol)


@pytest.mark.parametrize("nq,nkv,d,ps,window,norm,rope", [
    (32, 8, 128, 16, None, True, True),     # the 4B geometry
    (8, 2, 64, 16, None, True, True),
    (5, 1, 128, 24, None, True, True),      # five query heads per key head, pages of 24
    (16, 1, 64, 8, None, True, False),      # sixteen rows: no row to spare; no rotation
    (4, 4, 256, 16, None, False, True),     # one query head per key head, head size 256, no norm
    (6, 2, 192, 32, None, True, True),
    (8, 2, 64, 16, 40, True, True),         # a window over the cache and the token itself
    (8, 2, 128, 8, 1, True, True),          # a window of the token alone
])
def test_decode_attention_with_the_tokens_own_key_from_the_product(ops, nq, nkv, d, ps, window, norm, rope):
    """A step of single tokens in one kernel: queries and the token's key normalised and rotated
    inside the attention kernel, the token's key and value added from registers and stored into
    the cache. Against the plain norm-rotate-store followed by the plain attention: the output,
    the cache at the tokens' places, and the cache everywhere else (untouched). The tokens' places
    hold stale noise beforehand, which must not be read; contexts of 1 (no cached key at all) to
    2,100 keys (several key splits), ends of blocks of 32 and of pages."""
    kvs = [1, 2, 32, 33, 64, 65, 300, 2100, ps, ps + 1]
    seqs = [(1, kv) for kv in kvs]
    _, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, window=window, seed=3)
    t = len(seqs)
    qkv = rnd(t, (nq + 2 * nkv) * d, dtype=torch.bfloat16, seed=11)
    qw = 1 + 0.1 * rnd(d, seed=5) if norm else None
    kw = 1 + 0.1 * rnd(d, seed=6) if norm else None
    inv = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV) if rope else None
    table = cache.group.block_table.cpu()
    slots = torch.tensor([int(table[i, (kv - 1) // ps]) * ps + (kv - 1) % ps for i, kv in enumerate(kvs)],
                         dtype=torch.int32, device=DEV)
    cache.group.slots = slots
    scale = 1.0 / math.sqrt(d)
    want_k, want_v = cache.k.clone(), cache.v.clone()
    q = R.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, ctx.positions, want_k, want_v, slots, ps)
    want = R.paged_attention(q.to(torch.bfloat16), want_k, want_v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(),
                             cache.group.block_table, ps, nq, nkv, d, scale, window)
    before_k, before_v = cache.k.clone(), cache.v.clone()
    assert ops.fuses_decode_attention(ctx, qkv, nq, nkv, d, cache)
    got = ops.decode_attention(qkv, cache, ctx, nq, nkv, d, scale, window, qw, kw, 1e-6, inv)
    close(got, want, 2e-2, 2e-2)
    # the cache: the tokens' own places as the plain store leaves them, all else as before
    changed_k = (want_k != before_k)
    changed_v = (want_v != before_v)
    close(cache.k[changed_k], want_k[changed_k], 2e-2, 2e-2)
    close(cache.v[changed_v], want_v[changed_v], 0, 0)
    assert torch.equal(cache.k[~changed_k], before_k[~changed_k])
    assert torch.equal(cache.v[~changed_v], before_v[~changed_v])
    # with the keys cut over other numbers of blocks
    for splits in (1, 3, 16):
        cache.k.copy_(before_k)
        cache.v.copy_(before_v)
        ctx.scratch["attn_splits"] = splits
        close(ops.decode_attention(qkv, cache, ctx, nq, nkv, d, scale, window, qw, kw, 1e-6, inv), want, 2e-2, 2e-2)
    # ... and into pieces of one length, listed sequence by sequence (one block of keys each, so
    # that the longest has 66 and the shortest none but the token itself; three blocks; sixteen)
    del ctx.scratch["attn_splits"]
    for piece in (32, 96, 512):
        cache.k.copy_(before_k)
        cache.v.copy_(before_v)
        ctx.scratch["attn_piece"] = piece
        ctx.per_pass.clear()
        close(ops.decode_attention(qkv, cache, ctx, nq, nkv, d, scale, window, qw, kw, 1e-6, inv), want, 2e-2, 2e-2)
        assert torch.equal(cache.k[~changed_k], before_k[~changed_k]) and torch.equal(cache.v[~changed_v], before_v[~changed_v])


@pytest.mark.parametrize("nq,nkv,d,ps,window", [(32, 8, 128, 16, None), (8, 2, 64, 8, None), (8, 2, 64, 16, 40)])
def test_decode_attention_ignores_what_a_page_held_before(ops, nq, nkv, d, ps, window):
    """The one-kernel decode step with NaN and infinities in every place of the cache no sequence
    has written, the tokens' own places included (the kernel fills them; it must not read them)."""
    kvs = [1, 2, 9, 32, 33, 41, 64, 65, 300, 2100, ps, ps + 1]
    seqs = [(1, kv) for kv in kvs]
    _, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, window=window, seed=4, poison=True)
    t = len(seqs)
    qkv = rnd(t, (nq + 2 * nkv) * d, dtype=torch.bfloat16, seed=12)
    qw, kw = 1 + 0.1 * rnd(d, seed=5), 1 + 0.1 * rnd(d, seed=6)
    inv = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    table = cache.group.block_table.cpu()
    slots = torch.tensor([int(table[i, (kv - 1) // ps]) * ps + (kv - 1) % ps for i, kv in enumerate(kvs)],
                         dtype=torch.int32, device=DEV)
    cache.group.slots = slots
    pages, offs = (slots // ps).long(), (slots % ps).long()
    cache.k[pages, :, offs, :] = float("nan")
    cache.v[pages, :, :, offs] = float("inf")
    before_k, before_v = cache.k.clone(), cache.v.clone()
    scale = 1.0 / math.sqrt(d)
    want_k, want_v = cache.k.clone(), cache.v.clone()
    q = R.qk_norm_rope_store(qkv, nq, nkv, d, qw, kw, 1e-6, inv, ctx.positions, want_k, want_v, slots, ps)
    want = R.paged_attention(q.to(torch.bfloat16), want_k, want_v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(),
                             cache.group.block_table, ps, nq, nkv, d, scale, window)
    assert torch.isfinite(want.float()).all()
    for splits in (None, 1, 3):
        cache.k.copy_(before_k)
        cache.v.copy_(before_v)
        ctx.scratch.pop("attn_splits", None)
        if splits:
            ctx.scratch["attn_splits"] = splits
        close(ops.decode_attention(qkv, cache, ctx, nq, nkv, d, scale, window, qw, kw, 1e-6, inv), want, 2e-2, 2e-2)


@pytest.mark.parametrize("window,ps", [(40, 16), (33, 8), (None, 16)])
def test_decode_attention_at_the_windows_edge_and_the_tokens_own_key(ops, window, ps):
    """The one-kernel decode step with keys made to stand out: the key just outside the window
    (which would take all the weight if it were seen), the first key inside it, the last cached
    key and the token's own key (from the product, not from the cache), each with a value of its
    own, among faint others. A mask that is off by one at either end moves the output by a large
    part of a value, not by one part in ``window``. Contexts that end around blocks of 32 keys
    and around pages, the keys in one piece and cut over blocks."""
    nq, nkv, d = 8, 2, 64
    first = (window or 40) + 1
    kvs = [first, first + 1, 64, 65, 72, 73, 96, 97, 128, 129, 300, 1000]
    seqs = [(1, kv) for kv in kvs]
    _, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, window=window, seed=7)
    t = len(seqs)
    g = torch.Generator().manual_seed(3)
    u = torch.zeros(d)
    u[5] = 1.0
    cache.k.copy_((0.1 * torch.randn(cache.k.shape, generator=g)).to(torch.bfloat16))
    cache.v.copy_(torch.randn(cache.v.shape, generator=g).to(torch.bfloat16))
    table = cache.group.block_table.cpu()
    place = lambda s, pos: (int(table[s, pos // ps]), pos % ps)
    values = (3 * torch.randn(4, d, generator=g)).to(torch.bfloat16)
    for s, kv in enumerate(kvs):
        me = kv - 1
        marks = [(me - 1, 6.0, values[2])]                                  # the last cached key
        if window is not None:
            marks += [(me - window, 12.0, values[0]), (me - window + 1, 6.0, values[1])]   # outside, just inside
        for pos, strength, value in marks:
            page, off = place(s, pos)
            cache.k[page, :, off, :] = (strength * u).to(torch.bfloat16)
            cache.v[page, :, :, off] = value
    qkv = torch.zeros(t, (nq + 2 * nkv) * d)
    qkv[:, : nq * d] = (8.0 * u).repeat(nq)                                 # scores are then the strengths
    qkv[:, nq * d: (nq + nkv) * d] = (6.0 * u).repeat(nkv)                  # the token's own key
    qkv[:, (nq + nkv) * d:] = values[3].float().repeat(nkv)
    qkv = qkv.to(torch.bfloat16).to(DEV)
    slots = torch.tensor([place(s, kv - 1)[0] * ps + place(s, kv - 1)[1] for s, kv in enumerate(kvs)],
                         dtype=torch.int32, device=DEV)
    cache.group.slots = slots
    scale = 1.0 / math.sqrt(d)
    before_k, before_v = cache.k.clone(), cache.v.clone()

    def plain(win):
        k, v = before_k.clone(), before_v.clone()
        q = R.qk_norm_rope_store(qkv, nq, nkv, d, None, None, 0.0, None, ctx.positions, k, v, slots, ps)
        return R.paged_attention(q, k, v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table, ps, nq, nkv, d,
                                 scale, win).float()

    want = plain(window)
    if window is not None:  # what a mask off by one at the window's edge would give is far away
        assert float((plain(window + 1) - want).abs().max()) > 1.0 and float((plain(window - 1) - want).abs().max()) > 0.5
    assert ops.fuses_decode_attention(ctx, qkv, nq, nkv, d, cache)
    for splits in (None, 1, 2, 5):
        cache.k.copy_(before_k)
        cache.v.copy_(before_v)
        ctx.scratch.pop("attn_splits", None)
        if splits:
            ctx.scratch["attn_splits"] = splits
        close(ops.decode_attention(qkv, cache, ctx, nq, nkv, d, scale, window, None, None, 0.0, None), want, 3e-2, 2e-2)


def test_paged_attention_splits_agree(ops):
    """Long single sequences split over many blocks; empty splits must not leak."""
    seqs, nq, nkv, d, ps = [(1, 2100), (1, 40), (3, 900)], 8, 2, 64, 16
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 0.125)
    for splits in (1, 2, 7, 40):
        ctx.scratch["attn_splits"] = splits
        got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.125, None)
        close(got, want, 2e-2, 2e-2)


@pytest.mark.parametrize("seqs,nq,nkv,d,ps,window", [([(100, 1500), (30, 30)], 8, 2, 64, 16, None),
                                                     ([(300, 700)], 4, 1, 128, 8, None),
                                                     ([(90, 1200), (70, 75)], 6, 2, 32, 24, 200)])
def test_long_portions_split_over_blocks_agree(ops, seqs, nq, nkv, d, ps, window):
    """Portions of more than 64 rows (the kernel that shares keys through LDS) with the keys cut
    over 1 to 40 blocks: splits without a block of keys, a window, a page size that is no power
    of two."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, window=window)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 0.125, window)
    for splits in (1, 2, 3, 40):
        ctx.scratch["attn_splits"] = splits
        got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.125, window)
        close(got, want, 2e-2, 2e-2)


@pytest.mark.parametrize("groups", [1, 2])
@pytest.mark.parametrize("seqs,nq,nkv,d,ps,window,poison", [
    ([(300, 300)], 4, 1, 128, 16, None, True),                 # a whole prompt: the triangle
    ([(129, 129), (90, 1200), (70, 75)], 6, 2, 32, 24, None, True),
    ([(2048, 2048)], 32, 8, 128, 16, None, False),             # the measured prompt's own shape
    ([(200, 1000), (65, 65)], 8, 2, 64, 8, 150, True),         # a window: blocks of keys that begin late
    ([(100, 131)], 5, 1, 80, 40, None, True),                  # a 16-wide remainder of the head size
    ([(70, 70), (33, 140)], 4, 2, 16, 16, None, True),         # the smallest head size: the join needs more LDS than the stages
    ([(150, 150)], 3, 1, 48, 8, None, False),
    ([(260, 2000)], 2, 2, 208, 16, None, False),               # the largest head size whose stages fit
])
def test_long_portions_with_the_keys_cut_between_two_groups_of_waves(ops, groups, seqs, nq, nkv, d, ps, window, poison):
    """Portions of more than 64 rows in blocks of four waves, and in blocks of eight whose halves
    take the blocks of 32 keys in turn and join their sums at the end: odd and even numbers of
    key blocks, a group left without any, splits over blocks on top, unwritten places full of NaN."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, seed=5, window=window, poison=poison)
    scale = 1.0 / math.sqrt(d)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale, window)
    ops.prefill_key_groups = groups
    try:
        for splits in (None, 1, 2, 3, 40):
            ctx.scratch.clear()
            if splits:
                ctx.scratch["attn_splits"] = splits
            close(ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, window), want, 2e-2, 2e-2)
    finally:
        ops.prefill_key_groups = None


def test_which_long_portions_cut_their_keys_between_two_groups(ops):
    """The choice follows from the step's lengths alone: two groups where the longest tile's rounds
    reach what a compute unit gets on average, and never on top of a cut over blocks."""
    pick = lambda seqs, nq=32, nkv=8: ops.choose_key_groups([a for a, _ in seqs], [b for _, b in seqs], nq // nkv, nkv, 0)
    assert pick([(2048, 2048)]) == 2 and pick([(512, 512)]) == 2
    assert pick([(700, 700), (900, 1300), (448, 5000)]) == 2
    assert pick([(2048, 4096)]) == 1 and pick([(2048, 8192)]) == 1       # long histories: every tile is long
    assert pick([(1024, 1024)]) == 1                                      # few tiles: the keys are cut over blocks
    assert pick([(2048, 2048)], nq=64) == 1                               # twice the tiles for the same keys
    assert ops.choose_key_groups([2048], [2048], 4, 8, 0, forced_splits=3) == 1


@pytest.mark.parametrize("groups", [None, 2])
@pytest.mark.parametrize("seed", range(24))
def test_paged_attention_random_shapes(ops, seed, groups):
    """Seeded random mixes of decoded tokens, short and long portions, head counts, head sizes,
    page sizes, windows and key splits against the plain reference: every kernel variant and the
    edges between them (16, 64 rows; blocks of 32 keys; pages) get hit by some seed. Once with the
    kernels the lengths choose, once with long portions forced into blocks of eight waves."""
    import random

    rng = random.Random(1000 + seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3, 8])
    g = rng.choice([1, 2, 3, 4, 5, 8])
    nq = nkv * g
    ps = rng.choice([8, 16, 24, 32, 40, 64])
    kind = rng.choice(["decode", "short", "long", "mixed"])
    seqs = []
    for _ in range(rng.randint(1, 5)):
        k = kind if kind != "mixed" else rng.choice(["decode", "short", "long"])
        ql = {"decode": 1, "short": rng.randint(2, 20), "long": rng.randint(30, 260)}[k]
        seqs.append((ql, ql + rng.choice([0, 0, rng.randint(1, 40), rng.randint(100, 700)])))
    window = rng.choice([None, None, rng.randint(1, 300)])
    splits = rng.choice([None, None, rng.randint(2, 9)])
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, seed=seed, window=window)
    scale = 1.0 / math.sqrt(d)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale, window)
    if splits:
        ctx.scratch["attn_splits"] = splits
    ops.prefill_key_groups = groups
    try:
        got = ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, window)
    finally:
        ops.prefill_key_groups = None
    assert torch.isfinite(got.float()).all(), (seqs, nq, nkv, d, ps, window, splits)
    close(got, want, 2e-2, 2e-2)


MIXED_CASES = [
    # (seqs, nq, nkv, d, page, window): decoded tokens with a long context beside portions of prompts
    ([(1, 1500), (200, 200), (1, 40), (1, 2100)], 8, 2, 128, 16, None),
    ([(70, 900), (2, 1300), (1, 1), (3, 64)], 6, 2, 64, 24, None),
    ([(1, 1200), (1, 700), (33, 33), (17, 500)], 4, 1, 32, 8, 300),
    ([(16, 1100), (17, 1100)], 3, 3, 80, 16, None),   # one row count each side of the kernels' edge
]


@pytest.mark.parametrize("seqs,nq,nkv,d,ps,window", MIXED_CASES)
def test_mixed_steps_go_through_two_launches_and_agree(ops, seqs, nq, nkv, d, ps, window, monkeypatch):
    """A step with decoded tokens beside portions runs the decode kernel over the former and the
    prompt kernels over the latter. Each launch writes its own tokens only, with any number of key
    splits (the merge goes over the launch's tokens, not over all), and the result is the one
    launch's too."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, seed=11, window=window)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 0.125, window)
    launches = []
    inner = ops._launch_attention
    monkeypatch.setattr(ops, "_launch_attention", lambda *a: (launches.append(a[-2:]), inner(*a))[1])
    for min_kv, want_launches in ((1, 2), (1 << 30, 1)):
        monkeypatch.setattr(ops, "split_launch_min_kv", min_kv)
        for splits in (None, 1, 2, 5):
            ctx.scratch.clear()
            if splits:
                ctx.scratch["attn_splits"] = splits
            launches.clear()
            got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.125, window)
            assert len(launches) == want_launches, launches
            close(got, want, 2e-2, 2e-2)
    small = [s for s, (ql, _) in enumerate(seqs) if ql * (nq // nkv) <= 16]
    monkeypatch.setattr(ops, "split_launch_min_kv", 1)
    launches.clear()
    ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.125, window)
    assert launches[0] == (small, True) and launches[1][1] is False
    assert sorted(launches[0][0] + launches[1][0]) == list(range(len(seqs)))


def test_decode_attention_many_sequences_and_repeated_launches(ops):
    """Many sequences of very different lengths, launched again and again with other split counts."""
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(1, 1500, (37,), generator=g).tolist() + [1, 32, 33, 2048]
    seqs, nq, nkv, d, ps = [(1, n) for n in lens], 8, 2, 128, 16
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, seed=3)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 0.088)
    for splits in (5, 1, 16, 3, None):
        ctx.scratch.pop("attn_splits", None)
        if splits:
            ctx.scratch["attn_splits"] = splits
        got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 0.088, None)
        close(got, want, 2e-2, 2e-2)


@pytest.mark.parametrize("seqs,nq,nkv,d,ps,window", [
    ([(1, n) for n in (300, 5000, 1, 33, 2048, 700, 64, 4097)], 8, 2, 128, 16, None),
    ([(1, 300)] * 20 + [(1, 6000)] * 3, 32, 8, 128, 16, None),           # few long ones among many short
    ([(2, 1500), (4, 40), (1, 3000), (3, 3)], 4, 1, 64, 8, None),        # tiles of several tokens
    ([(1, 2500), (1, 90), (1, 700)], 6, 2, 32, 24, 200),                 # a window, pages of 24
    ([(1, 2100), (1, 20)], 2, 2, 256, 16, None),
])
def test_decode_attention_in_pieces_of_one_length(ops, seqs, nq, nkv, d, ps, window):
    """Sequences of very unequal lengths: the decode kernel walks a list of (sequence, piece), the
    pieces all of one length (the choice by the lengths, and lengths asked for outright: one
    block of 32 keys, so that the merge has up to 157 parts, and up to more than the longest
    sequence), unwritten places of the cache full of NaN. The list is made on the device from the
    step's lengths: also after the lengths have changed under the same context, as they do under
    a captured graph."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16, seed=8, window=window, poison=True)
    scale = 1.0 / math.sqrt(d)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale, window)
    kv_lens = [kv for _, kv in seqs]
    assert ops.decode_in_pieces(kv_lens) and ops.choose_decode_piece(kv_lens, nkv) % 32 == 0
    for piece in (None, 32, 512, 8192):
        ctx.scratch.pop("attn_piece", None)
        if piece:
            ctx.scratch["attn_piece"] = piece
        ctx.per_pass.clear()
        close(ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, window), want, 2e-2, 2e-2)
    # the same launch shapes over shorter sequences: every length cut to a third on the device only,
    # the host's view (what a captured launch was shaped for) unchanged
    ctx.scratch["attn_piece"] = 512
    short = [(q_len, max(q_len, kv // 3)) for q_len, kv in seqs]
    ctx.kv_lens.copy_(torch.tensor([kv for _, kv in short], dtype=torch.int32))
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, scale, window)
    ctx.per_pass.clear()
    close(ops.paged_attention(q, cache, ctx, nq, nkv, d, scale, window), want, 2e-2, 2e-2)


def test_which_decode_launches_go_in_pieces(ops):
    """Equal lengths keep equal parts; very unequal ones get pieces of at least 512 keys, at most 32
    for the longest sequence, about 1,536 blocks in all."""
    assert not ops.decode_in_pieces([2100] * 64) and not ops.decode_in_pieces([2048]) and not ops.decode_in_pieces([1900, 100])
    assert not ops.decode_in_pieces([2000, 3000, 2500, 2600])
    assert ops.decode_in_pieces([300] * 56 + [8000] * 8) and ops.decode_in_pieces([500, 16000])
    assert ops.choose_decode_piece([2100] * 64, 8) is None
    assert ops.choose_decode_piece([300] * 56 + [8000] * 8, 8) == 512
    assert ops.choose_decode_piece([500, 16000], 8) == 512
    assert ops.choose_decode_piece([1000, 30000] * 4, 8) == 960
    assert ops.choose_decode_piece(list(range(128, 4352, 33)), 8) == 1504


@pytest.mark.parametrize("seqs,nq,nkv,d,ps", [([(9, 50)], 3, 3, 80, 16), ([(2, 300), (1, 50)], 5, 1, 48, 8),
                                              ([(7, 90)], 2, 1, 112, 16), ([(40, 90)], 2, 1, 48, 16)])
def test_attention_repeats_bit_for_bit_at_head_sizes_with_a_16_wide_remainder(ops, seqs, nq, nkv, d, ps):
    """These head sizes once chained two MFMA shapes, whose results then differed from run to run."""
    q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, torch.bfloat16)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 1 / math.sqrt(d))
    first = ops.paged_attention(q, cache, ctx, nq, nkv, d, 1 / math.sqrt(d), None)
    close(first, want, 2e-2, 2e-2)
    for _ in range(100):
        assert torch.equal(ops.paged_attention(q, cache, ctx, nq, nkv, d, 1 / math.sqrt(d), None), first)


def test_attention_far_key_stands_out(ops):
    """One early key is made to dominate; the context must equal its value."""
    for dtype in (torch.float32, torch.bfloat16):
        seqs, nq, nkv, d, ps = [(1, 777)], 4, 2, 32, 16
        q, cache, ctx = build_attention_case(seqs, nq, nkv, d, ps, dtype)
        table = cache.group.block_table[0]
        far = 3
        page, off = int(table[far // ps]), far % ps
        cache.k[page, :, off, :] = 0
        cache.k[page, :, off, 0] = 40.0
        q[:] = 0
        q[:, ::d] = 40.0  # element 0 of every head
        got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 1.0, None)
        want = cache.v[page, :, :, off].repeat_interleave(nq // nkv, dim=0).reshape(1, -1)
        close(got, want, 1e-2, 1e-2)


@pytest.mark.parametrize("rise,jump_at", [(0.0, None), (5.0, None), (7.5, None), (3.0, 9), (0.5, 0)])
def test_prompt_attention_with_scores_that_climb(ops, rise, jump_at):
    """The prompt kernel takes its exponentials against a reference that follows a row's maximum
    only when a score rises above it by more than 2^8. Keys are made so that every block of 32
    lifts the maximum by ``rise`` (base-2 units of the scaled score: below the threshold, the
    reference stays behind and probabilities above one are summed), and one block by 30 (the
    reference must move and what was summed before must shrink). Values differ block by block,
    so a block weighed wrongly shows."""
    nq, nkv, d, ps, n = 8, 2, 128, 16, 640
    q, cache, ctx = build_attention_case([(n, n)], nq, nkv, d, ps, torch.bfloat16, seed=5, shuffle=True)
    table = cache.group.block_table[0].cpu()
    q[:] = 0
    q[:, ::d] = 1.0                                    # every head looks at element 0 of the keys
    ln2 = math.log(2.0)
    for pos in range(n):
        block = pos // 32
        level = rise * block + (30.0 if jump_at is not None and block >= jump_at else 0.0)
        page, off = int(table[pos // ps]), pos % ps
        cache.k[page, :, off, :] = 0
        cache.k[page, :, off, 0] = level * ln2 + 0.01 * (pos % 32)   # score = level (base 2), nearly flat inside a block
        cache.v[page, :, :, off] = float(block % 7) - 3.0 + 0.125 * (pos % 4)
    want = R.paged_attention(q, cache.k, cache.v, ctx.cu_q.cpu(), ctx.kv_lens.cpu(), cache.group.block_table,
                             ps, nq, nkv, d, 1.0)
    got = ops.paged_attention(q, cache, ctx, nq, nkv, d, 1.0, None)
    close(got, want, 2e-2, 2e-2)


def test_argmax_first_maximum(ops):
    x = torch.tensor([[1.0, 3.0, 3.0, 2.0], [0.0, 0.0, 0.0, 0.0], [3.0, -1.0, 2.5, 3.0]], device=DEV)
    assert ops.argmax(x).tolist() == [1, 0, 0]
    big = rnd(5, 151936)
    assert ops.argmax(big).tolist() == torch.argmax(big, dim=-1).tolist()
