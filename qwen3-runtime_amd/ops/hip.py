"""The engine's device ops: thin, checked wrappers over the HIP library.

Each method validates shapes, types and contiguity on the host (a kernel that
reads past a buffer can take the whole GPU down), then launches on torch's
current stream through ``ctypes``. There is no other implementation: if the
library cannot be built or loaded, construction fails. Tensors are torch
tensors on the GPU; outputs are allocated with torch's caching allocator.

Matrix products: float32 goes to the library's own fused-multiply-add kernel
(true 32-bit). bfloat16 with up to 64 rows (128 for the gated product and for
products cut along K) goes to the library's MFMA kernels, which stream the
weights; bfloat16 with more rows goes to the vendor BLAS through
``torch.matmul``, as the reference leaves its products to cuBLAS
(qwen3_runtime/models/qwen3.py:76-77,134-135).
"""

from __future__ import annotations

import ctypes
import math
from ctypes import POINTER, Structure, byref, c_float, c_int, c_long, c_void_p

import numpy as np
import torch

from . import build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class OpsError(RuntimeError):
    pass


class _QkArgs(Structure):
    _fields_ = [
        ("q_in", c_void_p), ("q_stride", c_long),
        ("k_in", c_void_p), ("k_stride", c_long),
        ("v_in", c_void_p), ("v_stride", c_long),
        ("q_weight", c_void_p), ("k_weight", c_void_p), ("inv_freq", c_void_p),
        ("positions", c_void_p), ("slots", c_void_p),
        ("q_out", c_void_p), ("k_out", c_void_p), ("v_out", c_void_p),
        ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("num_tokens", c_int), ("nq", c_int), ("nkv", c_int), ("nv", c_int),
        ("head_dim", c_int), ("page_size", c_int), ("eps", c_float), ("rope", c_void_p),
    ]


class _AttnArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("out", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("positions", c_void_p), ("seq_of_token", c_void_p), ("block_table", c_void_p),
        ("table_width", c_int), ("num_tokens", c_int), ("nq", c_int), ("nkv", c_int),
        ("head_dim", c_int), ("page_size", c_int), ("window", c_int), ("scale", c_float),
    ]


class _AttnTileArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("out", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("cu_q", c_void_p), ("kv_lens", c_void_p), ("block_table", c_void_p),
        ("tile_seq", c_void_p), ("tile_row0", c_void_p), ("part_o", c_void_p), ("part_lse", c_void_p),
        ("table_width", c_int), ("num_tiles", c_int), ("nq", c_int), ("nkv", c_int),
        ("page_size", c_int), ("window", c_int), ("num_splits", c_int), ("waves", c_int),
        ("scale_log2", c_float), ("row_tiles", c_int), ("use_lds", c_int),
        ("merge_tokens", c_void_p), ("num_merge_tokens", c_int),
        ("qkv", c_void_p), ("qkv_stride", c_long), ("q_weight", c_void_p), ("k_weight", c_void_p),
        ("rope", c_void_p), ("slots", c_void_p), ("eps", c_float), ("split_blocks", c_int),
        ("max_items", c_int), ("items", c_void_p),
    ]


class _SampleArgs(Structure):
    _fields_ = [
        ("logits", c_void_p), ("work", c_void_p), ("counts", c_void_p), ("slot", c_void_p),
        ("fparams", c_void_p), ("iparams", c_void_p), ("seeds", c_void_p),
        ("out_token", c_void_p), ("out_logprob", c_void_p), ("rows", c_int), ("vocab", c_int),
        ("write_work", c_int), ("partials", c_void_p), ("parts", c_int),
    ]


def _load(name: str) -> ctypes.CDLL:
    path = build.build_library(name)
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:
        raise OpsError(f"cannot load {path}: {exc}") from exc
    if hasattr(lib, "qrt_last_error"):  # a library from outside need not link runtime.hip
        lib.qrt_last_error.restype = ctypes.c_char_p
    return lib


_core: ctypes.CDLL | None = None
_attn: dict[int, ctypes.CDLL] = {}


def core_library() -> ctypes.CDLL:
    global _core
    if _core is None:
        _core = _load("core")
    return _core


def attention_library(head_dim: int) -> ctypes.CDLL:
    if head_dim not in _attn:
        _attn[head_dim] = _load(f"attn_bf16_d{head_dim}")
    return _attn[head_dim]


_extra: dict[str, ctypes.CDLL] = {}


def load_library(name: str) -> ctypes.CDLL:
    """A library registered with ``ops.build.register_library``, built if need be, as a
    ``ctypes.CDLL``; its entry points take raw device pointers and ``current_stream()``."""
    if name not in _extra:
        _extra[name] = _load(name)
    return _extra[name]


def _ptr(t: torch.Tensor | None):
    return None if t is None else c_void_p(t.data_ptr())


def _addr(t: torch.Tensor | None):
    """Address for a structure field (ctypes takes an int or None there)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> c_void_p:
    """torch's current stream on the current device. The two calls behind the public
    ``torch.cuda.current_stream()`` are used directly where this torch has them: the public one
    builds a Stream object and cost 9 us a launch, a quarter of a short prompt step's host time."""
    if _raw_stream is not None and _raw_device is not None:
        return c_void_p(_raw_stream(_raw_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


current_stream = _stream


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> torch.Tensor:
    if not t.is_cuda:
        raise OpsError(f"{name} must be on the GPU, it is on {t.device}")
    if not t.is_contiguous():
        raise OpsError(f"{name} must be contiguous, strides are {t.stride()} for shape {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise OpsError(f"{name} must be {dtype}, it is {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise OpsError(f"{name} must have shape {tuple(shape)}, it has {tuple(t.shape)}")
    return t


check_tensor = _need  # for parts that call a library of their own


class HipOps:
    # bfloat16 products with more rows than this go to the vendor BLAS
    own_max_rows = 64
    # the same for the two forms in which a block fetches fewer activations than weights: the
    # gated product, and the product cut along K whose planes the residual's norm adds
    own_max_rows_shared = 128
    # Rows from which a product takes the kernel that shares the activations through LDS
    # instead of the few-row kernel (both stream the weights as stored, through LDS by direct
    # loads). Measured at the 4B shapes on the matrices of 36 layers in turn: cut along K the
    # sharing kernel is faster from 9 rows on, gated from 12 rows on. (Timed on one weight
    # matrix over and over, the sharing kernel looks 15 to 40 % faster than the few-row kernel
    # down to one row, because a matrix of up to some 100 MB then stays in the memory-side
    # cache; in a step it is 5 % slower at 8 rows, and a decode step with it from one row on
    # lost 3 % at batch 8 and 9 % at batch 1.)
    shared_from_rows = {"whole": 17, "gated": 12, "planes": 9}
    # steps of single tokens: norm, rotation, cache write and attention in one kernel
    fuse_decode = True
    # tiles of 16 rows per wave in the attention kernel for long portions (1 or 2)
    prefill_row_tiles = 2
    # long portions: keys and values go through LDS, shared by the four waves of a block
    prefill_through_lds = True
    # ... in blocks of eight waves, two groups that take the blocks of keys in turn: 1 never, 2 always,
    # None where the longest tile's chain of rounds would otherwise set the kernel's time
    prefill_key_groups = None

    def __init__(self):
        self.lib = core_library()

    def _check(self, lib, code: int) -> None:
        if code != 0:
            raise OpsError(lib.qrt_last_error().decode())

    # ---- embedding, norms, activations ---------------------------------------
    def embed(self, ids, table):
        _need(ids, "ids", torch.int32)
        _need(table, "embedding table")
        t, (v, h) = ids.numel(), table.shape
        out = torch.empty((t, h), dtype=torch.float32, device=table.device)
        self._check(self.lib, self.lib.qrt_embed(_ptr(ids), _ptr(table), _CODE[table.dtype], _ptr(out),
                                                 c_int(t), c_int(v), c_int(h), _stream()))
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None):
        t, h = residual.shape
        _need(residual, "residual", torch.float32)
        _need(weight, "norm weight", torch.float32, (h,))
        planes, plane_stride = 1, 0
        if delta is not None:
            if delta.dim() == 3:  # the parts of a product whose K was cut: added here, in order
                planes, plane_stride = delta.shape[0], t * h
                _need(delta, "delta", shape=(planes, t, h))
            else:
                _need(delta, "delta", shape=(t, h))
        n_out = t
        if rows is not None:
            _need(rows, "rows", torch.int32)
            n_out = rows.numel()
        out = torch.empty((n_out, h), dtype=out_dtype, device=residual.device)
        self._check(self.lib, self.lib.qrt_add_rmsnorm(
            _ptr(residual), _ptr(delta), _CODE[delta.dtype] if delta is not None else F32, _ptr(weight),
            _ptr(rows), _ptr(out), _CODE[out_dtype], c_int(n_out), c_int(h), c_float(eps), c_int(planes),
            c_long(plane_stride), _stream()))
        return out

    def swiglu(self, gate_up):
        _need(gate_up, "gate_up")
        t, two_i = gate_up.shape
        if two_i % 2:
            raise OpsError(f"gate_up has odd width {two_i}")
        out = torch.empty((t, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
        self._check(self.lib, self.lib.qrt_swiglu(_ptr(gate_up), _ptr(out), _CODE[gate_up.dtype],
                                                  c_int(t), c_int(two_i // 2), _stream()))
        return out

    # ---- matrix products -------------------------------------------------------
    def linear(self, x, w, out_f32=False):
        _need(x, "x")
        _need(w, "weight")
        m, k = x.shape
        n, kw = w.shape
        if k != kw:
            raise OpsError(f"linear: x is {tuple(x.shape)}, weight is {tuple(w.shape)}")
        if w.dtype == torch.float32:
            # true 32-bit product; a float32 weight met by bfloat16 activations keeps its precision
            xin = x if x.dtype == torch.float32 else x.float()
            out = torch.empty((m, n), dtype=torch.float32, device=x.device)
            self._check(self.lib, self.lib.qrt_gemm_f32(_ptr(xin), _ptr(w), _ptr(out), c_int(m), c_int(n),
                                                        c_int(k), _stream()))
            return out if (out_f32 or x.dtype == torch.float32) else out.to(x.dtype)
        if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
            raise OpsError(f"linear: no product of {x.dtype} activations with {w.dtype} weights")
        kernel = self._own_kernel(m, n, k, "whole")
        if kernel is None:
            # many rows: the vendor library; both accumulate in float32
            if out_f32:
                return torch.mm(x, w.t(), out_dtype=torch.float32)
            return self._library_product(x, w)
        out = torch.empty((m, n), dtype=torch.float32 if out_f32 else torch.bfloat16, device=x.device)
        self._check(self.lib, self.lib.qrt_gemm_bf16(
            _ptr(x), _ptr(w), _ptr(out), F32 if out_f32 else BF16,
            c_int(m), c_int(n), c_int(k), c_int(0), c_int(kernel), c_int(1), _stream()))
        return out

    # rows from which a library product is made in two column chunks; False: never
    library_split_min_rows = 256

    def _library_product(self, x, w):
        """``x @ w.T`` by the vendor library, in one call or in two over column chunks of the result.

        The library's kernels work on tiles of the result (256 x 256 for these shapes), and a
        result whose tiles do not fill the 256 compute units a whole number of times leaves
        them idle in the last round: 2,048 x 19,456 is 608 tiles, 2.4 rounds (0.93 PFLOP/s, where
        2,048 x 24,576, three whole rounds, runs at 1.45). A first chunk of columns that fills
        whole rounds and a second call for the rest is faster wherever such a cut exists: over the
        products of the 1.7B to 32B sizes at 256 to 8,192 rows the two calls took 0.69 to 0.99 of
        the one call's time (0.80 for the case above), 1.02 at worst. The cut depends on the
        shape alone, so equal inputs give equal bits in every process (the two ways use other
        library kernels, which round differently)."""
        m, k = x.shape
        n = w.shape[0]
        split = self.library_split(m, n)
        if not split:
            return torch.matmul(x, w.t())
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
        torch.mm(x, w[:split].t(), out=out[:, :split])
        torch.mm(x, w[split:].t(), out=out[:, split:])
        return out

    def library_split(self, m: int, n: int) -> int:
        """Columns of the first chunk (0: one call): the most whose 256 x 256 tiles fill the
        compute units a whole number of times, if that leaves a second chunk."""
        if not self.library_split_min_rows or m < self.library_split_min_rows:
            return 0
        row_tiles = -(-m // 256)
        per_round = 256 * max(1, 256 // row_tiles)  # columns whose tiles fill the compute units once
        split = (n // per_round) * per_round
        return split if 0 < split < n else 0

    def _own_kernel(self, m: int, n: int, k: int, form: str) -> int | None:
        """Which of the library's kernels multiplies ``m`` rows by a weight [n, k]: 0 the few-row
        kernel (up to 16 rows), 1 the kernel that shares the activations through LDS (K a
        multiple of 64 and at least 128, n a multiple of 16), None the vendor library. Both read
        the weight as stored. ``form``: "whole", "gated", or "planes" (cut along K). Measured at
        the 4B shapes against the vendor library: 28 to 32 % less time over the four products of
        a layer at 32 and 64 rows; at 128 rows 71 us against 116 for the gated product and the
        two cut along K."""
        limit = self.own_max_rows if form == "whole" else self.own_max_rows_shared
        if (k % 64 == 0 and k >= 128 and n % 16 == 0 and n <= 1 << 20
                and self.shared_from_rows[form] <= m <= limit):
            return 1
        if m <= min(16, limit):
            return 0
        return None

    def linear_for_residual(self, x, w):
        """``linear(x, w)`` for a result that is only ever added to the residual stream.

        May return the result in planes ``[P, T, N]`` float32 whose sum it is (``add_rmsnorm``
        adds them): a product with few rows and few weight rows then cuts K over several blocks
        per row tile, which fills the chip (160 row tiles for 256 compute units at the 4B size)."""
        m, k = x.shape
        n = w.shape[0]
        kernel, parts = None, 1
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and k % 64 == 0:
            kernel = self._own_kernel(m, n, k, "planes")
            if kernel is not None:
                parts = self.choose_k_parts(n, k, m, kernel == 1)
        if parts == 1:
            return self.linear(x, w)
        _need(x, "x", torch.bfloat16)
        _need(w, "weight", torch.bfloat16, (n, k))
        out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
        self._check(self.lib, self.lib.qrt_gemm_bf16(
            _ptr(x), _ptr(w), _ptr(out), F32, c_int(m), c_int(n), c_int(k), c_int(0),
            c_int(kernel), c_int(parts), _stream()))
        return out

    @staticmethod
    def choose_k_parts(n: int, k: int, m: int = 1, shared: bool | None = None) -> int:
        """The few-row kernel: cut K when there are fewer row tiles than about two per compute
        unit and K is long. The kernel that shares activations (``shared``; by default from 17
        rows on): a block takes up to eight row tiles, and K is cut until there are about as
        many blocks as compute units, each part keeping 12 k-steps or more."""
        tiles = n // 16
        if shared is None:
            shared = m > 16
        if not shared:
            if tiles >= 384 or k < 2048:
                return 1
            # four parts up to 8,192 columns and eight beyond, in a number of planes the residual's
            # norm knows when compiling (timed on the matrices of 36 layers in turn at the 4B, 8B
            # and 32B sizes: the attention's output product 6.2, 7.6 and 17.6 us in four parts
            # against 6.8, 8.9 and 18.3 in eight; the down projection 10.6 and 40.6 us in eight
            # against 12.0 and 43.6 in four at the 4B and 32B sizes, level at the 8B size)
            return 4 if k <= 8192 else 8
        blocks = (tiles + 7) // 8
        return max(1, min(8, 256 // blocks, (k // 32) // 12))


    def gated_linear(self, x, w_gate_up):
        """``swiglu(linear(x, w_gate_up))`` with ``w_gate_up`` [2I, K], gate rows first. With few
        rows in bfloat16 one kernel forms both halves and applies the activation in its epilogue,
        so the [T, 2I] intermediate never reaches memory."""
        m, k = x.shape
        two_i, kw = w_gate_up.shape
        if k != kw or two_i % 2:
            raise OpsError(f"gated_linear: x is {tuple(x.shape)}, weight is {tuple(w_gate_up.shape)}")
        if x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and k % 32 == 0:
            _need(x, "x")
            _need(w_gate_up, "weight")
            kernel = self._own_kernel(m, two_i // 2, k, "gated")
            if kernel is not None:
                out = torch.empty((m, two_i // 2), dtype=torch.bfloat16, device=x.device)
                self._check(self.lib, self.lib.qrt_gemm_bf16(
                    _ptr(x), _ptr(w_gate_up), _ptr(out), BF16, c_int(m),
                    c_int(two_i // 2), c_int(k), c_int(1), c_int(kernel), c_int(1), _stream()))
                return out
        return self.swiglu(self.linear(x, w_gate_up))

    # ---- q/k norm, rotation, cache write ----------------------------------------
    def _qk(self, args: _QkArgs, dtype, num_pages=0):
        self._check(self.lib, self.lib.qrt_qk_norm_rope_store(byref(args), _CODE[dtype], c_long(num_pages), _stream()))

    # tokens from which the step's cosines and sines are computed once (rope_table) and looked up by
    # every layer, instead of being computed in every layer's kernel
    rope_table_from_tokens = 256

    def qk_norm_rope_store(self, qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions, cache, ctx=None,
                           angles_key=None):
        """Per-head RMSNorm of queries and keys, NeoX rotation, and the write of keys and values into
        the cache, in one pass over ``qkv``; returns the queries. With the step's context given,
        the angles of a long step come from ``rope_table`` (``angles_key`` as there)."""
        t, width = qkv.shape
        _need(qkv, "qkv", shape=(t, (nq + 2 * nkv) * d))
        for name, w in (("q_norm", q_w), ("k_norm", k_w)):
            if w is not None:
                _need(w, name, torch.float32, (d,))
        if inv_freq is not None:
            _need(inv_freq, "inv_freq", torch.float32, (d // 2,))
            _need(positions, "positions", torch.int32, (t,))
        q = torch.empty((t, nq * d), dtype=qkv.dtype, device=qkv.device)
        es = qkv.element_size()
        a = _QkArgs()
        a.q_in, a.q_stride = qkv.data_ptr(), width
        a.k_in, a.k_stride = qkv.data_ptr() + nq * d * es, width
        a.v_in, a.v_stride = qkv.data_ptr() + (nq + nkv) * d * es, width
        a.q_weight, a.k_weight, a.inv_freq = _addr(q_w), _addr(k_w), _addr(inv_freq)
        a.positions = _addr(positions) if inv_freq is not None else None
        if inv_freq is not None and ctx is not None and t >= self.rope_table_from_tokens and t == ctx.num_tokens \
                and positions is ctx.positions:
            a.rope = self.rope_table(ctx, inv_freq, angles_key).data_ptr()
        a.q_out = q.data_ptr()
        a.num_tokens, a.nq, a.nkv, a.nv, a.head_dim, a.eps = t, nq, nkv, nkv, d, eps
        pages = 0
        if cache is not None:
            pages = self._check_cache(cache, nkv, d, qkv.dtype)
            _need(cache.group.slots, "slots", torch.int32, (t,))
            a.slots, a.k_cache, a.v_cache = _addr(cache.group.slots), _addr(cache.k), _addr(cache.v)
            a.page_size = cache.group.page_size
        else:
            a.nkv = a.nv = 0  # keys and values go nowhere: only queries are needed
        self._qk(a, qkv.dtype, pages)
        return q

    def qk_norm_split(self, qkv, nq, nkv, d, q_w, k_w, eps):
        t, width = qkv.shape
        _need(qkv, "qkv", shape=(t, (nq + 2 * nkv) * d))
        q = torch.empty((t, nq, d), dtype=qkv.dtype, device=qkv.device)
        k = torch.empty((t, nkv, d), dtype=qkv.dtype, device=qkv.device)
        v = torch.empty((t, nkv, d), dtype=qkv.dtype, device=qkv.device)
        es = qkv.element_size()
        a = _QkArgs()
        a.q_in, a.q_stride = qkv.data_ptr(), width
        a.k_in, a.k_stride = qkv.data_ptr() + nq * d * es, width
        a.v_in, a.v_stride = qkv.data_ptr() + (nq + nkv) * d * es, width
        a.q_weight, a.k_weight = _addr(q_w), _addr(k_w)
        a.q_out, a.k_out, a.v_out = q.data_ptr(), k.data_ptr(), v.data_ptr()
        a.num_tokens, a.nq, a.nkv, a.nv, a.head_dim, a.eps = t, nq, nkv, nkv, d, eps
        self._qk(a, qkv.dtype)
        return q, k, v

    def rope_neox(self, q, k, positions, inv_freq):
        t, nq, d = q.shape
        nkv = k.shape[1]
        _need(q, "q")
        _need(k, "k", q.dtype, (t, nkv, d))
        _need(inv_freq, "inv_freq", torch.float32, (d // 2,))
        _need(positions, "positions", torch.int32, (t,))
        q_out, k_out = torch.empty_like(q), torch.empty_like(k)
        a = _QkArgs()
        a.q_in, a.q_stride = q.data_ptr(), nq * d
        a.k_in, a.k_stride = k.data_ptr(), nkv * d
        a.inv_freq, a.positions = _addr(inv_freq), _addr(positions)
        a.q_out, a.k_out = q_out.data_ptr(), k_out.data_ptr()
        a.num_tokens, a.nq, a.nkv, a.nv, a.head_dim = t, nq, nkv, 0, d
        self._qk(a, q.dtype)
        return q_out, k_out

    def kv_store(self, k, v, cache):
        t, nkv, d = k.shape
        _need(k, "k")
        _need(v, "v", k.dtype, (t, nkv, d))
        pages = self._check_cache(cache, nkv, d, k.dtype)
        _need(cache.group.slots, "slots", torch.int32, (t,))
        a = _QkArgs()
        a.k_in, a.k_stride = k.data_ptr(), nkv * d
        a.v_in, a.v_stride = v.data_ptr(), nkv * d
        a.slots, a.k_cache, a.v_cache = _addr(cache.group.slots), _addr(cache.k), _addr(cache.v)
        a.num_tokens, a.nq, a.nkv, a.nv, a.head_dim = t, 0, nkv, nkv, d
        a.page_size = cache.group.page_size
        self._qk(a, k.dtype, pages)

    @staticmethod
    def _check_cache(cache, nkv, d, dtype) -> int:
        ps = cache.group.page_size
        pages = cache.k.shape[0]
        _need(cache.k, "key cache", dtype, (pages, nkv, ps, d))
        _need(cache.v, "value cache", dtype, (pages, nkv, d, ps))
        return pages

    # ---- attention ---------------------------------------------------------------
    # ---- decoding: norm, rotation, cache write and attention in one kernel -------------
    def rope_table(self, ctx, inv_freq, angles_key=None):
        """Cosines and sines of the step's rotation angles, float32 [T, 2 * len(inv_freq)]
        (cosines first): computed once per pass and looked up by every layer that rotates inside
        its attention kernel. ``angles_key`` names the angles (layers with equal keys share the
        table); without it the tensor ``inv_freq`` itself does."""
        key = ("rope_table", angles_key if angles_key is not None else inv_freq.data_ptr())
        table = ctx.per_pass.get(key)
        if table is None:
            half = inv_freq.numel()
            _need(inv_freq, "inv_freq", torch.float32, (half,))
            _need(ctx.positions, "positions", torch.int32, (ctx.num_tokens,))
            table = torch.empty((ctx.num_tokens, 2 * half), dtype=torch.float32, device=inv_freq.device)
            self._check(self.lib, self.lib.qrt_rope_table(_ptr(ctx.positions), _ptr(inv_freq), _ptr(table),
                                                          c_int(ctx.num_tokens), c_int(half), _stream()))
            ctx.per_pass[key] = table
        return table

    def fuses_decode_attention(self, ctx, qkv, nq, nkv, d, cache) -> bool:
        """Whether ``decode_attention`` serves this step: one token per sequence, bfloat16, a head
        size that keeps a rotation pair in one lane (a multiple of 64, up to 256), at most 16
        query heads per key head, and a layer that writes its own cache."""
        return (self.fuse_decode and qkv.dtype == torch.bfloat16 and ctx.max_q_len == 1
                and ctx.num_tokens == ctx.num_seqs and d % 64 == 0 and d <= 256 and nq // nkv <= 16
                and cache is not None and cache.writes and cache.group.page_size % 8 == 0
                and cache.k.dtype == torch.bfloat16)

    def decode_attention(self, qkv, cache, ctx, nq, nkv, d, scale, window, q_w, k_w, eps, inv_freq,
                         angles_key=None):
        """``paged_attention(qk_norm_rope_store(qkv, ...))`` for a step of single tokens, in one
        kernel: each block forms its queries from ``qkv`` (RMSNorm per head, NeoX rotation by the
        step's angle table), attends over the cached keys before the token, adds the token's own
        key and value from registers and stores them into the cache for later steps. Saves the
        kernel between the product and the attention, and the round trip of the queries."""
        t, width = qkv.shape
        _need(qkv, "qkv", torch.bfloat16, (t, (nq + 2 * nkv) * d))
        self._check_cache(cache, nkv, d, qkv.dtype)
        for name, w in (("q_norm", q_w), ("k_norm", k_w)):
            if w is not None:
                _need(w, name, torch.float32, (d,))
        _need(cache.group.slots, "slots", torch.int32, (t,))
        table = _need(cache.group.block_table, "block table", torch.int32)
        if table.shape[0] != ctx.num_seqs:
            raise OpsError(f"block table has {table.shape[0]} rows for {ctx.num_seqs} sequences")
        ps = cache.group.page_size
        if table.shape[1] < (ctx.max_kv_len + ps - 1) // ps:
            raise OpsError(f"block table is {table.shape[1]} pages wide, the longest sequence needs more")
        if not scale > 0:
            raise OpsError(f"the bfloat16 attention kernels take a positive score scale, not {scale}")
        own = {"qkv": qkv, "q_weight": q_w, "k_weight": k_w, "eps": eps,
               "rope": None if inv_freq is None else self.rope_table(ctx, inv_freq, angles_key)}
        out = torch.empty((t, nq * d), dtype=qkv.dtype, device=qkv.device)
        self._launch_attention(None, out, cache, ctx, nq, nkv, d, scale, window or 0, None, True, own)
        return out

    def paged_attention(self, q, cache, ctx, nq, nkv, d, scale, window):
        t = ctx.num_tokens
        _need(q, "q", shape=(t, nq * d))
        self._check_cache(cache, nkv, d, q.dtype)
        table = _need(cache.group.block_table, "block table", torch.int32)
        if table.shape[0] != ctx.num_seqs:
            raise OpsError(f"block table has {table.shape[0]} rows for {ctx.num_seqs} sequences")
        ps = cache.group.page_size
        need_pages = (ctx.max_kv_len + ps - 1) // ps
        if table.shape[1] < need_pages:
            raise OpsError(f"block table is {table.shape[1]} pages wide, the longest sequence needs {need_pages}")
        out = torch.empty_like(q)
        if q.dtype == torch.bfloat16 and d % 16 == 0 and ps % 8 == 0:
            self._attention_mfma(q, out, cache, ctx, nq, nkv, d, scale, window or 0)
        else:
            a = _AttnArgs()
            a.q, a.out, a.k_cache, a.v_cache = q.data_ptr(), out.data_ptr(), cache.k.data_ptr(), cache.v.data_ptr()
            a.positions = _need(ctx.positions, "positions", torch.int32, (t,)).data_ptr()
            a.seq_of_token = _need(ctx.seq_of_token, "seq_of_token", torch.int32, (t,)).data_ptr()
            a.block_table, a.table_width = table.data_ptr(), table.shape[1]
            a.num_tokens, a.nq, a.nkv, a.head_dim, a.page_size = t, nq, nkv, d, ps
            a.window, a.scale = window or 0, scale
            self._check(self.lib, self.lib.qrt_attention_f32(byref(a), _CODE[q.dtype], _stream()))
        return out

    resident_blocks = 512  # blocks of the prompt kernels the chip holds at once: 2 on each of 256 CUs

    @staticmethod
    def plan_tiles(q_lens, kv_lens, group_size: int, rows_per_tile: int, nkv: int = 1, resident: int = 0,
                   seq_ids=None):
        """Work list of the MFMA attention kernels: (sequence, first row) per tile of rows.

        Tiles that see the most keys come first: blocks that start late are then the short ones,
        and the chip stays full until the end although causal tiles differ in length. When all
        blocks (tiles x ``nkv`` key heads) fit on the chip at once (``resident``), nothing starts
        late: each CU then holds block i and block i + resident / 2 of the launch order from start
        to end, so the second half of the list is turned round and long tiles share a CU with
        short ones."""
        items = []
        for i, (n, kv) in enumerate(zip(q_lens, kv_lens)):
            s = i if seq_ids is None else seq_ids[i]  # the lists may cover some of the step's sequences
            first = kv - n
            for r in range(0, n * group_size, rows_per_tile):
                last_tok = min(n * group_size, r + rows_per_tile) - 1
                items.append((-(first + last_tok // group_size), s, r))
        items.sort()
        half = resident // (2 * max(nkv, 1))
        if resident and half < len(items) <= 2 * half:
            items = items[:half] + items[half:][::-1]
        seqs = [s for _, s, _ in items]
        row0 = [r for _, _, r in items]
        return np.asarray(seqs + row0, dtype=np.int32), len(seqs)

    def choose_key_groups(self, q_lens, kv_lens, group_size: int, nkv: int, window: int, forced_splits=None) -> int:
        """Long portions through LDS: blocks of four waves, two to a compute unit (1), or blocks of
        eight waves whose two halves take the blocks of keys in turn (2). A tile of 128 rows walks
        its keys in rounds of 32, one after the other, and a lone block's round takes 0.78 of what
        it takes beside a second block: where the tile with the most rounds has about as many as a
        compute unit gets from all tiles together, that chain sets the kernel's time, and halving
        it pays although the eight waves, which meet at one barrier, walk a round more slowly than
        two blocks of four. Measured at head size 128 with 32 query heads on 8 key heads (two
        groups against one): a 2,048-token prompt 63 against 69 us; prompts of 1,024 tokens with
        0 and 1,976 tokens before them 83 against 98; portions of 700, 900 and 448 tokens with
        0, 400 and 4,552 before them 104 against 145; 2,048 tokens with 1,024 before them level;
        with 2,048 before them 148 against 142. Where the keys are cut over blocks anyway (few
        tiles), they are not cut again."""
        if self.prefill_key_groups is not None:
            return self.prefill_key_groups
        rounds = longest = tiles = 0
        for n, kv in zip(q_lens, kv_lens):
            first = kv - n
            for r in range(0, n * group_size, 128):
                hi = first + (min(n * group_size, r + 128) - 1) // group_size
                lo = max(0, first + r // group_size - window + 1) if window else 0
                t = (hi >> 5) - (lo >> 5) + 1
                rounds += t
                longest = max(longest, t)
                tiles += 1
        splits = forced_splits or self.choose_splits(tiles, nkv, max(kv_lens))
        if splits > 1:
            return 1
        return 2 if longest > self.key_groups_ratio * rounds * nkv / 256 else 1

    # see choose_key_groups: the longest tile's rounds over the mean rounds of a compute unit
    key_groups_ratio = 0.9

    @staticmethod
    def choose_splits(num_tiles: int, nkv: int, max_kv: int) -> int:
        """Portions: how many ways to split the keys so that few long sequences still fill the chip."""
        work = num_tiles * nkv
        if max_kv <= 512 or work >= 512:
            return 1
        return max(1, min((max_kv + 255) // 256, (1024 + work - 1) // work, 64))

    @staticmethod
    def choose_decode_splits(num_tiles: int, nkv: int, max_kv: int) -> int:
        """Decoding: blocks of four waves, two to a compute unit. The parts are chosen by a small
        model of the launch's time that the measurements fit: the busiest compute unit gets
        ceil(blocks / 256) blocks, each a part of a sequence's keys plus a fixed cost (some 2.5 us:
        0.06 of a walk over 2,100 keys), so the time goes as ceil(work * parts / 256) *
        (1 / parts + cost). Counts of blocks that leave some units one block more than others are
        what it avoids: 12 sequences of 2,100 keys on 8 key heads 32 us in 3 parts (288 blocks), 27
        in 2; 24 sequences 49 us in 2 parts, 42 in 4; 40 sequences 78 us in 1 part, 65 in 4. At
        least 8 key blocks of 32 a part (4 each measured 2 % slower over a batch-1 decode step at
        2,048 keys), at most 64 parts (what the merge kernel reads with every load in flight)."""
        work = num_tiles * nkv
        blocks = (max_kv + 31) // 32
        cost = 0.06 * 2100 / max(max_kv, 1)
        best, best_time = 1, None
        for parts in range(1, max(1, min(blocks // 8, 64)) + 1):
            time = -(-work * parts // 256) * (1.0 / parts + cost)
            if best_time is None or time < best_time * 0.999:
                best, best_time = parts, time
        return best

    # decoding over unequal lengths: from this ratio of the longest to the mean length on, pieces
    decode_piece_ratio = 1.35

    def decode_in_pieces(self, kv_lens) -> bool:
        """Whether a decode launch over sequences of these lengths cuts their keys into pieces
        of one length (as many per sequence as it has) instead of every sequence into equally
        many parts. Measured on 8 to 128 sequences with lengths drawn evenly around 1,024 to
        8,192: the pieces win from a longest length of 1.3 to 1.4 times the mean on (0.80 to 0.9
        of the time at 1.6 to 1.9), lose 5 to 12 % below it, and lose at any spread while the
        longest context is under some 2,000 keys (the merge of the parts then weighs too much)."""
        n, total = len(kv_lens), sum(kv_lens)
        return n >= 2 and max(kv_lens) * n > self.decode_piece_ratio * total and max(kv_lens) >= 2048

    def choose_decode_piece(self, kv_lens, nkv: int):
        """Keys per piece for such a launch (a multiple of 32), or None. Equal parts of every
        sequence make blocks whose work is the sequence's length: with 56 sequences of 300 keys
        and 8 of 8,000 the launch takes 231 us where the two kinds alone take 18 and 48, and more
        parts do not help, because the blocks reach the compute units in launch order, round
        robin, and heavy blocks a fixed stride apart land on the same few. Pieces of one length,
        whole ones first in the list: about 1,536 blocks in all, no piece under 512 keys (a block
        costs some 8 us before its first key arrives) and no sequence in more than 32 (the merge
        reads every piece's part, up to 64 with all its loads in flight at once: 8 sequences of
        1,000 to 30,000 keys 91 us in pieces of 1,024, 96 in pieces of 512, 126 in pieces of 4,096)."""
        if not self.decode_in_pieces(kv_lens):
            return None
        piece = max(512, -(-sum(kv_lens) * nkv // 1536), -(-max(kv_lens) // 32))
        return -(-piece // 32) * 32

    # mixed steps: sequences with few rows leave the prompt kernel when their context is this long
    split_launch_min_kv = 1024

    def _attention_mfma(self, q, out, cache, ctx, nq, nkv, d, scale, window):
        """Which kernel for which sequences. Steps of decoded tokens only: the decode kernel.
        Other steps: the prompt kernels; but sequences of at most 16 rows with a long context
        (decoded tokens beside a prompt portion) would each walk all their keys in one block
        there, and hold the step up, so they go to the decode kernel in a launch of their own,
        which cuts their keys over many blocks."""
        if not scale > 0:
            raise OpsError(f"the bfloat16 attention kernels take a positive score scale, not {scale}")
        g = nq // nkv
        seqs = range(ctx.num_seqs)
        if ctx.max_q_len * g <= 16 and d <= 256:
            return self._launch_attention(q, out, cache, ctx, nq, nkv, d, scale, window, None, True)
        small = [s for s in seqs if ctx.q_lens_host[s] * g <= 16]
        if (d <= 256 and small and len(small) < ctx.num_seqs
                and max(ctx.kv_lens_host[s] for s in small) >= self.split_launch_min_kv):
            small_set = set(small)
            big = [s for s in seqs if s not in small_set]
            self._launch_attention(q, out, cache, ctx, nq, nkv, d, scale, window, small, True)
            self._launch_attention(q, out, cache, ctx, nq, nkv, d, scale, window, big, False)
            return
        self._launch_attention(q, out, cache, ctx, nq, nkv, d, scale, window, None, False)

    def _launch_attention(self, q, out, cache, ctx, nq, nkv, d, scale, window, subset, decode, own=None):
        """One launch over the sequences in ``subset`` (None: all of the step's). ``own``: the
        decode kernel takes the tokens' queries, own keys and own values from the q/k/v product
        (``decode_attention``); ``q`` is then None."""
        lib = attention_library(d)
        g = nq // nkv
        if subset is None:  # the step's own maxima: under a graph they are those of its bucket
            q_lens, kv_lens = ctx.q_lens_host, ctx.kv_lens_host
            max_rows, max_kv = ctx.max_q_len * g, ctx.max_kv_len
        else:
            q_lens = [ctx.q_lens_host[s] for s in subset]
            kv_lens = [ctx.kv_lens_host[s] for s in subset]
            max_rows, max_kv = max(q_lens) * g, max(kv_lens)
        waves = 1 if max_rows <= 16 else (2 if max_rows <= 32 else 4)
        # long portions: several row tiles per wave, so that loaded keys and values serve more rows
        row_tiles = 1 if max_rows <= 64 else (self.prefill_row_tiles if d <= 128 else min(2, self.prefill_row_tiles))
        # the list depends on the rows a tile holds (head geometry and kernel choice): layers of
        # another geometry in the same step get a list of their own
        key = ("attn_plan", g, nkv, d, waves, row_tiles, decode, None if subset is None else tuple(subset))
        plan = ctx.scratch.get(key)
        if plan is None:  # the same for every layer of the step
            dev = out.device
            if decode:
                tiles = None if subset is None else torch.tensor(subset, dtype=torch.int32, device=dev)
                n_tiles = len(q_lens)
            else:
                lds = waves == 4 and row_tiles >= 2 and self.prefill_through_lds
                groups = self.choose_key_groups(q_lens, kv_lens, g, nkv, window,
                                                ctx.scratch.get("attn_splits")) if lds else 0
                host, n_tiles = self.plan_tiles(q_lens, kv_lens, g, 16 * waves * row_tiles, nkv,
                                                self.resident_blocks if waves == 4 and row_tiles >= 2 and groups < 2
                                                else 0, subset)
                tiles = torch.from_numpy(host).to(dev)
            tokens = None
            if subset is not None:  # the tokens of these sequences: where a merge of key splits may write
                cu = np.concatenate([[0], np.cumsum(ctx.q_lens_host)])
                tokens = torch.from_numpy(np.concatenate([np.arange(cu[s], cu[s + 1]) for s in subset])
                                          .astype(np.int32)).to(dev)
            plan = (tiles, n_tiles, tokens, 0 if decode else groups)
            ctx.scratch[key] = plan
        tiles, n_tiles, tokens, groups = plan
        splits = ctx.scratch.get("attn_splits") or (
            self.choose_decode_splits(n_tiles, nkv, max_kv) if decode else self.choose_splits(n_tiles, nkv, max_kv))
        a = _AttnTileArgs()
        piece = None
        if decode and n_tiles <= 1024:
            piece = ctx.scratch.get("attn_piece")  # keys per piece, a multiple of 32: asked for outright
            if piece is None and "attn_splits" not in ctx.scratch:
                # the lengths as they are; a capture sees its bucket's instead and is told them beside
                piece = self.choose_decode_piece(ctx.scratch.get("attn_lens") or kv_lens, nkv)
        if piece:
            a.split_blocks = piece // 32
            # 32-key blocks a sequence of this launch can have: all its keys, or those of its
            # window, which may begin and end inside a block
            span = (max_kv + 31) // 32 if not window else (min(max_kv, window + 32) + 31) // 32 + 1
            splits = max(1, -(-span // a.split_blocks))
            if n_tiles * splits > 65535:
                piece, a.split_blocks = None, 0
                splits = self.choose_decode_splits(n_tiles, nkv, max_kv)
        a.out, a.k_cache, a.v_cache = out.data_ptr(), cache.k.data_ptr(), cache.v.data_ptr()
        if own is None:
            a.q = q.data_ptr()
        else:  # the token's own query, key and value come from the product that made them
            a.qkv, a.qkv_stride = own["qkv"].data_ptr(), own["qkv"].shape[1]
            a.q_weight, a.k_weight, a.rope = _addr(own["q_weight"]), _addr(own["k_weight"]), _addr(own["rope"])
            a.slots, a.eps = cache.group.slots.data_ptr(), own["eps"]
        a.cu_q = _need(ctx.cu_q, "cu_q", torch.int32, (ctx.num_seqs + 1,)).data_ptr()
        a.kv_lens = _need(ctx.kv_lens, "kv_lens", torch.int32, (ctx.num_seqs,)).data_ptr()
        a.block_table, a.table_width = cache.group.block_table.data_ptr(), cache.group.block_table.shape[1]
        if tiles is not None:
            a.tile_seq = tiles.data_ptr()
            if not decode:
                a.tile_row0 = tiles.data_ptr() + 4 * n_tiles
        if tokens is not None:
            a.merge_tokens, a.num_merge_tokens = tokens.data_ptr(), tokens.numel()
        a.num_tiles, a.nq, a.nkv, a.page_size, a.window = n_tiles, nq, nkv, cache.group.page_size, window
        a.num_splits, a.waves, a.row_tiles = splits, waves, row_tiles
        a.use_lds = groups
        a.scale_log2 = scale * math.log2(math.e)
        if splits > 1:
            part_o = torch.empty((ctx.num_tokens * nq * splits, d), dtype=torch.float32, device=out.device)
            part_lse = torch.empty((ctx.num_tokens * nq * splits,), dtype=torch.float32, device=out.device)
            a.part_o, a.part_lse = part_o.data_ptr(), part_lse.data_ptr()
        if piece:
            # the list of (sequence, piece): from the step's lengths on the device, once per pass
            a.max_items = n_tiles * splits
            list_key = ("attn_items", key, window, own is not None, piece, a.max_items)
            items = ctx.per_pass.get(list_key)
            if items is None:
                items = torch.empty((a.max_items, 2), dtype=torch.int32, device=out.device)
                a.items = items.data_ptr()
                self._check(lib, lib.qrt_attention_work_list(byref(a), c_int(own is not None), _stream()))
                ctx.per_pass[list_key] = items
            a.items = items.data_ptr()
        if decode:
            self._check(lib, lib.qrt_attention_bf16_decode(byref(a), c_int(ctx.num_tokens * nq), _stream()))
        else:
            self._check(lib, lib.qrt_attention_bf16(byref(a), c_int(ctx.num_tokens * nq), _stream()))

    # ---- sampling ------------------------------------------------------------------
    def argmax(self, logits):
        _need(logits, "logits", torch.float32)
        r, v = logits.shape
        out = torch.empty((r,), dtype=torch.int32, device=logits.device)
        self._check(self.lib, self.lib.qrt_argmax(_ptr(logits), _ptr(out), c_int(r), c_int(v), _stream()))
        return out

    def sample(self, logits, slot, fparams, iparams, seeds, counts=None, keep_processed=False):
        """One token per row of ``logits``. Options are read from the row's state slot:
        ``fparams[slot]`` = temperature, top_p, min_p, repetition, presence, frequency;
        ``iparams[slot]`` = top_k; ``seeds[slot]`` = seed, index of the next draw (advanced
        here). Returns (token int32 [R], logprob float32 [R], processed logits [R, V], buffer); the
        first two are the rows of the int32 buffer [2, R], so that one copy brings both to the host."""
        _need(logits, "logits", torch.float32)
        r, v = logits.shape
        _need(slot, "slot", torch.int32, (r,))
        n = fparams.shape[0]
        _need(fparams, "fparams", torch.float32, (n, 8))
        _need(iparams, "iparams", torch.int32, (n, 2))
        _need(seeds, "seeds", torch.int64, (n, 2))
        if counts is not None:
            _need(counts, "counts", torch.int32, (n, v))
        work = torch.empty_like(logits)
        # ids and log-probabilities side by side, so that one copy brings both to the host
        both = torch.empty((2, r), dtype=torch.int32, device=logits.device)
        tok, lp = both[0], both[1].view(torch.float32)
        a = _SampleArgs()
        a.logits, a.work, a.counts, a.slot = logits.data_ptr(), work.data_ptr(), _addr(counts), slot.data_ptr()
        a.fparams, a.iparams, a.seeds = fparams.data_ptr(), iparams.data_ptr(), seeds.data_ptr()
        a.out_token, a.out_logprob, a.rows, a.vocab = tok.data_ptr(), lp.data_ptr(), r, v
        a.write_work = 1 if keep_processed else 0  # greedy rows skip the write unless asked
        # few rows: the first pass over each row is spread over blocks (about 256 in all)
        parts = min(64, 256 // r, v // 2048) if r <= 64 else 0
        if parts >= 2:
            partials = torch.empty((r, parts, 4), dtype=torch.float32, device=logits.device)
            a.partials, a.parts = partials.data_ptr(), parts
        self._check(self.lib, self.lib.qrt_sample(byref(a), _stream()))
        return tok, lp, work, both

    def count_tokens(self, counts, slots, tokens):
        _need(counts, "counts", torch.int32)
        _need(slots, "slots", torch.int32)
        _need(tokens, "tokens", torch.int32, tuple(slots.shape))
        self._check(self.lib, self.lib.qrt_count_tokens(_ptr(counts), _ptr(slots), _ptr(tokens),
                                                        c_int(slots.numel()), c_int(counts.shape[1]), _stream()))

    def add_bias(self, logits, rows, tokens, values):
        _need(logits, "logits", torch.float32)
        n = rows.numel()
        _need(rows, "rows", torch.int32)
        _need(tokens, "tokens", torch.int32, (n,))
        _need(values, "values", torch.float32, (n,))
        self._check(self.lib, self.lib.qrt_add_bias(_ptr(logits), _ptr(rows), _ptr(tokens), _ptr(values),
                                                    c_int(n), c_int(logits.shape[1]), _stream()))
