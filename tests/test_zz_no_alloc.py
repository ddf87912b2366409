"""The sampling entry point that allocates nothing (``qrt_sample_noalloc``) against the
existing one (``qrt_sample``), called through ``ctypes`` with buffers this test owns: two calls
in a row, the second with a smaller input, so that what the first call left in the library's
built-in buffer is still there when the second runs; then sizes beyond the buffer are refused."""

import ctypes
from ctypes import byref, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _library():
    from qwen3_runtime_amd.ops import hip

    lib = hip.core_library()
    return lib, hip._SampleArgs, hip.current_stream


def _case(rows, vocab, seed):
    """Inputs of one call: logits, per-slot options (greedy rows and drawing rows, with and
    without penalties), seeds, counts."""
    g = torch.Generator().manual_seed(seed)
    logits = (3.0 * torch.randn(rows, vocab, generator=g)).to(DEV)
    slots = rows + 3
    slot = torch.randperm(slots, generator=g)[:rows].to(torch.int32).to(DEV)
    fparams = torch.zeros(slots, 8)
    fparams[:, 0] = torch.tensor([0.0 if i % 3 == 0 else 0.5 + 0.25 * (i % 5) for i in range(slots)])  # temperature
    fparams[:, 1] = torch.tensor([1.0 if i % 2 else 0.9 for i in range(slots)])                       # top_p
    fparams[:, 2] = torch.tensor([0.0 if i % 4 else 0.01 for i in range(slots)])                      # min_p
    fparams[:, 3] = torch.tensor([1.0 if i % 2 == 0 else 1.3 for i in range(slots)])                  # repetition
    fparams[:, 4] = 0.1
    fparams[:, 5] = 0.05
    iparams = torch.zeros(slots, 2, dtype=torch.int32)
    iparams[:, 0] = torch.tensor([0 if i % 2 else 40 for i in range(slots)], dtype=torch.int32)      # top_k
    seeds = torch.stack([torch.arange(slots) * 7919 + seed, torch.arange(slots) % 4], dim=1).to(torch.int64)
    counts = torch.randint(0, 3, (slots, vocab), generator=g, dtype=torch.int32)
    return logits, slot, fparams.to(DEV), iparams.to(DEV), seeds.to(DEV), counts.to(DEV)


def _call(entry, case, parts, partials=None):
    """One call of ``entry`` on copies of the mutable inputs; returns tokens, log-probabilities,
    processed logits and the advanced seeds."""
    lib, Args, stream = _library()
    logits, slot, fparams, iparams, seeds, counts = case
    rows, vocab = logits.shape
    seeds = seeds.clone()
    work = torch.full_like(logits, float("nan"))
    tok = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    lp = torch.full((rows,), float("nan"), dtype=torch.float32, device=DEV)
    a = Args()
    a.logits, a.work, a.counts, a.slot = logits.data_ptr(), work.data_ptr(), counts.data_ptr(), slot.data_ptr()
    a.fparams, a.iparams, a.seeds = fparams.data_ptr(), iparams.data_ptr(), seeds.data_ptr()
    a.out_token, a.out_logprob, a.rows, a.vocab = tok.data_ptr(), lp.data_ptr(), rows, vocab
    a.write_work, a.parts = 1, parts
    a.partials = None if partials is None else partials.data_ptr()
    code = getattr(lib, entry)(byref(a), stream())
    torch.cuda.synchronize()
    return code, (tok.cpu(), lp.cpu(), work.cpu(), seeds.cpu())


def _same(got, want):
    for g, w in zip(got, want):
        assert torch.equal(g, w) or torch.allclose(g, w, rtol=0, atol=0, equal_nan=True)


def test_no_alloc_sampling_equals_the_existing_entry_point_twice_in_a_row():
    lib, _, _ = _library()
    lib.qrt_last_error.restype = ctypes.c_char_p
    torch.zeros(1, device=DEV)  # the device is current in this thread
    # set-up ahead of the first call, as a caller under stream capture would; again is harmless
    assert lib.qrt_sample_noalloc_setup() == 0, lib.qrt_last_error().decode()
    assert lib.qrt_sample_noalloc_setup() == 0
    # first call: 12 rows in 21 parts each; second, right after it: 5 rows of a shorter vocabulary
    # in 9 parts, which finds the first call's results still in the built-in buffer
    for rows, vocab, parts, seed in ((12, 50_000, 21, 1), (5, 20_480, 9, 2)):
        case = _case(rows, vocab, seed)
        partials = torch.empty((rows, parts, 4), dtype=torch.float32, device=DEV)
        code, want = _call("qrt_sample", case, parts, partials)
        assert code == 0, lib.qrt_last_error().decode()
        before = torch.cuda.memory_allocated()
        code, got = _call("qrt_sample_noalloc", case, parts)
        assert code == 0, lib.qrt_last_error().decode()
        assert torch.cuda.memory_allocated() == before
        assert (want[0] >= 0).all() and (want[0] < vocab).all() and torch.isfinite(want[1]).all()
        _same(got, want)
    # no parts at all: one block per row does both passes; the buffer is not touched
    case = _case(3, 1000, 3)
    _, want = _call("qrt_sample", case, 0)
    code, got = _call("qrt_sample_noalloc", case, 0)
    assert code == 0
    _same(got, want)


def test_no_alloc_sampling_refuses_what_its_buffer_cannot_hold():
    lib, _, _ = _library()
    lib.qrt_last_error.restype = ctypes.c_char_p
    case = _case(65, 4096, 4)
    code, (tok, _, _, _) = _call("qrt_sample_noalloc", case, 64)  # 65 * 64 * 16 bytes > 64 KiB
    assert code != 0 and "need 66560 bytes" in lib.qrt_last_error().decode()
    assert (tok == -7).all(), "nothing ran"
    code, _ = _call("qrt_sample_noalloc", _case(64, 4096, 5), 64)  # exactly the buffer
    assert code == 0, lib.qrt_last_error().decode()
