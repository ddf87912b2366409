"""The engine on the GPU against the plain implementation, in float32 and bfloat16:
each request whole; the last 32 tokens one by one; portions of changing size;
up to four live requests mixed, with so few pages that they are reused."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parents[1]
WORKLOADS = {"tiny_a": [1, 7, 33, 70], "tiny_b": [3, 17, 40, 64, 95]}
# float32: rounding of a few hundred float32 operations.
TOL_F32 = dict(atol=5e-5, rtol=5e-5)


def check(got, want, dtype):
    """float32 to rounding of float32 sums; bfloat16 as noise relative to the logits' own spread
    (about 0.2 at these sizes), which a wrong or stale key at one position does not pass."""
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        traces.compare_rounding_noise(got, want)


def load_gpu(folder, page_size, num_pages, dtype, max_seqs=4, hip_graph=False):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    cfg = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs, dtype=dtype,
                       device="cuda:0", hip_graph=hip_graph)
    return load(folder, cfg)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(model_folders, tiny_configs, name, cut, dtype):
    cfg, page = tiny_configs[name]
    reqs = traces.make_requests(cfg.vocab_size, WORKLOADS[name], seed=5)
    steps = getattr(traces, cut)(reqs)
    # as many pages as the live requests hold at the peak, counted in pages
    loaded = load_gpu(model_folders[name], page, traces.peak_tokens(steps, unit=page) // page, dtype)
    got = traces.replay(loaded, steps)
    check(got, traces.plain_logits(model_folders[name], reqs), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [4, 8, 16])
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
def test_page_sizes_under_the_cutting_pattern(model_folders, tiny_configs, name, page, dtype):
    """Pages of 4, 8 and 16 tokens (the reference's pattern, tests/invariance/test_kv.py:12-69) with
    requests mixed in a pool at its peak. Pages of 4 are no multiple of 8, so bfloat16 attention
    then runs in the general kernel instead of the MFMA ones."""
    cfg, _ = tiny_configs[name]
    reqs = traces.make_requests(cfg.vocab_size, REUSE_WORKLOADS[name][:6], seed=13)
    steps = traces.mixed(reqs, seed=page, max_live=3)
    loaded = load_gpu(model_folders[name], page, traces.peak_tokens(steps, unit=page) // page, dtype)
    got = traces.replay(loaded, steps)
    check(got, traces.plain_logits(model_folders[name], reqs), dtype)


@pytest.fixture(scope="module")
def odd_folder(tmp_path_factory):
    """A third tiny model with sizes the kernels' fast paths do not take: head size 80 (a 16-wide
    remainder for the MFMA, no power of two for the wide q/k kernel), three query heads per key
    head, a width, a feed-forward size and a vocabulary that are multiples of nothing much."""
    from qwen3_runtime_amd.config.model import Qwen3Config
    from qwen3_runtime_amd.weights import write_model_folder

    cfg = Qwen3Config(vocab_size=333, hidden_size=176, num_hidden_layers=2, num_attention_heads=6,
                      num_key_value_heads=2, head_dim=80, intermediate_size=208, rms_norm_eps=3e-6,
                      rope_theta=50000.0, max_position_embeddings=512, tie_word_embeddings=True)
    folder = tmp_path_factory.mktemp("odd")
    write_model_folder(folder, cfg.to_dict(), seed=31)
    return cfg, folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "portions", "mixed"])
def test_odd_sizes_and_pages_of_24(odd_folder, cut, dtype):
    """Pages of 24 tokens (no power of two: the kernels divide instead of shifting)."""
    cfg, folder = odd_folder
    page = 24
    reqs = traces.make_requests(cfg.vocab_size, [5, 50, 97, 130], seed=2)
    steps = getattr(traces, cut)(reqs)
    loaded = load_gpu(folder, page, -(-traces.peak_tokens(steps, unit=72) // page), dtype)
    got = traces.replay(loaded, steps)
    check(got, traces.plain_logits(folder, reqs), dtype)


REUSE_WORKLOADS = {"tiny_a": [33, 70, 1, 7, 20, 45, 64, 16, 50, 31], "tiny_b": [40, 64, 95, 17, 33, 80, 130, 2]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
def test_mixed_with_page_reuse(model_folders, tiny_configs, name, dtype):
    """More requests than may be live at once, in a pool of exactly the pages the live ones hold
    at the peak (counted in pages, not rounded up): pages freed by a finished request are taken
    by later tokens of others, whose logits must not show what the pages held before."""
    cfg, page = tiny_configs[name]
    reqs = traces.make_requests(cfg.vocab_size, REUSE_WORKLOADS[name], seed=9)
    steps = traces.mixed(reqs, seed=3, max_live=3 if name == "tiny_a" else 4)
    pages = traces.peak_tokens(steps, unit=page) // page
    assert pages < sum(-(-len(t) // page) for t in reqs.values())
    loaded = load_gpu(model_folders[name], page, pages, dtype)
    users: dict = {}
    got = traces.replay(loaded, steps, page_users=users)
    shared = [p for p, who in users.items() if len(who) > 1]
    assert len(shared) >= pages // 2, f"only {len(shared)} of {pages} pages served two requests"
    check(got, traces.plain_logits(model_folders[name], reqs), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
def test_pages_that_come_back_full_of_nan(model_folders, tiny_configs, name, dtype):
    """The same with every page filled with NaN and infinities at the start and again whenever its
    request ends: a later holder writes its own keys and values into part of such a page, and the
    places it has not written yet (the rest of the page, within the last group of 8 keys too)
    must not be multiplied, not even by a probability of zero."""
    cfg, page = tiny_configs[name]
    reqs = traces.make_requests(cfg.vocab_size, REUSE_WORKLOADS[name], seed=19)
    steps = traces.mixed(reqs, seed=4, max_live=3 if name == "tiny_a" else 4)
    loaded = load_gpu(model_folders[name], page, traces.peak_tokens(steps, unit=page) // page, dtype)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, traces.plain_logits(model_folders[name], reqs), dtype)


@pytest.mark.parametrize("seed", [3, 5, 6, 17, 26, 45])
def test_random_models_and_random_traces(tmp_path, seed):
    """A model and a trace drawn from the seed: head sizes 16 to 256 (64 and up also take the decode
    kernel that forms its own queries and keys), 1 to 4 key heads with 1 to 16 query heads each,
    widths and vocabularies that are multiples of nothing much, pages of 8 to 64, prompts of 1 to
    1,500 tokens cut at random beside decoded tokens, a pool of exactly the pages the live requests
    hold at the peak. In float32 and in bfloat16, with and without graphs, against the plain model.
    (Hundreds of further seeds of this generator were run once; these six are kept.)"""
    import random

    from qwen3_runtime_amd.config.model import Qwen3Config
    from qwen3_runtime_amd.weights import write_model_folder

    rng = random.Random(seed)
    d = rng.choice((16, 48, 64, 64, 128, 128, 192, 256))
    nkv, g = rng.choice((1, 2, 3, 4)), rng.choice((1, 2, 4, 5, 8, 16))
    cfg = Qwen3Config(vocab_size=rng.choice((257, 512, 1000)), hidden_size=rng.choice((96, 160, 256, 264)),
                      num_hidden_layers=rng.choice((1, 2, 3)), num_attention_heads=nkv * g, num_key_value_heads=nkv,
                      head_dim=d, intermediate_size=rng.choice((128, 208, 512)), rms_norm_eps=rng.choice((1e-6, 1e-5)),
                      rope_theta=rng.choice((10000.0, 1e6)), max_position_embeddings=4096,
                      tie_word_embeddings=rng.random() < 0.5)
    page = rng.choice((8, 16, 16, 24, 32, 64))
    lengths = [rng.choice((1, 2, 5, 33, 64, 65, 127, 200, 400, 700, 1100, 1500)) for _ in range(rng.randint(2, 6))]
    write_model_folder(tmp_path, cfg.to_dict(), seed=seed)
    reqs = traces.make_requests(cfg.vocab_size, lengths, seed=seed)
    steps = traces.random_trace(reqs, rng, rng.randint(1, 4))
    pages = traces.peak_tokens(steps, unit=page) // page
    want = None
    for dtype in ("float32", "bfloat16"):
        loaded = load_gpu(tmp_path, page, pages, dtype, hip_graph=rng.random() < 0.5)
        got = traces.replay(loaded, steps)
        if want is None:
            full = traces.plain_logits(tmp_path, reqs)
            want = {k: full[k] for k in got}
        if dtype == "float32":
            traces.compare(got, want, atol=1e-4, rtol=1e-4)
        else:
            traces.compare_rounding_noise(got, want)
        del loaded
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_folders, tiny_configs, dtype):
    """A short prompt, then 400 tokens one by one: crosses many pages and attention key blocks."""
    cfg, page = tiny_configs["tiny_a"]
    reqs = traces.make_requests(cfg.vocab_size, [420], seed=2)
    steps = traces.tail_one_by_one(reqs, tail=400)
    loaded = load_gpu(model_folders["tiny_a"], page, traces.peak_tokens(steps) // page, dtype)
    got = traces.replay(loaded, steps)
    check(got, traces.plain_logits(model_folders["tiny_a"], reqs), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, tiny_configs, tmp_path, dtype):
    """bin/trace_run as a user runs it: steps on stdin, files out, 'done' lines."""
    cfg, page = tiny_configs["tiny_b"]
    reqs = traces.make_requests(cfg.vocab_size, [19, 45, 70], seed=4)
    steps = traces.mixed(reqs, seed=1, max_live=3)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_folders["tiny_b"]),
         "--dtype", dtype, "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps))],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    got, pos = {}, {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        if n_want:
            arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n_want, cfg.vocab_size)
            row = 0
            for e in s["entries"]:
                for w in e["want"]:
                    got[(e["id"], pos.get(e["id"], 0) + w)] = torch.from_numpy(arr[row].copy())
                    row += 1
        for e in s["entries"]:
            pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
    check(got, traces.plain_logits(model_folders["tiny_b"], reqs), dtype)


def test_trace_run_program_with_a_preset_and_a_page_count(tmp_path):
    """``--preset NAME --seed S`` in place of a folder and ``--num-pages`` in place of ``--max-tokens``:
    the logits are those of an engine built in this process from the same registered
    configuration and seed, stepped the same way."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import build_model, load
    from qwen3_runtime_amd.registry import preset_config
    from qwen3_runtime_amd.weights import RandomSource

    raw = preset_config("tiny_a")
    reqs = traces.make_requests(raw["vocab_size"], [21, 40], seed=8)
    steps = traces.portions(reqs)
    pages = traces.peak_tokens(steps, unit=16) // 16
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--preset", "tiny_a", "--seed", "6", "--dtype", "float32",
         "--out", str(out), "--num-pages", str(pages)],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-3000:]
    source = RandomSource(build_model(raw)[1].tensor_decls(), 6, norm_jitter=0.1)
    loaded = load(None, EngineConfig(page_size=16, num_pages=pages, max_num_seqs=4, dtype="float32", device="cuda:0",
                                     hip_graph=False), source=source, raw_config=raw)
    want = traces.replay(loaded, steps)
    pos: dict = {}
    for s in steps:
        arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, raw["vocab_size"])
        row = 0
        for e in s["entries"]:
            for w in e["want"]:
                assert torch.equal(torch.from_numpy(arr[row].copy()), want[(e["id"], pos.get(e["id"], 0) + w)])
                row += 1
            pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        assert row == arr.shape[0]
    # neither or both of a pair of options is a usage error
    for bad in (["--max-tokens", "64"], ["--preset", "tiny_a", "--model", "x", "--max-tokens", "64"],
                ["--preset", "tiny_a"]):
        proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--out", str(out), *bad],
                              input="", capture_output=True, text=True, timeout=120)
        assert proc.returncode == 2, (bad, proc.stderr[-500:])
