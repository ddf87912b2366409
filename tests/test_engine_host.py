"""The step function, the cache and the ways of cutting, on the CPU.

The engine's ops are replaced by their plain torch versions (the kernels cannot
run here), so what these tests pin is the host side: packing, block tables,
slots, page reuse, lengths. Logits must equal the plain implementation's under
every cutting, in float32.
"""

import pytest
import torch

import traces
from plain.ops_ref import TorchOps


def load_cpu(folder, page_size, num_pages, max_seqs=4):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    cfg = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs, dtype="float32",
                       device="cpu", hip_graph=False)
    return load(folder, cfg, ops=TorchOps())


WORKLOADS = {"tiny_a": [1, 7, 33, 70], "tiny_b": [3, 17, 40, 64, 95]}


@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(model_folders, tiny_configs, name, cut):
    cfg, page = tiny_configs[name]
    reqs = traces.make_requests(cfg.vocab_size, WORKLOADS[name], seed=5)
    steps = getattr(traces, cut)(reqs)
    pages = traces.peak_tokens(steps) // page
    loaded = load_cpu(model_folders[name], page, pages)
    got = traces.replay(loaded, steps)
    traces.compare(got, traces.plain_logits(model_folders[name], reqs), atol=2e-5, rtol=2e-5)


def test_pages_are_reused_in_the_mixed_trace(model_folders, tiny_configs):
    cfg, page = tiny_configs["tiny_b"]
    reqs = traces.make_requests(cfg.vocab_size, [40, 64, 95, 17, 33, 80], seed=9)
    steps = traces.mixed(reqs, seed=3)
    pages = traces.peak_tokens(steps) // page
    total_needed = sum(-(-len(t) // page) for t in reqs.values())
    assert pages < total_needed  # so some page must serve two requests
    loaded = load_cpu(model_folders["tiny_b"], page, pages)
    got = traces.replay(loaded, steps)
    traces.compare(got, traces.plain_logits(model_folders["tiny_b"], reqs), atol=2e-5, rtol=2e-5)


def test_step_refuses_bad_entries(model_folders, tiny_configs):
    from qwen3_runtime_amd.cache import CacheFull
    from qwen3_runtime_amd.engine.batch import StepEntry

    cfg, page = tiny_configs["tiny_a"]
    loaded = load_cpu(model_folders["tiny_a"], page, 2)
    loaded.cache.admit("a")
    with pytest.raises(ValueError, match="twice"):
        loaded.runner.step([StepEntry("a", [1]), StepEntry("a", [2])])
    with pytest.raises(ValueError, match="outside"):
        loaded.runner.step([StepEntry("a", [cfg.vocab_size])])
    with pytest.raises(ValueError, match="wants row"):
        loaded.runner.step([StepEntry("a", [1, 2], want=[2])])
    with pytest.raises(CacheFull):
        loaded.runner.step([StepEntry("a", list(range(3 * page)))])
    assert loaded.cache.length("a") == 0
    loaded.cache.check()


def test_which_kernel_multiplies_how_many_rows():
    """The host's choice between the few-row kernel, the kernel that shares activations through
    LDS and the vendor library, by form of the product and number of rows; and the attention work
    list: every row of every sequence once, longest tiles first, the subset's own sequence ids."""
    from qwen3_runtime_amd.ops.hip import HipOps

    ops = HipOps.__new__(HipOps)          # the choices need no library and no GPU
    assert [ops._own_kernel(m, 6144, 2560, "whole") for m in (1, 16, 17, 64, 65)] == [0, 0, 1, 1, None]
    assert [ops._own_kernel(m, 9728, 2560, "gated") for m in (1, 11, 12, 64, 128, 129)] == [0, 0, 1, 1, 1, None]
    assert [ops._own_kernel(m, 2560, 4096, "planes") for m in (1, 8, 9, 128, 129)] == [0, 0, 1, 1, None]
    assert [ops._own_kernel(m, 1000, 2560, "whole") for m in (1, 16, 17)] == [0, 0, None]   # rows no multiple of 16
    assert [ops._own_kernel(m, 2560, 96, "planes") for m in (8, 16, 17)] == [0, 0, None]    # K no multiple of 64
    # the few-row kernel cuts K when there are few row tiles (four parts up to 8,192 columns, eight
    # beyond: the 4B, 8B and 32B output and down projections); the sharing kernel until the chip is full
    assert HipOps.choose_k_parts(2560, 4096, 8) == 4 and HipOps.choose_k_parts(2560, 9728, 8) == 8
    assert HipOps.choose_k_parts(4096, 4096, 8) == 4 and HipOps.choose_k_parts(4096, 12288, 1) == 8
    assert HipOps.choose_k_parts(5120, 8192, 8) == 4 and HipOps.choose_k_parts(5120, 25600, 8) == 8
    assert HipOps.choose_k_parts(6144, 2560, 8) == 1 and HipOps.choose_k_parts(2560, 64, 8) == 1
    assert HipOps.choose_k_parts(2560, 4096, 64) == 8 and HipOps.choose_k_parts(2560, 4096, 12, True) == 8
    assert HipOps.choose_k_parts(2560, 384, 64) == 1 and HipOps.choose_k_parts(65536, 4096, 64) == 1

    q_lens, kv_lens, g = [70, 1, 33], [200, 900, 33], 4
    tiles, n = HipOps.plan_tiles(q_lens, kv_lens, g, 64, nkv=2)
    seqs, row0 = tiles[:n].tolist(), tiles[n: 2 * n].tolist()
    covered = {}
    for s, r in zip(seqs, row0):
        covered.setdefault(s, []).append(r)
    assert {s: sorted(r) for s, r in covered.items()} == {0: [0, 64, 128, 192, 256], 1: [0], 2: [0, 64, 128]}
    assert seqs[0] == 1                  # the tile that sees 900 keys goes first
    sub, n_sub = HipOps.plan_tiles([70, 33], [200, 33], g, 64, nkv=2, seq_ids=[0, 2])
    assert sorted(set(sub[:n_sub].tolist())) == [0, 2]


def cpu_engine(folder, page_size, num_pages):
    from qwen3_runtime_amd.llm import build_engine

    return build_engine(folder, block_size=page_size, num_kv_blocks=num_pages, max_num_seqs=2, dtype="float32",
                        device="cpu", cuda_graph=False, ops=TorchOps())


def test_ids_that_would_index_device_memory_are_checked_on_arrival(model_folders, tiny_configs):
    """Prompt ids, forced ids and logit_bias keys all end up as indices in kernels (embedding
    rows, columns of the logits, penalty counts): one outside the vocabulary is refused when the
    request is added, with nothing queued."""
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg, page = tiny_configs["tiny_a"]
    eng = cpu_engine(model_folders["tiny_a"], page, 8)
    v = cfg.vocab_size
    with pytest.raises(ValueError, match="prompt token"):
        eng.add_request([1, v])
    with pytest.raises(ValueError, match="prompt token"):
        eng.add_request([-1])
    with pytest.raises(ValueError, match=f"forced token {v + 5}"):
        eng.add_request([1, 2], forced_tokens=[3, v + 5])
    with pytest.raises(ValueError, match="logit_bias key -2"):
        eng.add_request([1, 2], sampling=SamplingParams(logit_bias={-2: 1.0}))
    with pytest.raises(ValueError, match=f"logit_bias key {v}"):
        eng.add_request([1, 2], sampling=SamplingParams(logit_bias={0: 1.0, v: 1.0}))
    for bad in (float("nan"), float("inf")):
        with pytest.raises(ValueError, match="a bias is a finite number"):
            eng.add_request([1, 2], sampling=SamplingParams(logit_bias={3: bad}))
    assert eng.is_finished() and not eng._live
    # in range, and -inf (an excluded id), are taken
    eng.add_request([1, v - 1], forced_tokens=[0, v - 1], sampling=SamplingParams(logit_bias={v - 1: float("-inf")}))
    assert not eng.is_finished()


def test_default_page_count_is_capped_by_what_requests_can_use(monkeypatch, model_folders):
    """No page count given: the pool is sized from free memory but never beyond
    max_num_seqs requests of max_model_len tokens (plus a spare page each)."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.config.model import read_config_json
    from qwen3_runtime_amd.engine import factory

    _, model = factory.build_model(read_config_json(model_folders["tiny_b"]))
    per_page = 2 * 3 * 2 * 32 * 8 * 2          # keys and values, 3 layers, 2 heads of 32, 8 tokens, bfloat16
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (200 * 2**30, 288 * 2**30))
    cfg = EngineConfig(page_size=8, max_num_seqs=4, max_model_len=100, dtype="bfloat16")
    assert factory.pages_for_memory(model, cfg, torch.bfloat16, "cuda:0") == 4 * (13 + 1)
    # memory is the limit when it is the smaller one; never fewer than 32 pages
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (40 * per_page, 288 * 2**30))
    assert factory.pages_for_memory(model, cfg, torch.bfloat16, "cuda:0") == int(40 * 0.85)
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (per_page, 288 * 2**30))
    assert factory.pages_for_memory(model, cfg, torch.bfloat16, "cuda:0") == 32
    # without max_model_len the model's position limit stands in
    cfg = EngineConfig(page_size=8, max_num_seqs=2, dtype="bfloat16")
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (200 * 2**30, 288 * 2**30))
    limit = model.plan.max_positions
    assert factory.pages_for_memory(model, cfg, torch.bfloat16, "cuda:0") == 2 * (-(-limit // 8) + 1)


def test_bytes_and_operations_of_a_step_come_from_the_plan():
    """What a measurement prices a step with, for the 4B configuration, against the architecture's
    own arithmetic: every matrix once (the tied table as the head, not twice), two norm vectors and
    the q/k norms per layer, the cache of the live requests; a 2,048-token prompt's operations."""
    from qwen3_runtime_amd.cache import CacheManager
    from qwen3_runtime_amd.engine.factory import build_model
    from qwen3_runtime_amd.registry import preset_config

    raw = preset_config("qwen3_4b")
    _, model = build_model(raw)
    h, d, i, v, layers = 2560, 128, 9728, 151936, 36
    q, kv = 32 * d, 8 * d
    per_layer = h * (q + 2 * kv) + q * h + 3 * h * i
    weights = 2 * (v * h + layers * (per_layer + 2 * h + 2 * d) + h)
    decode = model.step_cost([(1, 2090)] * 8, rows=8, elem_bytes=2)
    assert decode.total_weight_bytes == weights and round(weights / 1e9, 3) == 8.045
    cache = CacheManager(model.plan.caches, page_size=16, num_pages=2, max_requests=8, device="cpu",
                         dtype=torch.bfloat16, allocate=False)
    assert cache.bytes_read([2090] * 8) == 8 * 2090 * 2 * layers * kv * 2          # 147,456 bytes a token
    assert round((weights + cache.bytes_read([2090] * 8)) / 1e9, 2) == 10.51
    prompt = model.step_cost([(2048, 2048)], rows=1, elem_bytes=2)
    attention = 4 * 32 * d * (2048 * 2049 // 2) * layers
    assert prompt.flop == 2 * 2048 * layers * per_layer + attention + 2 * v * h
    assert abs(prompt.flop / 1.612e13 - 1) < 1e-3
    # an untied head: the embedding table is looked up (one row per token), the head is read whole
    raw8 = preset_config("qwen3_8b")
    _, model8 = build_model(raw8)
    cost = model8.step_cost([(1, 100)], rows=1, elem_bytes=2)
    assert cost.weight_bytes["model.embed_tokens.weight"] == 4096 * 2
    assert cost.weight_bytes["lm_head.weight"] == 151936 * 4096 * 2
