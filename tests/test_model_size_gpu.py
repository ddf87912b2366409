"""The engine at the layer sizes of the 4B and 8B models (two layers, a small vocabulary)
against the plain implementation: the kernels' production paths (few-row products on
tile-major weights with K cut into planes, the gated epilogue, decode attention at head size
128 with four query heads per key head, prompt attention through LDS, the vendor products for
long portions) as parts of a whole model, in float32 and bfloat16."""

import dataclasses

import pytest
import torch

import traces

pytestmark = pytest.mark.gpu

# float32: the longest sums have 12,288 terms instead of the tiny models' few hundred.
TOL_F32 = dict(atol=2e-4, rtol=2e-4)


check_rounding_noise = traces.compare_rounding_noise


@pytest.fixture(scope="module")
def sized_folders(tmp_path_factory):
    from qwen3_runtime_amd.config.presets import preset
    from qwen3_runtime_amd.weights import write_model_folder

    out = {}
    for i, name in enumerate(("qwen3_4b", "qwen3_8b")):
        cfg = dataclasses.replace(preset(name), num_hidden_layers=2, vocab_size=2048, eos_token_id=None)
        folder = tmp_path_factory.mktemp(name)
        write_model_folder(folder, cfg.to_dict(), seed=21 + i)
        out[name] = (cfg, folder)
    return out


@pytest.fixture(scope="module")
def plain_results(sized_folders):
    out = {}
    for name, (cfg, folder) in sized_folders.items():
        reqs = traces.make_requests(cfg.vocab_size, [150, 41, 9], seed=6)
        out[name] = (reqs, traces.plain_logits(folder, reqs))
    return out


@pytest.mark.parametrize("dtype,cut", [("float32", "portions"), ("bfloat16", "mixed"), ("bfloat16", "tail_one_by_one")])
@pytest.mark.parametrize("name", ["qwen3_4b", "qwen3_8b"])
def test_model_sized_layers_match_plain(sized_folders, plain_results, name, dtype, cut):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    cfg, folder = sized_folders[name]
    reqs, want = plain_results[name]
    steps = getattr(traces, cut)(reqs)
    page = 16
    engine_cfg = EngineConfig(page_size=page, num_pages=traces.peak_tokens(steps) // page, max_num_seqs=4, dtype=dtype,
                              device="cuda:0", hip_graph=False)
    loaded = load(folder, engine_cfg)
    got = traces.replay(loaded, steps)
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)


@pytest.mark.parametrize("live", [20, 40, 64])
def test_many_requests_decode_together_at_model_sizes(sized_folders, live):
    """17 to 64 requests decoding in one step at the 4B layer sizes: the products with that many
    rows (own kernel on tile-major weights: whole result, gated, K cut into planes), decode
    attention over many sequences. Prompts in three steps, then six steps with a token of every
    request, against the plain implementation of each request alone."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    cfg, folder = sized_folders["qwen3_4b"]
    lengths = [9 + (5 * i) % 23 for i in range(live)]
    reqs = traces.make_requests(cfg.vocab_size, lengths, seed=30 + live)
    rids = list(reqs)
    steps, decode = [], 6
    for lo in range(0, live, (live + 2) // 3):
        part = rids[lo: lo + (live + 2) // 3]
        steps.append({"entries": [{"id": r, "tokens": reqs[r][:-decode], "want": [len(reqs[r]) - decode - 1]}
                                  for r in part], "end": []})
    for d in range(decode, 0, -1):
        steps.append({"entries": [{"id": r, "tokens": reqs[r][len(reqs[r]) - d: len(reqs[r]) - d + 1], "want": [0]}
                                  for r in rids], "end": rids if d == 1 else []})
    steps = traces._number(steps)
    want_all = traces.plain_logits(folder, reqs)
    engine_cfg = EngineConfig(page_size=16, num_pages=live * 3, max_num_seqs=live, max_num_batched_tokens=1024,
                              dtype="bfloat16", device="cuda:0", hip_graph=False)
    loaded = load(folder, engine_cfg)
    assert loaded.runner.ops._tiled, "the weights have tile-major copies: the own kernels run"
    got = traces.replay(loaded, steps)
    assert len(got) == live * (decode + 1)
    check_rounding_noise(got, {k: want_all[k] for k in got})


def test_long_context_decode_beside_a_prompt_portion(sized_folders, monkeypatch):
    """Decoded tokens of a request that holds 1,100 keys in the same steps as portions of another
    request's prompt: attention then runs as two launches (the decode kernel with its keys cut
    over blocks, the prompt kernels for the portion). Against the plain implementation."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load
    from qwen3_runtime_amd.ops.hip import HipOps

    cfg, folder = sized_folders["qwen3_4b"]
    reqs = traces.make_requests(cfg.vocab_size, [1106, 150], seed=12)
    long_ids, other = reqs["r0"], reqs["r1"]
    steps = [{"entries": [{"id": "r0", "tokens": long_ids[:1100], "want": [1099]}], "end": []}]
    cuts = [0, 40, 70, 100, 120, 137, 150]
    for i in range(6):
        steps.append({"entries": [{"id": "r0", "tokens": long_ids[1100 + i: 1101 + i], "want": [0]},
                                  {"id": "r1", "tokens": other[cuts[i]: cuts[i + 1]],
                                   "want": list(range(cuts[i + 1] - cuts[i]))}],
                      "end": ["r0", "r1"] if i == 5 else []})
    steps = traces._number(steps)
    launches = []
    inner = HipOps._launch_attention
    monkeypatch.setattr(HipOps, "_launch_attention",
                        lambda self, *a: (launches.append(a[-2:]), inner(self, *a))[1])
    engine_cfg = EngineConfig(page_size=16, num_pages=traces.peak_tokens(steps) // 16, max_num_seqs=4, dtype="bfloat16",
                              device="cuda:0", hip_graph=False)
    got = traces.replay(load(folder, engine_cfg), steps)
    assert ([0], True) in launches and ([1], False) in launches, "the mixed steps ran as two launches"
    want = traces.plain_logits(folder, reqs)
    check_rounding_noise(got, {k: want[k] for k in got})


def test_model_sized_decode_graph_equals_eager(sized_folders):
    """Three requests at the 4B layer sizes, decoded eagerly and then from replayed HIP graphs that
    are fed the eager tokens: at every token the graph's log-probability of it is the eager one up
    to the rounding of bfloat16. (A graph cuts the keys for the length of its bucket, an eager step
    for the length of the step's longest context, so the partial sums of attention are formed in
    another order; random weights make the distribution over 2,048 tokens nearly flat, and tokens
    chosen freely part ways at the first near-tie, which says nothing. Measured difference: 0.01
    for the request whose keys are cut differently, 5e-7 for the two that are not.)"""
    from qwen3_runtime_amd.llm import LLM

    cfg, folder = sized_folders["qwen3_4b"]
    prompts = list(traces.make_requests(cfg.vocab_size, [70, 20, 5], seed=8).values())

    def run(graph, forced=None):
        llm = LLM(str(folder), dtype="bfloat16", max_num_seqs=4, max_num_batched_tokens=64, block_size=16,
                  num_kv_blocks=64, cuda_graph=graph)
        eng = llm.engine
        reqs = [eng.request(eng.add_request(p, 24, forced_tokens=None if forced is None else forced[i]))
                for i, p in enumerate(prompts)]
        while not eng.is_finished():
            eng.step()
        replayed = bool(eng.runner._graphs)
        out = [r.output_tokens for r in reqs], [r.logprobs for r in reqs]
        del llm, eng
        torch.cuda.empty_cache()
        return out, replayed

    (tokens, logprobs), _ = run(False)
    (again, graph_logprobs), replayed = run(True, forced=tokens)
    assert replayed, "no decode step was replayed from a graph"
    assert again == tokens
    for a, b in zip(graph_logprobs, logprobs):
        torch.testing.assert_close(torch.tensor(a), torch.tensor(b), atol=0.03, rtol=0)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_the_2048_token_prompt_the_measurement_times(sized_folders, dtype):
    """One 2,048-token prompt in one step at the 4B layer sizes, the step whose time is reported as
    prefill throughput: the vendor products at 2,048 rows, the prompt attention through LDS with
    128 row tiles and their work list, the wide q/k kernel. Logits at every 16th position and at
    the last ones against the plain implementation."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    cfg, folder = sized_folders["qwen3_4b"]
    reqs = traces.make_requests(cfg.vocab_size, [2048], seed=44)
    want_all = traces.plain_logits(folder, reqs)
    wanted = sorted(set(range(0, 2048, 16)) | set(range(2040, 2048)))
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": reqs["r0"], "want": wanted}], "end": ["r0"]}]
    engine_cfg = EngineConfig(page_size=16, num_pages=128, max_num_seqs=1, max_num_batched_tokens=2048, dtype=dtype,
                              device="cuda:0", hip_graph=False)
    got = traces.replay(load(folder, engine_cfg), steps)
    want = {("r0", p): want_all[("r0", p)] for p in wanted}
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)
