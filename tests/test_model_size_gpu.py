"""The engine at the layer sizes of the 4B, 8B and 32B models (two layers, a small vocabulary; one
model of the 4B width six layers deep) against the plain implementation: the kernels'
production paths (few-row products with K cut into planes, the gated epilogue, the products
that share their activations through LDS, decode attention at head size 128 with four and eight
query heads per key head, prompt attention through LDS, the vendor products for long portions)
as parts of a whole model, in float32 and bfloat16, under every way of cutting the requests into
steps.

Weights of these widths are drawn on the device and the plain implementation's float64 torch
routines run there too: the host takes minutes for either."""

import dataclasses

import pytest
import torch

import traces

pytestmark = pytest.mark.gpu

# float32: the longest sums have 12,288 (25,600 at the 32B sizes) terms instead of the tiny models' few hundred.
TOL_F32 = dict(atol=2e-4, rtol=2e-4)
DEVICE = "cuda:0"
# name -> (preset, layers)
MODELS = {"qwen3_4b": ("qwen3_4b", 2), "qwen3_8b": ("qwen3_8b", 2), "qwen3_32b": ("qwen3_32b", 2),
          "deep_4b": ("qwen3_4b", 6)}
CUTS = ["whole", "tail_one_by_one", "portions", "mixed"]

check_rounding_noise = traces.compare_rounding_noise


class _Sized:
    """Model folders and plain results, made when first asked for and kept for the module."""

    def __init__(self, factory):
        self.factory = factory
        self.folders: dict = {}
        self.plain: dict = {}

    def __getitem__(self, name):
        if name not in self.folders:
            from qwen3_runtime_amd.config.presets import preset
            from qwen3_runtime_amd.weights import write_model_folder

            base, layers = MODELS[name]
            cfg = dataclasses.replace(preset(base), num_hidden_layers=layers, vocab_size=2048, eos_token_id=None)
            folder = self.factory.mktemp(name)
            write_model_folder(folder, cfg.to_dict(), seed=21 + list(MODELS).index(name), device=DEVICE)
            self.folders[name] = (cfg, folder)
        return self.folders[name]

    def plain_logits(self, name, lengths, seed, positions=None):
        key = (name, tuple(lengths), seed, None if positions is None else tuple((r, tuple(p)) for r, p in sorted(positions.items())))
        if key not in self.plain:
            cfg, folder = self[name]
            reqs = traces.make_requests(cfg.vocab_size, lengths, seed=seed)
            self.plain[key] = (reqs, traces.plain_logits(folder, reqs, device=DEVICE, positions=positions))
            torch.cuda.empty_cache()
        return self.plain[key]


@pytest.fixture(scope="module")
def sized(tmp_path_factory):
    return _Sized(tmp_path_factory)


def load_sized(folder, steps, dtype, *, page=16, graph=False, max_seqs=4, pages=None, budget=2048):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    engine_cfg = EngineConfig(page_size=page, num_pages=pages or -(-traces.peak_tokens(steps) // page),
                              max_num_seqs=max_seqs, max_num_batched_tokens=budget, dtype=dtype, device=DEVICE,
                              hip_graph=graph)
    return load(folder, engine_cfg)


def test_the_plain_implementation_is_the_same_on_the_device(model_folders, tiny_configs):
    """What the comparisons below lean on: the plain implementation run by torch on the device
    gives the logits it gives on the host (float64 both ways)."""
    cfg, _ = tiny_configs["tiny_b"]
    reqs = traces.make_requests(cfg.vocab_size, [70, 9], seed=3)
    host = traces.plain_logits(model_folders["tiny_b"], reqs)
    device = traces.plain_logits(model_folders["tiny_b"], reqs, device=DEVICE)
    traces.compare(device, host, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", CUTS)
@pytest.mark.parametrize("name", ["qwen3_4b", "qwen3_8b"])
def test_model_sized_layers_match_plain(sized, name, cut, dtype):
    cfg, folder = sized[name]
    reqs, want = sized.plain_logits(name, [150, 41, 9], seed=6)
    steps = getattr(traces, cut)(reqs)
    loaded = load_sized(folder, steps, dtype)
    got = traces.replay(loaded, steps)
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)


@pytest.mark.parametrize("dtype,cut", [("float32", "portions"), ("float32", "tail_one_by_one"), ("bfloat16", "whole"),
                                       ("bfloat16", "tail_one_by_one"), ("bfloat16", "portions"),
                                       ("bfloat16", "mixed")])
def test_32b_layer_sizes(sized, dtype, cut):
    """Width 5,120, 64 query heads on 8 key heads (eight rows of one sequence per decode tile), a
    feed-forward of 25,600 (the down product's K of 25,600 cut into planes, 1,600 gate/up tiles)."""
    cfg, folder = sized["qwen3_32b"]
    reqs, want = sized.plain_logits("qwen3_32b", [150, 41, 9], seed=16)
    steps = getattr(traces, cut)(reqs)
    loaded = load_sized(folder, steps, dtype)
    got = traces.replay(loaded, steps)
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)


@pytest.mark.parametrize("name,live", [("qwen3_4b", 12), ("qwen3_4b", 20), ("qwen3_4b", 40), ("qwen3_4b", 64),
                                       ("qwen3_8b", 33), ("qwen3_32b", 8), ("qwen3_32b", 32), ("qwen3_32b", 100)])
def test_many_requests_decode_together_at_model_sizes(sized, name, live):
    """8 to 100 requests decoding in one step at the models' layer sizes: the products with that
    many rows (the few-row kernel, the kernel that shares activations: whole result, gated, K cut
    into planes; the vendor library beyond 64 or 128 rows), decode attention over many sequences. Prompts in three steps, then six steps with a token of every request, against
    the plain implementation of each request alone."""
    cfg, folder = sized[name]
    lengths = [9 + (5 * i) % 23 for i in range(live)]
    decode = 6
    reqs, want_all = sized.plain_logits(name, lengths, seed=30 + live)
    rids = list(reqs)
    steps = []
    for lo in range(0, live, (live + 2) // 3):
        part = rids[lo: lo + (live + 2) // 3]
        steps.append({"entries": [{"id": r, "tokens": reqs[r][:-decode], "want": [len(reqs[r]) - decode - 1]}
                                  for r in part], "end": []})
    for d in range(decode, 0, -1):
        steps.append({"entries": [{"id": r, "tokens": reqs[r][len(reqs[r]) - d: len(reqs[r]) - d + 1], "want": [0]}
                                  for r in rids], "end": rids if d == 1 else []})
    steps = traces._number(steps)
    loaded = load_sized(folder, steps, "bfloat16", max_seqs=live, pages=live * 3, budget=1024)
    got = traces.replay(loaded, steps)
    assert len(got) == live * (decode + 1)
    check_rounding_noise(got, {k: want_all[k] for k in got})


def test_long_context_decode_beside_a_prompt_portion(sized, monkeypatch):
    """Decoded tokens of a request that holds 1,100 keys in the same steps as portions of another
    request's prompt: attention then runs as two launches (the decode kernel with its keys cut
    over blocks, the prompt kernels for the portion). Against the plain implementation."""
    from qwen3_runtime_amd.ops.hip import HipOps

    cfg, folder = sized["qwen3_4b"]
    reqs, want = sized.plain_logits("qwen3_4b", [1106, 150], seed=12)
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
    got = traces.replay(load_sized(folder, steps, "bfloat16"), steps)
    assert ([0], True) in launches and ([1], False) in launches, "the mixed steps ran as two launches"
    check_rounding_noise(got, {k: want[k] for k in got})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_six_layers_deep(sized, dtype):
    """The 4B width six layers deep, the last 32 tokens of each request decoded one by one from
    replayed HIP graphs: what the rounding of bfloat16 in every layer adds up to through the
    float32 residual stays noise within the bound the two-layer models are held to (measured: an
    rms of 1.0 % of the logits' deviation at two layers, 1.5 % at eight),
    and float32 stays at float32's rounding."""
    cfg, folder = sized["deep_4b"]
    reqs, want = sized.plain_logits("deep_4b", [150, 41, 36], seed=26)
    steps = traces.tail_one_by_one(reqs)
    loaded = load_sized(folder, steps, dtype, graph=True)
    got = traces.replay(loaded, steps)
    assert loaded.runner._graphs, "no decode step was replayed from a graph"
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)


@pytest.mark.parametrize("graph", [False, True])
def test_contexts_of_very_unequal_lengths_decode_in_pieces(sized, graph, monkeypatch):
    """Requests of 2,300, 45 and 260 tokens decode together, eagerly and from replayed graphs: the
    decode attention then cuts the keys into pieces of one length from a list made on the device
    at every step (a captured graph is told the lengths at its capture and shaped for its bucket;
    the lengths go on growing under it). Logits of the last eight tokens of each request against
    the plain implementation."""
    from qwen3_runtime_amd.ops.hip import HipOps

    cfg, folder = sized["qwen3_4b"]
    reqs, want = sized.plain_logits("qwen3_4b", [2300, 45, 260], seed=52)
    rids, decode = list(reqs), 8
    steps = [{"entries": [{"id": r, "tokens": reqs[r][:-decode], "want": [len(reqs[r]) - decode - 1]}], "end": []}
             for r in rids]
    for d in range(decode, 0, -1):
        steps.append({"entries": [{"id": r, "tokens": reqs[r][len(reqs[r]) - d: len(reqs[r]) - d + 1], "want": [0]}
                                  for r in rids], "end": rids if d == 1 else []})
    steps = traces._number(steps)
    pieces = []
    inner = HipOps.choose_decode_piece
    monkeypatch.setattr(HipOps, "choose_decode_piece",
                        lambda self, lens, nkv: (pieces.append(inner(self, lens, nkv)), pieces[-1])[1])
    loaded = load_sized(folder, steps, "bfloat16", graph=graph)
    got = traces.replay(loaded, steps)
    assert pieces and all(p == 512 for p in pieces), "the decode steps were cut into pieces"
    if graph:
        assert any(key[2] for key in loaded.runner._graphs), "a graph for unequal lengths was captured and replayed"
    assert len(got) == 3 * (decode + 1)
    check_rounding_noise(got, {k: want[k] for k in got})


def test_traffic_of_unequal_lengths_through_the_scheduler_from_graphs(sized):
    """Eight requests of 30 to 3,500 prompt tokens arrive one after the other at an engine with
    room for four and a pool that holds the first four prompts and little more; they decode from
    graphs, steps launched ahead, the attention in equal parts or in pieces as the lengths of the
    moment say. Every request is fed given tokens, and the engine's log-probability of each (after
    portions and waiting, beside whichever others were there) has to be the plain
    implementation's up to rounding noise."""
    import random

    from plain import qwen3_plain as P
    from qwen3_runtime_amd.llm import LLM

    cfg, folder = sized["qwen3_4b"]
    rng = random.Random(4)
    lengths = [3500, 40, 900, 2600, 30, 300, 3100, 120]
    prompts = list(traces.make_requests(cfg.vocab_size, lengths, seed=61).values())
    forced = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(6, 20))] for _ in lengths]
    arrive = [0, 0, 1, 3, 6, 9, 12, 20]
    pages = sum(lengths[:4]) // 16 + 6  # the first four prompts and a little: they cannot all grow
    llm = LLM(str(folder), dtype="bfloat16", max_num_seqs=4, max_num_batched_tokens=1024, block_size=16,
              num_kv_blocks=pages, cuda_graph=True)
    eng = llm.engine
    reqs, step = {}, 0
    while len(reqs) < len(lengths) or not eng.is_finished():
        while len(reqs) < len(lengths) and arrive[len(reqs)] <= step:
            i = len(reqs)
            reqs[i] = eng.request(eng.add_request(prompts[i], len(forced[i]), forced_tokens=forced[i]))
        eng.step()
        eng.cache.check()
        step += 1
        assert step < 5000, "the engine makes no progress"
    keys = list(eng.runner._graphs)
    assert any(key[2] for key in keys) and eng.cache.num_free_pages == pages
    assert eng.runner.steps_ahead[1] >= 1, "no step was launched ahead of its turn"
    cfg_plain, w = P.read_model(folder, device=DEVICE)
    got_lp, want_lp = [], []
    for i in range(len(lengths)):
        assert reqs[i].output_tokens == forced[i]
        lp, _, std = traces.plain_logprobs(cfg_plain, w, prompts[i], forced[i])
        got_lp += reqs[i].logprobs
        want_lp += lp
    traces.compare_logprobs(got_lp, want_lp, std)


@pytest.mark.parametrize("lengths", [[70, 20, 5], [2200, 30, 300]])
def test_model_sized_decode_graph_equals_eager(sized, lengths):
    """(The second set of lengths is unequal enough for the decode attention to walk pieces from
    its work list, under graphs whose key says so, with steps launched ahead of their turn.)
    Three requests at the 4B layer sizes, decoded eagerly and then from replayed HIP graphs that
    are fed the eager tokens: at every token the graph's log-probability of it is the eager one up
    to the rounding of bfloat16. (A graph cuts the keys for the length of its bucket, an eager step
    for the length of the step's longest context, so the partial sums of attention are formed in
    another order; random weights make the distribution over 2,048 tokens nearly flat, and tokens
    chosen freely part ways at the first near-tie, which says nothing. Measured difference: 0.01
    for the request whose keys are cut differently, 5e-7 for the two that are not.)"""
    from qwen3_runtime_amd.llm import LLM

    cfg, folder = sized["qwen3_4b"]
    prompts = list(traces.make_requests(cfg.vocab_size, lengths, seed=8).values())

    def run(graph, forced=None):
        llm = LLM(str(folder), dtype="bfloat16", max_num_seqs=4, max_num_batched_tokens=max(64, max(lengths) // 4),
                  block_size=16, num_kv_blocks=64 + sum(lengths) // 16, cuda_graph=graph)
        eng = llm.engine
        reqs = [eng.request(eng.add_request(p, 24, forced_tokens=None if forced is None else forced[i]))
                for i, p in enumerate(prompts)]
        while not eng.is_finished():
            eng.step()
        replayed = bool(eng.runner._graphs) and (max(lengths) < 2048 or any(key[2] for key in eng.runner._graphs))
        out = [r.output_tokens for r in reqs], [r.logprobs for r in reqs]
        del llm, eng
        torch.cuda.empty_cache()
        return out, replayed

    (tokens, logprobs), _ = run(False)
    (again, graph_logprobs), replayed = run(True, forced=tokens)
    assert replayed, "no decode step was replayed from a graph"
    assert again == tokens
    # both are bfloat16 with other partial sums: rounding noise in units of the logits' deviation
    _, want = sized.plain_logits("qwen3_4b", lengths, seed=8)
    std = float(torch.stack(list(want.values())).double().std())
    traces.compare_logprobs([x for lp in graph_logprobs for x in lp], [x for lp in logprobs for x in lp], std)


@pytest.mark.parametrize("name,dtype", [("qwen3_4b", "bfloat16"), ("qwen3_4b", "float32"), ("qwen3_32b", "bfloat16")])
def test_the_2048_token_prompt_the_measurement_times(sized, name, dtype):
    """One 2,048-token prompt in one step, the step whose time is reported as prefill throughput:
    the vendor products at 2,048 rows, the prompt attention through LDS with 128 (256 at the 32B
    sizes) row tiles and their work list, the wide q/k kernel. Logits at every 16th position and
    at the last ones against the plain implementation."""
    cfg, folder = sized[name]
    wanted = sorted(set(range(0, 2048, 16)) | set(range(2040, 2048)))
    reqs, want = sized.plain_logits(name, [2048], seed=44, positions={"r0": wanted})
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": reqs["r0"], "want": wanted}], "end": ["r0"]}]
    got = traces.replay(load_sized(folder, steps, dtype, max_seqs=1), steps)
    if dtype == "float32":
        traces.compare(got, want, **TOL_F32)
    else:
        check_rounding_noise(got, want)
