"""Generation through the entry point on the GPU: greedy tokens equal the plain
implementation's, batched continuously or alone, from captured graphs or not, with so
few pages that requests are preempted; the sampler against its plain formulas."""

import math

import pytest
import torch

import traces
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def llm(folder, dtype="float32", page=8, pages=64, seqs=4, budget=64, graph=False):
    from qwen3_runtime_amd.llm import LLM

    return LLM(folder, dtype=dtype, block_size=page, num_kv_blocks=pages, max_num_seqs=seqs,
               max_num_batched_tokens=budget, cuda_graph=graph)


def prompts_for(cfg, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]


@pytest.mark.parametrize("name,lengths,n_out", [("tiny_a", [1, 7, 33, 70], 16), ("tiny_b", [3, 17, 40, 64, 95], 12)])
def test_greedy_generation_equals_plain(model_folders, tiny_configs, name, lengths, n_out):
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg, w = P.read_model(model_folders[name])
    prompts = prompts_for(cfg, lengths)
    want = [P.greedy_generate(cfg, w, p, n_out) for p in prompts]
    page = tiny_configs[name][1]
    m = llm(model_folders[name], page=page, pages=80, budget=24)
    assert m.generate(prompts, SamplingParams(), max_tokens=n_out) == want       # batched together
    assert [m.generate(p, max_tokens=n_out) for p in prompts] == want            # one after another
    m.engine.cache.check()
    assert m.engine.cache.num_free_pages == 80


def test_first_tokens_of_a_sequence(model_folders):
    """Prompts of one and two tokens: position 0 alone, no history at all."""
    cfg, w = P.read_model(model_folders["tiny_a"])
    m = llm(model_folders["tiny_a"], page=16)
    for prompt in ([5], [200, 3]):
        assert m.generate(prompt, max_tokens=5) == P.greedy_generate(cfg, w, prompt, 5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager(model_folders, dtype):
    cfg, _ = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [30, 9, 61], seed=3)
    eager = llm(model_folders["tiny_b"], dtype=dtype, graph=False).generate(prompts, max_tokens=40)
    m = llm(model_folders["tiny_b"], dtype=dtype, graph=True)
    assert m.generate(prompts, max_tokens=40) == eager
    assert m.engine.runner._graphs, "no decode step was replayed from a graph"
    # replays interleaved with eager work and synchronisation give the same again
    torch.cuda.synchronize()
    assert m.generate(prompts, max_tokens=40) == eager


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_before_they_are_asked_for(model_folders, dtype):
    """While the host waits for a decode step's ids the device already runs the next step, if
    nothing can make that step another one. The tokens are those of an engine that never does
    so, also where a launched step is not asked for after all: a request arrives, one is
    cancelled, one may stop at an id, a limit is reached."""
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg, _ = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [30, 9, 61, 5], seed=8)
    params = [SamplingParams(temperature=0.7, seed=40 + i, repetition_penalty=1.2 if i == 1 else 1.0)
              for i in range(4)]

    def run(ahead: bool):
        eng = llm(model_folders["tiny_b"], dtype=dtype, graph=True, pages=128).engine
        eng.runner.repeatable = ahead
        reqs = [eng.request(eng.add_request(prompts[i], 60 - 7 * i, sampling=params[i])) for i in range(2)]
        for _ in range(20):
            eng.step()
        reqs.append(eng.request(eng.add_request(prompts[2], 30, sampling=params[2])))  # arrives in between
        for _ in range(15):
            eng.step()
        eng.finish_request(reqs[1].request_id)                                        # cancelled in between
        for _ in range(5):
            eng.step()
        late = eng.add_request(prompts[3], 25, sampling=params[3], ignore_eos=False, stop_token_ids=(3,))
        reqs.append(eng.request(late))
        while not eng.is_finished():
            eng.step()
        eng.cache.check()
        assert eng.cache.num_free_pages == 128
        return [(r.output_tokens, r.finish_reason) for r in reqs], eng.runner.steps_ahead

    plain_order, none = run(False)
    assert none == [0, 0]
    ahead_order, (launched, taken) = run(True)
    assert ahead_order == plain_order
    assert taken >= 20 and launched > taken, (launched, taken)  # most were asked for, some were not


def test_the_collector_stays_out_of_a_capture(model_folders):
    """An engine with captured graphs, dropped while part of a reference cycle, lives on until the
    collector of cycles runs. If that happened inside a later engine's capture, the old graphs
    would be destroyed while a stream captures, which is an error raised in a destructor: the
    process ends. So the collector is switched off inside every capture (and on again after);
    the garbage goes at the next collection outside one, here by hand at the end."""
    import gc

    cfg, _ = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [12, 5], seed=4)
    first = llm(model_folders["tiny_b"], graph=True)
    want = first.generate(prompts, max_tokens=8)
    assert first.engine.runner._graphs
    cycle = [first]
    cycle.append(cycle)
    del first, cycle

    second = llm(model_folders["tiny_b"], graph=True)
    model = second.engine.runner.model
    forward, seen = model.forward, []

    def forward_and_collect(*args, **kwargs):
        if torch.cuda.is_current_stream_capturing():
            seen.append(gc.isenabled())
        return forward(*args, **kwargs)

    model.forward = forward_and_collect
    assert second.generate(prompts, max_tokens=8) == want
    assert seen and not any(seen), "no capture happened, or the collector was left on inside it"
    assert gc.isenabled()
    gc.collect()  # the first engine's graphs go now, outside any capture
    assert second.generate(prompts, max_tokens=8) == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_across_a_context_bucket(model_folders, dtype):
    """A request that grows past 512 tokens while decoding moves to the graph of the next bucket
    (wider block table, other key splits); a request that ends changes the batch size. The graphs
    are fed the tokens of eager steps and must give them the log-probabilities eager steps gave
    (a graph cuts the keys for its bucket's length, so bfloat16 differs by rounding); in float32
    the tokens chosen freely are the same."""
    cfg, plain_w = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [490, 20, 300], seed=5)
    n_out = (60, 25, 60)

    def run(graph, forced=None):
        m = llm(model_folders["tiny_b"], dtype=dtype, pages=160, budget=128, graph=graph)
        eng = m.engine
        reqs = [eng.request(eng.add_request(p, n, forced_tokens=None if forced is None else forced[i]))
                for i, (p, n) in enumerate(zip(prompts, n_out))]
        while not eng.is_finished():
            eng.step()
        return m, [r.output_tokens for r in reqs], [r.logprobs for r in reqs]

    _, want, want_lp = run(False)
    m, got, got_lp = run(True, forced=want)
    assert got == want
    for p, toks, a, b in zip(prompts, want, got_lp, want_lp):
        if dtype == "float32":
            torch.testing.assert_close(torch.tensor(a), torch.tensor(b), atol=1e-4, rtol=1e-4)
        else:  # both are bfloat16 with other partial sums: rounding noise in units of the logits' deviation
            traces.compare_logprobs(a, b, traces.plain_logprobs(cfg, plain_w, p, toks)[2])
    keys = set(m.engine.runner._graphs)
    assert {key[1] for key in keys} >= {512, 1024} and {key[0] for key in keys} >= {2, 3}
    if dtype == "float32":
        assert run(True)[1] == want


def test_preemption_does_not_change_tokens(model_folders):
    """12 pages of 8 for three requests that need 9 each: some are preempted and recomputed
    (reference: tests/invariance/test_preempt.py:10-33)."""
    cfg, w = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [40, 35, 44], seed=8)
    want = [P.greedy_generate(cfg, w, p, 24) for p in prompts]
    m = llm(model_folders["tiny_b"], page=8, pages=12, seqs=3, budget=32)
    assert m.generate(prompts, max_tokens=24) == want
    assert m.engine.scheduler.num_preemptions >= 1
    m.engine.cache.check()
    assert m.engine.cache.num_free_pages == 12 and m.engine.cache.slots.num_free == 3


@pytest.mark.parametrize("seed,graph", [(0, False), (0, True), (1, True), (2, False), (2, True), (3, True)])
def test_random_traffic_with_few_pages(model_folders, seed, graph):
    """Requests of random lengths arriving at random steps into a pool too small for them:
    portions, decoding, waiting, preemption and recomputation in every order the seed gives.
    Every request ends with the tokens it gets when it runs alone; after every step no page is
    lost or held twice, and at the end all pages and slots are free. With graphs, decode steps
    also reserve the next step's pages ahead, which must change none of this."""
    import random

    rng = random.Random(seed)
    cfg, _ = P.read_model(model_folders["tiny_b"])
    n = 14
    prompts = prompts_for(cfg, [rng.randint(1, 90) for _ in range(n)], seed=seed)
    n_out = [rng.randint(1, 20) for _ in range(n)]
    arrive = sorted(rng.randint(0, 60) for _ in range(n))
    alone = llm(model_folders["tiny_b"], pages=64, graph=False).engine
    want = [alone.generate(p, max_tokens=k) for p, k in zip(prompts, n_out)]
    m = llm(model_folders["tiny_b"], page=8, pages=17, seqs=4, budget=rng.choice([16, 40, 64]), graph=graph)
    eng = m.engine
    reqs, step = {}, 0
    while len(reqs) < n or not eng.is_finished():
        while len(reqs) < n and arrive[len(reqs)] <= step:
            i = len(reqs)
            reqs[i] = eng.request(eng.add_request(prompts[i], n_out[i]))
        eng.step()
        eng.cache.check()
        step += 1
        assert step < 5000, "the engine makes no progress"
    assert [reqs[i].output_tokens for i in range(n)] == want
    assert eng.scheduler.num_preemptions >= 1
    assert eng.cache.num_free_pages == 17 and eng.cache.slots.num_free == 4


@pytest.mark.parametrize("seed", [4])
def test_random_traffic_with_few_pages_in_bfloat16(model_folders, seed):
    """The same traffic in bfloat16 from graphs, in a pool that forces preemptions. Tokens chosen
    freely part ways with the plain model at the first near-tie, so every request is fed the plain
    model's own greedy tokens, and the engine's log-probability of each of them (after portions,
    waiting, preemption and recomputation, from whichever pages it got) has to be the plain one
    up to rounding noise."""
    import random

    rng = random.Random(seed)
    cfg, w = P.read_model(model_folders["tiny_b"])
    n = 12
    prompts = prompts_for(cfg, [rng.randint(1, 90) for _ in range(n)], seed=seed)
    n_out = [rng.randint(2, 20) for _ in range(n)]
    arrive = sorted(rng.randint(0, 50) for _ in range(n))
    want = [P.greedy_generate(cfg, w, p, k) for p, k in zip(prompts, n_out)]
    m = llm(model_folders["tiny_b"], dtype="bfloat16", page=8, pages=17, seqs=4, budget=rng.choice([16, 40, 64]),
            graph=True)
    eng = m.engine
    reqs, step = {}, 0
    while len(reqs) < n or not eng.is_finished():
        while len(reqs) < n and arrive[len(reqs)] <= step:
            i = len(reqs)
            reqs[i] = eng.request(eng.add_request(prompts[i], n_out[i], forced_tokens=want[i]))
        eng.step()
        eng.cache.check()
        step += 1
        assert step < 5000, "the engine makes no progress"
    assert eng.scheduler.num_preemptions >= 1 and eng.runner._graphs
    assert eng.cache.num_free_pages == 17 and eng.cache.slots.num_free == 4
    got_lp, want_lp = [], []
    for i in range(n):
        assert reqs[i].output_tokens == want[i]
        lp, _, std = traces.plain_logprobs(cfg, w, prompts[i], want[i])
        got_lp += reqs[i].logprobs
        want_lp += lp
    traces.compare_logprobs(got_lp, want_lp, std)


def test_engine_refuses_work_after_a_failed_step(model_folders):
    """A step that fails on the device side (forced here from the host: the step function raises)
    leaves cache and device in an unknown state; the engine then refuses steps and requests."""
    from qwen3_runtime_amd.ops.hip import OpsError

    cfg, _ = P.read_model(model_folders["tiny_a"])
    eng = llm(model_folders["tiny_a"], page=16).engine
    prompt = prompts_for(cfg, [9], seed=2)[0]
    assert len(eng.generate(prompt, max_tokens=3)) == 3
    eng.add_request(prompt, 4)
    real = eng.runner.step

    def failing(entries):
        raise OpsError("attention: launch failed (forced by the test)")

    eng.runner.step = failing
    with pytest.raises(OpsError):
        eng.step()
    eng.runner.step = real
    with pytest.raises(RuntimeError, match="engine terminated"):
        eng.step()
    with pytest.raises(RuntimeError, match="engine terminated"):
        eng.add_request(prompt, 2)


def test_requests_arriving_mid_decode_and_seeded_sampling(model_folders):
    """Temperature 0.8 with per-request seeds: tokens do not depend on batch mates or admission time."""
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg, _ = P.read_model(model_folders["tiny_b"])
    prompts = prompts_for(cfg, [3, 17, 40, 64, 95], seed=1)
    params = [SamplingParams(temperature=0.8, seed=100 + i) for i in range(5)]
    m = llm(model_folders["tiny_b"], budget=24, seqs=4, pages=128)
    alone = [m.engine.generate(p, max_tokens=12, sampling=s) for p, s in zip(prompts, params)]
    eng = m.engine
    reqs = [eng.request(eng.add_request(prompts[i], 12, sampling=params[i])) for i in range(2)]
    for _ in range(5):
        eng.step()
    reqs += [eng.request(eng.add_request(prompts[i], 12, sampling=params[i])) for i in range(2, 5)]
    while not eng.is_finished():
        eng.step()
    assert [r.output_tokens for r in reqs] == alone
    assert all(len(r.logprobs) == 12 and all(lp <= 0 for lp in r.logprobs) for r in reqs)
    other = m.engine.generate(prompts[2], max_tokens=12, sampling=SamplingParams(temperature=0.8, seed=999))
    assert other != alone[2]


def test_stop_token_and_forced_tokens(model_folders):
    cfg, w = P.read_model(model_folders["tiny_a"])
    prompt = prompts_for(cfg, [9], seed=2)[0]
    want = P.greedy_generate(cfg, w, prompt, 8)
    eng = llm(model_folders["tiny_a"], page=16).engine
    out = eng.generate(prompt, max_tokens=8, ignore_eos=False, stop_token_ids=(want[3],))
    assert out == want[: want.index(want[3]) + 1]
    forced = [1, 2, 3]
    rid = eng.add_request(prompt, 5, forced_tokens=forced)
    req = eng.request(rid)
    out = list(eng.stream_request(rid))
    assert out[:3] == forced and len(out) == 5
    logits = P.forward(cfg, w, prompt)[-1]
    assert req.logprobs[0] == pytest.approx(float(torch.log_softmax(logits, -1)[1]), abs=1e-4)
    assert out[3:] == P.greedy_generate(cfg, w, prompt + forced, 2)


# ---- the sampling kernel against the plain formulas ---------------------------------------------------
def sample_rows(logits, rows_params, counts_tokens=None):
    """Run the device sampler on [R, V] logits with one SamplingParams per row."""
    from qwen3_runtime_amd.cache import StateSlots
    from qwen3_runtime_amd.ops.hip import HipOps
    from qwen3_runtime_amd.sampling.sampler import Sampler

    r, v = logits.shape
    slots = StateSlots(r, DEV)
    s = Sampler(HipOps(), slots, v, DEV)
    for i, (p, seed) in enumerate(rows_params):
        slot = slots.take(i)
        s.admit(slot, p, seed, (counts_tokens or {}).get(i, []))
    slot_rows = torch.tensor([slots.slot(i) for i in range(r)], dtype=torch.int32, device=DEV)
    return s, slot_rows


class _Req:
    def __init__(self, p):
        self.sampling = p

    def forced_next(self):
        return None


def test_sampler_greedy_ties_and_logprob():
    from qwen3_runtime_amd.sampling.params import SamplingParams

    x = torch.tensor([[1.0, 3.0, 3.0, 2.0], [0.0, 0.0, 0.0, 0.0], [0.0, 4.0, 1.0, 3.0]], device=DEV)
    params = [(SamplingParams(), 0), (SamplingParams(temperature=-1.0), 0), (SamplingParams(), 0)]
    s, rows = sample_rows(x, params)
    tok, lp = s.sample(x, rows, [_Req(p) for p, _ in params])
    assert tok == [1, 0, 1]
    assert lp[2] == pytest.approx(float(torch.log_softmax(x[2].cpu(), -1)[1]), abs=1e-5)


def test_sampler_filters_match_plain_and_draws_follow_the_distribution():
    from qwen3_runtime_amd.sampling.params import SamplingParams

    torch.manual_seed(0)
    v = 1000
    base = (torch.randn(v) * 2.0)
    cases = [
        SamplingParams(temperature=0.7),
        SamplingParams(temperature=1.3, top_k=5),
        SamplingParams(temperature=1.0, top_p=0.6),
        SamplingParams(temperature=0.9, min_p=0.05),
        SamplingParams(temperature=1.1, top_k=50, top_p=0.9, min_p=0.01),
        SamplingParams(temperature=1.0, repetition_penalty=1.7, presence_penalty=0.4, frequency_penalty=0.2),
    ]
    seen = [3, 3, 3, 10, 999, 10, 500]
    n_draws = 4000
    for p in cases:
        x = base.clone().double()
        if p.has_penalties():
            x = P.apply_penalties(x, seen, p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
        x = x / p.temperature
        if p.min_p > 0:
            x = P.min_p_filter(x, p.min_p)
        if p.top_k > 0:
            x = P.top_k_filter(x, p.top_k)
        if p.top_p < 1:
            x = P.top_p_filter(x, p.top_p)
        want = torch.softmax(x, -1)
        logits = base.to(DEV).repeat(n_draws, 1).contiguous()
        params = [(p, 1000 + i) for i in range(n_draws)]
        from qwen3_runtime_amd.cache import StateSlots  # noqa: F401

        s, rows = sample_rows(logits, params, {i: seen for i in range(n_draws)} if p.has_penalties() else None)
        tok, lp = s.sample(logits, rows, [_Req(p)] * n_draws)
        tok_t = torch.tensor(tok)
        assert (want[tok_t] > 0).all(), f"{p}: an id outside the kept set was drawn"
        freq = torch.bincount(tok_t, minlength=v).double() / n_draws
        top = torch.topk(want, 5).indices
        assert (freq[top] - want[top]).abs().max() < 4 * math.sqrt(0.25 / n_draws) + 0.01, str(p)
        got_lp = torch.tensor(lp).double()
        torch.testing.assert_close(got_lp, want[tok_t].log(), atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("v", [8192, 151936, 10001])
def test_sampler_first_pass_in_parts_equals_one_block_per_row(v):
    """Few rows and a large vocabulary: the first pass over a row runs in several blocks. Tokens,
    log-probabilities and processed logits equal those of the one-block path (many rows), greedy
    rows pick torch's first maximum, ties included."""
    from qwen3_runtime_amd.sampling.params import SamplingParams

    torch.manual_seed(3)
    x = (torch.randn(5, v) * 2.0).to(DEV)
    x[1, 77] = x[1, v - 5] = x[1].max() + 1.0          # a tie far apart: the lower id wins
    seen = {i: [3, 3, 77, v - 1, 500] for i in range(5)}
    params = [(SamplingParams(), 0), (SamplingParams(), 0),
              (SamplingParams(temperature=0.8), 11),
              (SamplingParams(temperature=1.2, top_k=40, top_p=0.9), 12),
              (SamplingParams(temperature=0.0, repetition_penalty=1.5, presence_penalty=0.3, frequency_penalty=0.1), 0)]
    reqs = [_Req(p) for p, _ in params]
    s, rows = sample_rows(x, params, seen)
    tok_parts, lp_parts = s.sample(x, rows, reqs)
    # the one-block path: the same five rows among many (parts are used up to 64 rows)
    many = x.repeat(14, 1).contiguous()
    params_many = params * 14
    s2, rows2 = sample_rows(many, params_many, {i: seen[0] for i in range(70)})
    tok_one, lp_one = s2.sample(many, rows2, [_Req(p) for p, _ in params_many])
    if v >= 4096:
        assert min(64, 256 // 5, v // 2048) >= 2       # the first call did run in parts
    assert tok_parts == tok_one[:5]
    torch.testing.assert_close(torch.tensor(lp_parts), torch.tensor(lp_one[:5]), atol=1e-5, rtol=1e-5)
    assert tok_parts[0] == int(torch.argmax(x[0]))
    assert tok_parts[1] == 77
    assert lp_parts[0] == pytest.approx(float(torch.log_softmax(x[0].double(), -1).max()), abs=1e-4)


def test_sampler_is_seeded_and_counter_based():
    from qwen3_runtime_amd.sampling.params import SamplingParams

    torch.manual_seed(1)
    x = torch.randn(6, 500, device=DEV)
    p = SamplingParams(temperature=1.0)
    s1, rows1 = sample_rows(x, [(p, 42)] * 6)
    a1, _ = s1.sample(x, rows1, [_Req(p)] * 6)
    a2, _ = s1.sample(x, rows1, [_Req(p)] * 6)        # second draw of the same requests
    s2, rows2 = sample_rows(x[:3].contiguous(), [(p, 42)] * 3)
    b1, _ = s2.sample(x[:3].contiguous(), rows2, [_Req(p)] * 3)
    b2, _ = s2.sample(x[:3].contiguous(), rows2, [_Req(p)] * 3)
    assert a1[:3] == b1 and a2[:3] == b2               # independent of the batch
    assert a1 != a2                                    # the draw index advances
    top1 = SamplingParams(temperature=1.5, top_k=1)
    s3, rows3 = sample_rows(x, [(top1, 7)] * 6)
    assert s3.sample(x, rows3, [_Req(top1)] * 6)[0] == torch.argmax(x, -1).tolist()


def test_logit_bias_and_penalty_counts_follow_the_output(model_folders):
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg, w = P.read_model(model_folders["tiny_a"])
    prompt = prompts_for(cfg, [6], seed=4)[0]
    eng = llm(model_folders["tiny_a"], page=16).engine
    out = eng.generate(prompt, 3, sampling=SamplingParams(logit_bias={77: 1000.0}))
    assert out == [77, 77, 77]
    # a strong frequency penalty forbids repeats: every output differs, and differs from the prompt
    out = eng.generate(prompt, 20, sampling=SamplingParams(frequency_penalty=1000.0))
    assert len(set(out)) == 20 and not set(out) & set(prompt)
    # plain replay of the same rule
    ids, want = list(prompt), []
    for _ in range(20):
        logits = P.apply_penalties(P.forward(cfg, w, ids)[-1], ids, 1.0, 0.0, 1000.0)
        want.append(P.greedy(logits))
        ids.append(want[-1])
    assert out == want


def test_engine_without_a_page_count(model_folders):
    """``LLM(folder)`` as the README shows it, no ``num_kv_blocks``: the pool is sized from free
    memory, capped by what max_num_seqs requests of the model's position limit can use (a tiny
    model must not claim the device). Generates; every page and slot comes back."""
    from qwen3_runtime_amd.llm import LLM

    cfg, w = P.read_model(model_folders["tiny_b"])
    free_before, _ = torch.cuda.mem_get_info()
    m = LLM(str(model_folders["tiny_b"]), dtype="bfloat16", block_size=8)
    cache = m.engine.cache
    limit = cfg["max_position_embeddings"]
    assert 32 <= cache.num_pages <= 4 * (-(-limit // 8) + 1)
    free_after, _ = torch.cuda.mem_get_info()
    assert free_before - free_after < 2**30, "a tiny model's cache took more than a GiB"
    prompts = prompts_for(cfg, [12, 30], seed=2)
    outs = m.generate(prompts, max_tokens=6)
    assert [len(o) for o in outs] == [6, 6]
    for p, out in zip(prompts, outs):
        traces.check_tokens_chosen_in_bfloat16(cfg, w, p, out)
    # the plain model's own greedy tokens fed through the engine: its log-probabilities of them
    eng = m.engine
    for p in prompts:
        want = P.greedy_generate(cfg, w, p, 6)
        req = eng.request(eng.add_request(p, 6, forced_tokens=want))
        while not eng.is_finished():
            eng.step()
        want_lp, _, std = traces.plain_logprobs(cfg, w, p, want)
        traces.compare_logprobs(req.logprobs, want_lp, std)
    cache.check()
    assert cache.num_free_pages == cache.num_pages and cache.slots.num_free == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line(model_folders, dtype):
    """``python -m qwen3_runtime_amd.cli --model DIR`` as a user runs it, with no page count:
    the ``runtime [...]`` line holds the plain implementation's greedy tokens
    (reference, for the lines it prints: qwen3_runtime/reference/cli.py:51-56)."""
    import ast
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    cfg, w = P.read_model(model_folders["tiny_a"])
    prompt = [5, 17, 3, 250, 9]
    proc = subprocess.run(
        [sys.executable, "-m", "qwen3_runtime_amd.cli", "--model", str(model_folders["tiny_a"]), "--dtype", dtype,
         "--prompt-tokens", *map(str, prompt), "--max-tokens", "6"],
        capture_output=True, text=True, timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = dict(l.split(" ", 1) for l in proc.stdout.splitlines() if " " in l)
    got = ast.literal_eval(lines["runtime"])
    want = P.greedy_generate(cfg, w, prompt, 6)
    if dtype == "float32":
        assert got == want
    else:
        assert len(got) == 6
        traces.check_tokens_chosen_in_bfloat16(cfg, w, prompt, got)
    assert lines["bytes_per_block"] == str(2 * 2 * 2 * 16 * 16 * (4 if dtype == "float32" else 2))
    assert lines["device"] == "cuda:0" and lines["backend"] == "hip" and lines["cuda_graph"] == "True"


def test_graph_buffer_is_repacked_when_a_request_id_comes_back(model_folders):
    """A decode graph keeps the packed block tables of its last step and, when the same request
    ids come one token further, only patches them. A request that was released and admitted again
    under the same id (or restarted after a preemption) owns other pages by then: the kept tables
    must not be trusted. Same id, same length as the graph last saw plus one, other pages."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.engine.factory import load

    cfg, _ = P.read_model(model_folders["tiny_b"])
    ids = prompts_for(cfg, [40], seed=11)[0]
    other = prompts_for(cfg, [40], seed=12)[0]

    def run(graph):
        engine_cfg = EngineConfig(page_size=8, num_pages=10, max_num_seqs=2, dtype="float32", device=DEV,
                                  hip_graph=graph)
        loaded = load(model_folders["tiny_b"], engine_cfg)
        runner, cache = loaded.runner, loaded.cache
        out = []
        cache.admit("a")
        runner.step([StepEntry("a", ids[:30], [])])
        for p in range(30, 34):                      # eager, capture, replays
            out.append(runner.step([StepEntry("a", ids[p: p + 1], [0])])[0].cpu().clone())
        old_pages = list(cache.block_table(0, "a"))
        cache.release("a")
        cache.admit("a")                             # the same id again: the pool hands it other pages
        runner.step([StepEntry("a", ids[:34], [])])  # up to the length the graph saw last
        assert not set(cache.block_table(0, "a")) & set(old_pages)
        cache.admit("squatter")                      # takes the pages "a" held before, and fills them
        runner.step([StepEntry("squatter", other[:36], [])])
        assert set(cache.block_table(0, "squatter")) == set(old_pages)
        for p in range(34, 38):
            out.append(runner.step([StepEntry("a", ids[p: p + 1], [0])])[0].cpu().clone())
        return torch.stack(out), bool(runner._graphs)

    eager, _ = run(False)
    replayed, used = run(True)
    assert used, "no decode step was replayed from a graph"
    torch.testing.assert_close(replayed, eager, atol=2e-5, rtol=2e-5)
    _, w = P.read_model(model_folders["tiny_b"])
    want = P.forward(cfg, w, ids[:38])
    torch.testing.assert_close(replayed, torch.cat([want[30:34], want[34:38]]).float(), atol=5e-5, rtol=5e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_taken_ahead_by_a_replayed_step_go_back_when_another_step_needs_them(model_folders, dtype):
    """While the device runs a replayed decode step, the host takes the pages of the step it
    expects next. With a pool that holds exactly the live tokens, a different next step (another
    request's prompt) finds no page; the pages taken ahead then go back and the step runs."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.engine.factory import load

    cfg, _ = P.read_model(model_folders["tiny_b"])
    ids, other = prompts_for(cfg, [24, 8], seed=21)

    def run(graph):
        loaded = load(model_folders["tiny_b"], EngineConfig(page_size=8, num_pages=3, max_num_seqs=2, dtype=dtype,
                                                            device=DEV, hip_graph=graph))
        runner, cache = loaded.runner, loaded.cache
        out = []
        cache.admit("a")
        runner.step([StepEntry("a", ids[:13], [])])
        for p in range(13, 16):                       # eager, capture, replay: "a" now fills two pages
            out.append(runner.step([StepEntry("a", ids[p: p + 1], [0])])[0].cpu().clone())
        ahead = cache.num_free_pages == 0             # the third page was taken for token 16
        cache.admit("b")
        out.append(runner.step([StepEntry("b", other[:8], [7])])[0].cpu().clone())  # needs that page
        cache.release("b")
        for p in range(16, 19):
            out.append(runner.step([StepEntry("a", ids[p: p + 1], [0])])[0].cpu().clone())
        cache.check()
        return torch.stack(out), ahead

    eager, _ = run(False)
    replayed, ahead = run(True)
    assert ahead, "the replayed step did not take its next page ahead: the case is not met"
    if dtype == "float32":
        torch.testing.assert_close(replayed, eager, atol=2e-5, rtol=2e-5)
    else:  # other key splits under the graph: rounding noise, in units of the logits' spread
        assert float((replayed - eager).pow(2).mean().sqrt() / eager.std()) < 0.015


def test_sampler_with_an_excluded_id():
    """A bias of -inf excludes an id: the row's first value being -inf must not poison the sum
    of exponentials (greedy log-probability) nor be drawn."""
    from qwen3_runtime_amd.sampling.params import SamplingParams

    x = torch.tensor([[2.0, 1.0, 0.5, -1.0] * 64, [0.0, 3.0, 1.0, 2.0] * 64], device=DEV)
    ban = {0: float("-inf"), 4: float("-inf")}
    params = [(SamplingParams(logit_bias=ban), 0), (SamplingParams(temperature=1.0, seed=5, logit_bias={1: float("-inf")}), 5)]
    s, rows = sample_rows(x, params)
    tok, lp = s.sample(x, rows, [_Req(p) for p, _ in params])
    biased = x.clone().cpu()
    biased[0, [0, 4]] = float("-inf")
    biased[1, 1] = float("-inf")
    assert tok[0] == int(biased[0].argmax()) == 8
    assert lp[0] == pytest.approx(float(torch.log_softmax(biased[0], -1)[8]), abs=1e-5)
    assert tok[1] != 1 and math.isfinite(lp[1])
    assert lp[1] == pytest.approx(float(torch.log_softmax(biased[1], -1)[tok[1]]), abs=1e-4)


def test_a_step_launched_ahead_with_other_ids_is_not_the_step_asked_for(model_folders):
    """``ModelRunner.step_ahead`` launches the next decode step with ids on the device; the next
    ``step`` finds its logits computed only if it brings those ids. With other ids it runs as any
    step does, and gives the logits of the ids it was given."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.engine.factory import load

    cfg, w = P.read_model(model_folders["tiny_b"])
    prompt = prompts_for(cfg, [20], seed=3)[0]
    follow = [7, 11, 13, 17, 19, 23]
    loaded = load(model_folders["tiny_b"], EngineConfig(page_size=8, num_pages=16, max_num_seqs=2, dtype="float32",
                                                        device=DEV, hip_graph=True))
    runner = loaded.runner
    loaded.cache.admit("r")
    runner.step([StepEntry("r", prompt, [len(prompt) - 1])])
    got = []
    for i, tok in enumerate(follow):
        got.append(runner.step([StepEntry("r", [tok], [0])])[0].float().cpu())
        if i + 1 < len(follow) and i >= 2:  # graphs replay from the third decode step on
            # odd steps: the ids the next step will bring; even steps: other ids
            fed = follow[i + 1] if i % 2 else (follow[i + 1] + 1) % cfg["vocab_size"]
            assert runner.step_ahead(torch.tensor([fed], dtype=torch.int32, device=DEV))
    launched, taken = runner.steps_ahead
    assert launched == 3 and taken == 1, (launched, taken)
    want = P.forward(cfg, w, prompt + follow)[len(prompt):]
    torch.testing.assert_close(torch.stack(got), want.float(), atol=5e-5, rtol=5e-5)
