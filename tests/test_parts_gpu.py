"""Each layer part alone against the plain functions, and the generality of the
assembly: a toy architecture, defined and registered here without touching the
framework's files, with a mixer that keeps state of its own, another position
encoding, a windowed attention layer, a layer that runs twice and a step that
reads another step's cache. It is stepped under every cutting and compared with a
whole-sequence computation written out below."""

import math
from pathlib import Path

import pytest
import torch

import traces
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOY_KERNELS = Path(__file__).resolve().parent / "toy_ops.hip"


class DictFetch:
    """A WeightFetcher over a dict of CPU tensors."""

    def __init__(self, tensors, dtype):
        from qwen3_runtime_amd.weights.loader import WeightLoader

        class Src:
            def get(self, name, device="cpu"):
                # stored in the engine's type, as a model file for that engine would be
                return tensors[name].to(dtype).to(device)

        self.loader = WeightLoader(Src(), DEV, dtype)

    def __getattr__(self, name):
        return getattr(self.loader, name)


def context(q_lens, kv_lens, dtype, page_size=8, window=None, pages_per_seq=None):
    """A StepContext and cache pages for sequences processed whole or with history."""
    from qwen3_runtime_amd.ops.hip import HipOps
    from qwen3_runtime_amd.parts.base import GroupView, StepContext

    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    cu, pos, seq = [0], [], []
    for s, (q, kv) in enumerate(zip(q_lens, kv_lens)):
        cu.append(cu[-1] + q)
        pos += list(range(kv - q, kv))
        seq += [s] * q
    width = max(-(-kv // page_size) for kv in kv_lens)
    table = torch.arange(len(q_lens) * width, dtype=torch.int32).view(len(q_lens), width)
    slots = [int(table[s, p // page_size]) * page_size + p % page_size for s, p in zip(seq, pos)]
    group = GroupView(page_size, window, table.to(DEV), i32(slots))
    return StepContext(
        ops=HipOps(), dtype=dtype, device=torch.device(DEV), num_tokens=len(pos), num_seqs=len(q_lens),
        positions=i32(pos), cu_q=i32(cu), kv_lens=i32(kv_lens), seq_of_token=i32(seq),
        state_slots=i32(list(range(len(q_lens)))), first_span=i32([int(q == kv) for q, kv in zip(q_lens, kv_lens)]),
        q_lens_host=list(q_lens), kv_lens_host=list(kv_lens), max_q_len=max(q_lens), max_kv_len=max(kv_lens),
        groups=[group]), table.numel()


TOL = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=3e-2, rtol=3e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_embedding_head_feed_forward_alone(dtype):
    from qwen3_runtime_amd.parts import build_part
    from qwen3_runtime_amd.parts.plan import PartSpec

    torch.manual_seed(0)
    h, inter, v, t = 96, 272, 384, 11
    w = {"n": 1 + 0.1 * torch.randn(h), "e": 0.5 * torch.randn(v, h), "g": 0.1 * torch.randn(inter, h),
         "u": 0.1 * torch.randn(inter, h), "d": 0.1 * torch.randn(h, inter)}
    w = {k: x.to(torch.bfloat16).float() for k, x in w.items()}
    fetch = DictFetch(w, dtype)
    ctx, _ = context([t], [t], dtype)
    ids = torch.randint(0, v, (t,), dtype=torch.int32, device=DEV)

    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": v, "hidden_size": h}, {"weight": "e"}))
    emb.load(fetch)
    resid = emb.forward(ctx, ids)
    assert resid.dtype == torch.float32
    torch.testing.assert_close(resid.cpu(), w["e"][ids.cpu().long()])

    norm = build_part("norm", PartSpec("rmsnorm", {"size": h, "eps": 1e-5}, {"weight": "n"}))
    norm.load(fetch)
    delta = (0.3 * torch.randn(t, h)).to(dtype).to(DEV)
    before = resid.clone()
    y = norm.forward(ctx, resid, delta)
    summed = before.cpu().double() + delta.cpu().double()
    torch.testing.assert_close(resid.cpu().double(), summed, atol=1e-6, rtol=1e-6)   # the add is float32
    torch.testing.assert_close(y.float().cpu(), P.rms_norm(summed, w["n"].double(), 1e-5).float(), **TOL[dtype])

    ff = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": h, "intermediate_size": inter},
                                             {"gate": "g", "up": "u", "down": "d"}))
    ff.load(fetch)
    x = torch.randn(t, h).to(dtype)
    want = P.feed_forward(x.double(), {"m.gate_proj.weight": w["g"].double(), "m.up_proj.weight": w["u"].double(),
                                       "m.down_proj.weight": w["d"].double()}, "m")
    torch.testing.assert_close(ff.forward(ctx, x.to(DEV)).float().cpu(), want.float(), **TOL[dtype])

    head = build_part("head", PartSpec("linear_head", {"vocab_size": v, "hidden_size": h}, {"weight": "e"}))
    head.load(fetch)
    assert head.weight.data_ptr() == emb.weight.data_ptr()      # tied: one tensor
    logits = head.forward(ctx, x.to(DEV))
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), (x.double() @ w["e"].double().T).float(), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,h,theta,eps", [(4, 2, 16, 64, 1e4, 1e-6), (6, 2, 32, 96, 1e6, 1e-5)])
def test_attention_mixer_alone(dtype, nq, nkv, d, h, theta, eps):
    from qwen3_runtime_amd.parts import build_part
    from qwen3_runtime_amd.parts.base import CacheView
    from qwen3_runtime_amd.parts.plan import PartSpec

    torch.manual_seed(1)
    t, ps = 29, 8
    names = {k: f"a.{k}_proj.weight" for k in "qkvo"} | {"q_norm": "a.q_norm.weight", "k_norm": "a.k_norm.weight"}
    w = {"a.q_proj.weight": torch.randn(nq * d, h) / 8, "a.k_proj.weight": torch.randn(nkv * d, h) / 8,
         "a.v_proj.weight": torch.randn(nkv * d, h) / 8, "a.o_proj.weight": torch.randn(h, nq * d) / 8,
         "a.q_norm.weight": 1 + 0.2 * torch.randn(d), "a.k_norm.weight": 1 + 0.2 * torch.randn(d)}
    w = {k: x.to(torch.bfloat16).float() for k, x in w.items()}
    mixer = build_part("mixer", PartSpec("gqa_attention", {
        "hidden_size": h, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d, "qk_norm_eps": eps,
        "position": PartSpec("rope_neox", {"head_dim": d, "theta": theta})}, names))
    for part in (mixer, mixer.position):
        part.load(DictFetch(w, dtype))
    ctx, n_pages = context([t], [t], dtype, ps)
    spec = mixer.cache_spec()
    cache = CacheView(spec, group=ctx.groups[0],
                      k=torch.zeros(n_pages, nkv, ps, d, dtype=dtype, device=DEV),
                      v=torch.zeros(n_pages, nkv, d, ps, dtype=dtype, device=DEV))
    x = torch.randn(t, h).to(dtype)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, hidden_size=h, rms_norm_eps=eps,
               rope_theta=theta)
    want = P.attention_layer(x.double(), {k: v.double() for k, v in w.items()}, "a", cfg, torch.arange(t))
    got = mixer.forward(ctx, x.to(DEV), cache)
    torch.testing.assert_close(got.float().cpu(), want.float(), **TOL[dtype])


# ------------------------------------------------------------------------------------------------
# A toy architecture, registered from here.
# ------------------------------------------------------------------------------------------------
def register_toy():
    from qwen3_runtime_amd.parts.base import FeedForward, Mixer, PositionEncoding
    from qwen3_runtime_amd.parts.plan import CacheSpec, LayerSpec, ModelPlan, PartSpec, RunStep, TensorDecl
    from qwen3_runtime_amd.registry import register_architecture, register_part

    @register_part("mixer", "toy_ema")
    class EmaMixer(Mixer):
        """state <- decay * state + x_t;  y_t = gain * state.  One float32 vector per request.
        It reads the slots on the host, which a captured graph cannot replay, and says so; and it
        asks for portions of a multiple of four tokens, as a mixer with blocks of its own would."""

        graph_capturable = False
        portion_multiple = 4

        def __init__(self, hidden_size, decay, tensors=None):
            super().__init__(tensors)
            self.hidden_size, self.decay, self.gain = hidden_size, decay, None

        def cache_spec(self):
            return CacheSpec("state", shape=(self.hidden_size,), dtype="float32")

        def tensor_decls(self):
            return [TensorDecl(self._name("gain"), (self.hidden_size,), init="norm")]

        def load(self, fetch):
            self.gain = fetch.vector_f32(self._name("gain"))

        def forward(self, ctx, x, cache):
            out = torch.empty_like(x)
            slots, row = ctx.state_slots.tolist(), 0
            for s, n in enumerate(ctx.q_lens_host):          # tokens of a span in order, state carried on
                state = cache.state[slots[s]]
                for i in range(row, row + n):
                    state = self.decay * state + x[i].float()
                    out[i] = (self.gain * state).to(x.dtype)
                cache.state[slots[s]] = state
                row += n
            return out

    @register_part("position", "toy_scale")
    class ScalePosition(PositionEncoding):
        """q and k are scaled by 1 + rate * position: not a rotation, not fused with anything, and
        computed by a kernel of its own, which the part brings along as a library."""

        def __init__(self, rate, tensors=None):
            from qwen3_runtime_amd.ops import build

            super().__init__(tensors)
            self.rate = rate
            build.register_library("toy_ops", ["runtime.hip", TOY_KERNELS])

        def rotate(self, ctx, q, k):
            from ctypes import c_float, c_int, c_void_p

            from qwen3_runtime_amd.ops import hip

            lib = hip.load_library("toy_ops")
            out = []
            for x in (q, k):
                hip.check_tensor(x, "toy_scale input")
                y = torch.empty_like(x)
                code = lib.toy_scale_by_position(
                    c_void_p(x.data_ptr()), c_void_p(y.data_ptr()), c_void_p(ctx.positions.data_ptr()),
                    c_float(self.rate), c_int(x.shape[0]), c_int(x.shape[1] * x.shape[2]),
                    c_int(0 if x.dtype == torch.float32 else 1), hip.current_stream())
                assert code == 0, lib.qrt_last_error().decode()
                out.append(y)
            return tuple(out)

    @register_part("feed_forward", "toy_routed")
    class RoutedFeedForward(FeedForward):
        """Experts with a router: p = softmax(scale * router x) in float32, an expert's weight is
        max(p - floor, 0) over the sum of these, and an expert runs only over the tokens that give
        it a weight (the weights are continuous in x, so rounding cannot flip a choice)."""

        def __init__(self, hidden_size, intermediate_size, experts, scale, floor, tensors=None):
            super().__init__(tensors)
            self.h, self.i, self.e, self.scale, self.floor = hidden_size, intermediate_size, experts, scale, floor
            self.router, self.gate_up, self.down = None, [], []

        def tensor_decls(self):
            decls = [TensorDecl(self._name("router"), (self.e, self.h))]
            for e in range(self.e):
                decls += [TensorDecl(f"{self._name('expert')}.{e}.gate", (self.i, self.h)),
                          TensorDecl(f"{self._name('expert')}.{e}.up", (self.i, self.h)),
                          TensorDecl(f"{self._name('expert')}.{e}.down", (self.h, self.i))]
            return decls

        def load(self, fetch):
            self.router = fetch.matrix(self._name("router"))
            for e in range(self.e):
                base = f"{self._name('expert')}.{e}"
                self.gate_up.append(fetch.fused([f"{base}.gate", f"{base}.up"], dim=0))
                self.down.append(fetch.matrix(f"{base}.down"))

        def forward(self, ctx, x):
            p = torch.softmax(self.scale * (x.float() @ self.router.float().T), dim=-1)
            w = (p - self.floor).clamp_min(0)
            w = w / w.sum(-1, keepdim=True)
            out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            for e in range(self.e):
                rows = (w[:, e] > 0).nonzero().flatten()
                if rows.numel():
                    act = ctx.ops.gated_linear(x.index_select(0, rows).contiguous(), self.gate_up[e])
                    out.index_add_(0, rows, ctx.ops.linear(act, self.down[e], out_f32=True) * w[rows, e, None])
            return out.to(x.dtype)

    def read_config(raw):
        return dict(raw)

    def make_plan(c):
        h, d = c["hidden_size"], c["head_dim"]

        def norm(name):
            return PartSpec("rmsnorm", {"size": h, "eps": c["eps"]}, {"weight": name})

        def attn(i, nq, nkv, position, window=None):
            p = f"toy.{i}.attn"
            return PartSpec("gqa_attention", {"hidden_size": h, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
                                              "qk_norm_eps": c["eps"], "position": position, "window": window},
                            {k: f"{p}.{k}" for k in ("q", "k", "v", "o", "q_norm", "k_norm")})

        def ff(i):
            return PartSpec("swiglu", {"hidden_size": h, "intermediate_size": c["intermediate_size"]},
                            {k: f"toy.{i}.ff.{k}" for k in ("gate", "up", "down")})

        def routed(i):
            return PartSpec("toy_routed", {"hidden_size": h, "intermediate_size": c["expert_size"], "experts": c["experts"],
                                           "scale": c["router_scale"], "floor": c["router_floor"]},
                            {"router": f"toy.{i}.router", "expert": f"toy.{i}.expert"})

        def layer(i, mixer, feed_forward=None):
            return LayerSpec(PartSpec("pre_norm"), mixer, feed_forward or ff(i),
                             {"input": norm(f"toy.{i}.norm_in"), "post_mixer": norm(f"toy.{i}.norm_post")})

        rope = PartSpec("rope_neox", {"head_dim": d, "theta": c["theta"]})
        layers = [
            layer(0, attn(0, 4, 2, rope)),
            layer(1, PartSpec("toy_ema", {"hidden_size": h, "decay": 0.7}, {"gain": "toy.1.gain"}), routed(1)),
            layer(2, attn(2, 2, 1, PartSpec("toy_scale", {"rate": 0.02}), window=c["window"])),
        ]
        kv = lambda heads, window=None: CacheSpec("paged_kv", heads=heads, head_dim=d, window=window)
        caches = [kv(2), CacheSpec("state", shape=(h,), dtype="float32"), kv(1, c["window"]), kv(2)]
        order = [RunStep(0, 0), RunStep(1, 1), RunStep(2, 2), RunStep(0, 3), RunStep(2, 2, writes_cache=False)]
        sizes = {"vocab_size": c["vocab_size"], "hidden_size": h}
        return ModelPlan(h, c["vocab_size"], c["max_positions"],
                         PartSpec("token_embedding", sizes, {"weight": "toy.embed"}), layers, caches, order,
                         norm("toy.norm"), PartSpec("linear_head", sizes, {"weight": "toy.head"}))

    register_architecture("ToyMixedForCausalLM", read_config, make_plan)


TOY = {"architectures": ["ToyMixedForCausalLM"], "vocab_size": 200, "hidden_size": 48, "head_dim": 16,
       "intermediate_size": 80, "eps": 1e-5, "theta": 5000.0, "window": 11, "max_positions": 512,
       "experts": 3, "expert_size": 48, "router_scale": 30.0, "router_floor": 0.3}


def toy_plain(folder, ids):
    """The toy model on a whole sequence, from the plain functions."""
    c, w = P.read_model(folder)
    t = len(ids)
    pos = torch.arange(t)
    x = w["toy.embed"][torch.as_tensor(ids)]
    kept = {}

    def attn(i, nq, nkv, x, scale_pos, window, reuse=False):
        p, d = f"toy.{i}.attn", c["head_dim"]
        q = P.rms_norm((x @ w[f"{p}.q"].T).view(t, nq, d), w[f"{p}.q_norm"], c["eps"])
        if reuse:
            k, v = kept[i]
        else:
            k = P.rms_norm((x @ w[f"{p}.k"].T).view(t, nkv, d), w[f"{p}.k_norm"], c["eps"])
            v = (x @ w[f"{p}.v"].T).view(t, nkv, d)
        if scale_pos:
            f = (1.0 + 0.02 * pos.double())[:, None, None]
            q = q * f
            k = k if reuse else k * f
        else:
            q = P.rope_neox(q, pos, c["theta"])
            k = k if reuse else P.rope_neox(k, pos, c["theta"])
        kept[i] = (k, v)
        return P.causal_attention(q, k, v, window=window) @ w[f"{p}.o"].T

    def ema(x):
        state, out = torch.zeros(c["hidden_size"]).double(), []
        for i in range(t):
            state = 0.7 * state + x[i]
            out.append(w["toy.1.gain"] * state)
        return torch.stack(out)

    def routed(i, n):
        p = torch.softmax(c["router_scale"] * (n @ w[f"toy.{i}.router"].T), dim=-1)
        wt = (p - c["router_floor"]).clamp_min(0)
        wt = wt / wt.sum(-1, keepdim=True)
        out = torch.zeros_like(n)
        for e in range(c["experts"]):
            ffw = {f"f.{k}_proj.weight": w[f"toy.{i}.expert.{e}.{k}"] for k in ("gate", "up", "down")}
            out = out + wt[:, e, None] * P.feed_forward(n, ffw, "f")
        if t >= 30:  # the routing routes: every expert is left out by some tokens and taken by others
            taken = (wt > 0).sum(0)
            assert bool(((taken > 0) & (taken < t)).all()), taken
        return out

    def block(i, x, mix, routing=False):
        x = x + mix(P.rms_norm(x, w[f"toy.{i}.norm_in"], c["eps"]))
        n = P.rms_norm(x, w[f"toy.{i}.norm_post"], c["eps"])
        if routing:
            return x + routed(i, n)
        ffw = {f"f.{k}_proj.weight": w[f"toy.{i}.ff.{k}"] for k in ("gate", "up", "down")}
        return x + P.feed_forward(n, ffw, "f")

    x = block(0, x, lambda n: attn(0, 4, 2, n, False, None))
    x = block(1, x, ema, routing=True)
    x = block(2, x, lambda n: attn(2, 2, 1, n, True, c["window"]))
    x = block(0, x, lambda n: attn(0, 4, 2, n, False, None))
    x = block(2, x, lambda n: attn(2, 2, 1, n, True, c["window"], reuse=True))
    return P.rms_norm(x, w["toy.norm"], c["eps"]) @ w["toy.head"].T


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from qwen3_runtime_amd.registry import unregister_architecture, unregister_part
    from qwen3_runtime_amd.weights import write_model_folder

    register_toy()
    folder = write_model_folder(tmp_path_factory.mktemp("toy"), TOY, seed=21)
    yield folder
    unregister_architecture("ToyMixedForCausalLM")
    unregister_part("mixer", "toy_ema")
    unregister_part("position", "toy_scale")
    unregister_part("feed_forward", "toy_routed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_toy_architecture_under_every_cutting(toy_folder, cut, dtype):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    reqs = traces.make_requests(TOY["vocab_size"], [5, 37, 64, 90], seed=6)
    steps = getattr(traces, cut)(reqs)
    page = 8
    cfg = EngineConfig(page_size=page, num_pages=traces.peak_tokens(steps) // page, max_num_seqs=4, dtype=dtype,
                       device=DEV, hip_graph=False)
    loaded = load(toy_folder, cfg)
    assert len(loaded.cache.groups) == 2          # two full caches share a pool, the window has its own; state takes no pages
    got = traces.replay(loaded, steps)
    want = {}
    for rid, toks in reqs.items():
        logits = toy_plain(toy_folder, toks)
        for p in range(len(toks)):
            want[(rid, p)] = logits[p].float()
    tol = dict(atol=5e-5, rtol=5e-5) if dtype == "float32" else dict(atol=4e-2, rtol=4e-2)
    traces.compare(got, want, **tol)


def test_window_layer_gives_pages_back_while_decoding(toy_folder):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.engine.factory import load

    cfg = EngineConfig(page_size=8, num_pages=16, max_num_seqs=2, dtype="float32", device=DEV, hip_graph=False)
    loaded = load(toy_folder, cfg)
    cache = loaded.cache
    win = next(i for i, g in enumerate(cache.groups) if g.window is not None)
    cache.admit("r")
    ids = traces.make_requests(TOY["vocab_size"], [100], seed=1)["r0"]
    got = [loaded.runner.step([StepEntry("r", ids[:60], [59])])[0].cpu()]
    for p in range(60, 100):
        got.append(loaded.runner.step([StepEntry("r", ids[p: p + 1], [0])])[0].cpu())
    held = [p for p in cache.block_table(win, "r") if p >= 0]
    assert len(held) <= TOY["window"] // 8 + 2 and cache.block_table(win, "r")[0] == -1
    want = toy_plain(toy_folder, ids)
    torch.testing.assert_close(torch.stack(got), want[59:].float(), atol=5e-5, rtol=5e-5)
    cache.release("r")
    cache.check()


def test_toy_architecture_with_graphs_asked_for(toy_folder):
    """HIP graphs are asked for, but the toy's state mixer declares that it cannot be captured:
    the runner then steps eagerly, with no change to the package, and the logits are right."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    reqs = traces.make_requests(TOY["vocab_size"], [45], seed=3)
    steps = traces.tail_one_by_one(reqs, tail=20)
    cfg = EngineConfig(page_size=8, num_pages=8, max_num_seqs=2, dtype="float32", device=DEV, hip_graph=True)
    loaded = load(toy_folder, cfg)
    assert not loaded.model.graph_capturable and not loaded.runner.hip_graph
    got = traces.replay(loaded, steps)
    logits = toy_plain(toy_folder, reqs["r0"])
    traces.compare(got, {("r0", p): logits[p].float() for p in range(45)}, atol=5e-5, rtol=5e-5)


def test_toy_architecture_generates_through_the_engine_in_portions_it_asked_for(toy_folder):
    """Through scheduler and sampler: the toy's mixer wants portions of a multiple of four tokens,
    the token limit is 10, so prompts advance by 8 until their last portion; greedy tokens equal
    the whole-sequence computation's."""
    from qwen3_runtime_amd.llm import build_engine

    eng = build_engine(str(toy_folder), block_size=8, num_kv_blocks=24, max_num_seqs=2, max_num_batched_tokens=10,
                       dtype="float32", device=DEV, cuda_graph=True)
    assert eng.scheduler.portion_multiple == 4
    prompts = list(traces.make_requests(TOY["vocab_size"], [23, 9], seed=4).values())
    inner, log = eng.scheduler.schedule, []

    def spy():
        batch = inner()
        log.extend((r.grant, eng.scheduler.behind(r)) for r in batch)  # before the step: what it gets, what it lacks
        return batch

    eng.scheduler.schedule = spy
    outs = eng.generate_batch(prompts, max_tokens=5)
    cut = [g for g, lacking in log if g < lacking]
    assert cut and all(g % 4 == 0 for g in cut), log
    for p, out in zip(prompts, outs):
        ids = list(p)
        for _ in range(5):
            ids.append(int(toy_plain(toy_folder, ids)[-1].argmax()))
        assert out == ids[len(p):]


def test_toy_architecture_from_its_configuration_alone(toy_folder):
    """``build_engine(None, config=...)`` with the toy's config.json as a dict (no folder, no typed
    configuration class, no preset): seeded random weights on the device, generation through
    scheduler and sampler, and what a measurement needs (bytes a step reads, its operations) from
    the parts and the cache manager, with no edit in the package."""
    from qwen3_runtime_amd.llm import build_engine
    from qwen3_runtime_amd.weights import RandomSource

    eng = build_engine(None, config=TOY, seed=5, norm_jitter=0.1, block_size=8, num_kv_blocks=24, max_num_seqs=2,
                       max_num_batched_tokens=32, dtype="float32", device=DEV)
    prompts = list(traces.make_requests(TOY["vocab_size"], [21, 6], seed=9).values())
    outs = eng.generate_batch(prompts, max_tokens=4)
    # the same weights, written to a folder, through the plain computation
    model = eng.loaded.model
    src = RandomSource(model.tensor_decls(), 5, norm_jitter=0.1)
    import json
    import tempfile

    from safetensors.torch import save_file

    with tempfile.TemporaryDirectory() as folder:
        # drawn where the engine drew them: a seed's values differ between devices
        save_file({d.file_name: src.get(d.file_name, DEV).cpu().contiguous() for d in model.tensor_decls()},
                  f"{folder}/model.safetensors")
        Path(folder, "config.json").write_text(json.dumps(TOY))
        for p, out in zip(prompts, outs):
            ids = list(p)
            for _ in range(4):
                ids.append(int(toy_plain(folder, ids)[-1].argmax()))
            assert out == ids[len(p):]
    # a decode step of two requests that hold 30 and 9 tokens
    spans = [(1, 30), (1, 9)]
    cost = model.step_cost(spans, rows=2, elem_bytes=4)
    h, d, v, inter = TOY["hidden_size"], TOY["head_dim"], TOY["vocab_size"], TOY["intermediate_size"]
    attn0 = (4 + 2 + 2) * d * h + h * 4 * d
    attn2 = (2 + 1 + 1) * d * h + h * 2 * d
    ff = 3 * h * inter
    experts = TOY["experts"] * (h + 3 * h * TOY["expert_size"])
    # layers 0 and 2 run twice: their matrices are read once and multiply twice; the embedding is
    # looked up (two rows), the head multiplies the two wanted rows
    want_flop = 2 * 2 * (2 * (attn0 + ff) + 2 * (attn2 + ff) + experts) + 2 * 2 * v * h
    want_flop += 4 * d * (2 * 4 * (30 + 9) + 2 * 2 * (min(30, TOY["window"]) + min(9, TOY["window"])))
    assert cost.flop == pytest.approx(want_flop)
    norms = 4 * (6 * h + 4 * d + h) + 4 * h          # norm vectors, q/k norms, the toy mixer's gain, final norm
    assert cost.total_weight_bytes == 4 * (attn0 + attn2 + 2 * ff + experts + v * h + 2 * h) + norms
    # the cache: two full groups' worth of keys and values, a window, one state per request
    read = eng.cache.bytes_read([30, 9], 4)
    assert read == 4 * (2 * (2 * 2 * d) * 39 + (2 * 1 * d) * (11 + 9)) + 2 * h * 4


# ------------------------------------------------------------------------------------------------
# A mixer whose paged cache is neither keys nor values: one latent vector per token.
# ------------------------------------------------------------------------------------------------
LATENT = {"architectures": ["ToyLatentForCausalLM"], "vocab_size": 90, "hidden_size": 32, "latent": 12,
          "intermediate_size": 48, "eps": 1e-5, "max_positions": 256}


@pytest.fixture(scope="module")
def latent_folder(tmp_path_factory):
    from qwen3_runtime_amd.parts.base import Mixer
    from qwen3_runtime_amd.parts.plan import (CacheSpec, LayerSpec, ModelPlan, PagedStream, PartSpec, RunStep,
                                              TensorDecl)
    from qwen3_runtime_amd.registry import (register_architecture, register_part, unregister_architecture,
                                            unregister_part)
    from qwen3_runtime_amd.weights import write_model_folder

    @register_part("mixer", "toy_latent")
    class LatentMixer(Mixer):
        """c_t = W_in x_t is stored per token in pages of its own (one stream, no keys, no values);
        y_t = W_out mean(c_0 .. c_t). It gathers with torch on the host's say-so, so no graph."""

        graph_capturable = False

        def __init__(self, hidden_size, latent, tensors=None):
            super().__init__(tensors)
            self.h, self.r = hidden_size, latent

        def cache_spec(self):
            return CacheSpec("paged", streams=(PagedStream("latent", 1, self.r),))

        def tensor_decls(self):
            return [TensorDecl(self._name("in"), (self.r, self.h)), TensorDecl(self._name("out"), (self.h, self.r))]

        def load(self, fetch):
            self.w_in, self.w_out = fetch.matrix(self._name("in")), fetch.matrix(self._name("out"))

        def forward(self, ctx, x, cache):
            latent = ctx.ops.linear(x, self.w_in)
            pages = cache.pages["latent"]                         # [pages, 1, page_size, r]
            ps = cache.group.page_size
            flat = pages.view(-1, self.r)
            flat.index_copy_(0, cache.group.slots.long(), latent.to(flat.dtype))
            mean = torch.empty((ctx.num_tokens, self.r), dtype=torch.float32, device=x.device)
            row = 0
            for s, (q, kv) in enumerate(zip(ctx.q_lens_host, ctx.kv_lens_host)):
                pos = torch.arange(kv, device=x.device)
                places = cache.group.block_table[s, pos // ps].long() * ps + pos % ps
                sums = flat[places].float().cumsum(0)
                mean[row: row + q] = sums[kv - q:] / (pos[kv - q:] + 1)[:, None]
                row += q
            return ctx.ops.linear(mean.to(x.dtype), self.w_out)

    def make_plan(c):
        h = c["hidden_size"]
        norm = lambda name: PartSpec("rmsnorm", {"size": h, "eps": c["eps"]}, {"weight": name})
        layers, caches, order = [], [], []
        for i in range(2):
            mixer = PartSpec("toy_latent", {"hidden_size": h, "latent": c["latent"]},
                             {"in": f"lat.{i}.in", "out": f"lat.{i}.out"})
            ff = PartSpec("swiglu", {"hidden_size": h, "intermediate_size": c["intermediate_size"]},
                          {k: f"lat.{i}.ff.{k}" for k in ("gate", "up", "down")})
            layers.append(LayerSpec(PartSpec("pre_norm"), mixer, ff,
                                    {"input": norm(f"lat.{i}.norm_in"), "post_mixer": norm(f"lat.{i}.norm_post")}))
            caches.append(CacheSpec("paged", streams=(PagedStream("latent", 1, c["latent"]),)))
            order.append(RunStep(i, i))
        sizes = {"vocab_size": c["vocab_size"], "hidden_size": h}
        return ModelPlan(h, c["vocab_size"], c["max_positions"],
                         PartSpec("token_embedding", sizes, {"weight": "lat.embed"}), layers, caches, order,
                         norm("lat.norm"), PartSpec("linear_head", sizes, {"weight": "lat.embed"}))

    register_architecture("ToyLatentForCausalLM", dict, make_plan)
    folder = write_model_folder(tmp_path_factory.mktemp("latent"), LATENT, seed=3)
    yield folder
    unregister_architecture("ToyLatentForCausalLM")
    unregister_part("mixer", "toy_latent")


def latent_plain(folder, ids):
    c, w = P.read_model(folder)
    x = w["lat.embed"][torch.as_tensor(ids)]
    steps = torch.arange(1, len(ids) + 1).double()[:, None]
    for i in range(2):
        n = P.rms_norm(x, w[f"lat.{i}.norm_in"], c["eps"])
        x = x + ((n @ w[f"lat.{i}.in"].T).cumsum(0) / steps) @ w[f"lat.{i}.out"].T
        n = P.rms_norm(x, w[f"lat.{i}.norm_post"], c["eps"])
        x = x + P.feed_forward(n, {f"f.{k}_proj.weight": w[f"lat.{i}.ff.{k}"] for k in ("gate", "up", "down")}, "f")
    return P.rms_norm(x, w["lat.norm"], c["eps"]) @ w["lat.embed"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_paged_cache_of_latent_vectors(latent_folder, dtype):
    """The cache manager pages whatever per-token tensors a mixer's ``CacheSpec`` names: block
    tables, slots, reuse of pages and the step function are those of keys and values. Mixed
    steps in a pool at its peak, against the whole-sequence computation."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    reqs = traces.make_requests(LATENT["vocab_size"], [30, 7, 52, 18, 41, 9], seed=2)
    steps = traces.mixed(reqs, seed=1, max_live=3)
    page = 8
    pages = traces.peak_tokens(steps, unit=page) // page
    assert pages < sum(-(-len(t) // page) for t in reqs.values())
    loaded = load(latent_folder, EngineConfig(page_size=page, num_pages=pages, max_num_seqs=3, dtype=dtype, device=DEV))
    assert not loaded.runner.hip_graph and loaded.runner.repeatable
    assert loaded.cache.bytes_per_page(loaded.model.plan.caches, page, 2) == 2 * 12 * page * 2
    got = traces.replay(loaded, steps, poison_freed=True)
    want = {(rid, p): row.float() for rid, toks in reqs.items() for p, row in enumerate(latent_plain(latent_folder, toks))}
    if dtype == "float32":
        traces.compare(got, want, atol=5e-5, rtol=5e-5)
    else:
        traces.compare_rounding_noise(got, want)


# ------------------------------------------------------------------------------------------------
# A third toy: a norm and an arrangement of the block of its own, around the framework's attention
# and feed-forward.
# ------------------------------------------------------------------------------------------------
PARALLEL = {"architectures": ["ToyParallelForCausalLM"], "vocab_size": 150, "hidden_size": 64, "head_dim": 16,
            "heads": 4, "kv_heads": 2, "intermediate_size": 96, "eps": 1e-5, "theta": 20000.0, "max_positions": 256}


@pytest.fixture(scope="module")
def parallel_folder(tmp_path_factory):
    from qwen3_runtime_amd.parts.base import Block, Norm
    from qwen3_runtime_amd.parts.plan import CacheSpec, LayerSpec, ModelPlan, PartSpec, RunStep, TensorDecl
    from qwen3_runtime_amd.registry import (register_architecture, register_part, unregister_architecture,
                                            unregister_part)
    from qwen3_runtime_amd.weights import write_model_folder

    @register_part("norm", "toy_centered")
    class CenteredNorm(Norm):
        """y = c * rsqrt(mean(c^2) + eps) * w with c = x - mean(x): the mean goes too, unlike RMSNorm.
        In float32, in torch; it adds what is pending into the residual stream first, as any norm
        here does (one matrix or several planes), and normalises only the rows asked for."""

        def __init__(self, size, eps, tensors=None):
            super().__init__(tensors)
            self.size, self.eps, self.weight = size, eps, None

        def tensor_decls(self):
            return [TensorDecl(self._name("weight"), (self.size,), init="norm")]

        def load(self, fetch):
            self.weight = fetch.vector_f32(self._name("weight"))

        def forward(self, ctx, residual, delta=None, rows=None):
            pending = None if delta is None else (delta.sum(0) if delta.dim() == 3 else delta.float())
            if rows is None:
                if pending is not None:
                    residual.add_(pending)
                x = residual
            else:
                x = residual.index_select(0, rows.long())
                if pending is not None:
                    x = x + pending.index_select(0, rows.long())
            c = x - x.mean(-1, keepdim=True)
            return (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight).to(ctx.dtype)

    @register_part("block", "toy_parallel")
    class ParallelBlock(Block):
        """x += mixer(n) + feed_forward(n), n = norm(x): one norm, both sub-layers read it, and what
        they give is handed on as one pending sum for the next norm to add."""

        norm_names = ("input",)

        def __init__(self, mixer, feed_forward, norms, tensors=None):
            super().__init__(tensors)
            self.mixer, self.feed_forward, self.norm_in = mixer, feed_forward, norms["input"]

        def children(self):
            return (self.norm_in, self.mixer, self.feed_forward)

        def forward(self, ctx, residual, delta, cache):
            n = self.norm_in.forward(ctx, residual, delta)
            whole = lambda d: d.sum(0) if d.dim() == 3 else d.float()   # planes of a product cut along K
            return residual, whole(self.mixer.forward(ctx, n, cache)) + whole(self.feed_forward.forward(ctx, n))

    def make_plan(c):
        h, d = c["hidden_size"], c["head_dim"]
        centered = lambda name: PartSpec("toy_centered", {"size": h, "eps": c["eps"]}, {"weight": name})
        rope = PartSpec("rope_neox", {"head_dim": d, "theta": c["theta"]})
        layers, caches, order = [], [], []
        for i in range(3):
            attn = PartSpec("gqa_attention", {"hidden_size": h, "num_heads": c["heads"], "num_kv_heads": c["kv_heads"],
                                              "head_dim": d, "qk_norm_eps": c["eps"], "position": rope, "window": None},
                            {k: f"par.{i}.attn.{k}" for k in ("q", "k", "v", "o", "q_norm", "k_norm")})
            ff = PartSpec("swiglu", {"hidden_size": h, "intermediate_size": c["intermediate_size"]},
                          {k: f"par.{i}.ff.{k}" for k in ("gate", "up", "down")})
            layers.append(LayerSpec(PartSpec("toy_parallel"), attn, ff, {"input": centered(f"par.{i}.norm")}))
            caches.append(CacheSpec("paged_kv", heads=c["kv_heads"], head_dim=d))
            order.append(RunStep(i, i))
        sizes = {"vocab_size": c["vocab_size"], "hidden_size": h}
        return ModelPlan(h, c["vocab_size"], c["max_positions"],
                         PartSpec("token_embedding", sizes, {"weight": "par.embed"}), layers, caches, order,
                         centered("par.norm"), PartSpec("linear_head", sizes, {"weight": "par.head"}))

    register_architecture("ToyParallelForCausalLM", dict, make_plan)
    folder = write_model_folder(tmp_path_factory.mktemp("parallel"), PARALLEL, seed=13, norm_jitter=0.2)
    yield folder
    unregister_architecture("ToyParallelForCausalLM")
    unregister_part("block", "toy_parallel")
    unregister_part("norm", "toy_centered")


def parallel_plain(folder, ids):
    c, w = P.read_model(folder)
    t, d, nq, nkv = len(ids), c["head_dim"], c["heads"], c["kv_heads"]
    pos = torch.arange(t)

    def centered(x, weight):
        x = x - x.mean(-1, keepdim=True)
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + c["eps"]) * weight

    x = w["par.embed"][torch.as_tensor(ids)]
    for i in range(3):
        n, p = centered(x, w[f"par.{i}.norm"]), f"par.{i}.attn"
        q = P.rope_neox(P.rms_norm((n @ w[f"{p}.q"].T).view(t, nq, d), w[f"{p}.q_norm"], c["eps"]), pos, c["theta"])
        k = P.rope_neox(P.rms_norm((n @ w[f"{p}.k"].T).view(t, nkv, d), w[f"{p}.k_norm"], c["eps"]), pos, c["theta"])
        v = (n @ w[f"{p}.v"].T).view(t, nkv, d)
        ffw = {f"f.{k}_proj.weight": w[f"par.{i}.ff.{k}"] for k in ("gate", "up", "down")}
        x = x + P.causal_attention(q, k, v) @ w[f"{p}.o"].T + P.feed_forward(n, ffw, "f")
    return centered(x, w["par.norm"]) @ w["par.head"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_a_norm_and_a_block_arrangement_of_their_own(parallel_folder, cut, dtype):
    """A norm that also takes the mean away and a block in which mixer and feed-forward read one
    normalised input and their outputs are added together, both defined here: registered, built
    from a plan, loaded, and stepped under every way of cutting (decode steps from HIP graphs:
    nothing in these parts stands in a capture's way), around the framework's own attention and
    feed-forward, whose kernels run unchanged."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load

    reqs = traces.make_requests(PARALLEL["vocab_size"], [70, 9, 41, 33], seed=4)
    steps = getattr(traces, cut)(reqs)
    page = 8
    loaded = load(parallel_folder, EngineConfig(page_size=page, num_pages=-(-traces.peak_tokens(steps, unit=page) // page),
                                                max_num_seqs=4, dtype=dtype, device=DEV, hip_graph=True))
    got = traces.replay(loaded, steps)
    assert loaded.runner.hip_graph and (cut != "tail_one_by_one" or loaded.runner._graphs)
    want = {(rid, p): row.float() for rid, toks in reqs.items() for p, row in enumerate(parallel_plain(parallel_folder, toks))}
    if dtype == "float32":
        traces.compare(got, want, atol=5e-5, rtol=5e-5)
    else:
        traces.compare_rounding_noise(got, want)
