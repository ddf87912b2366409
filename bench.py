#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-4B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (schedule, graph replay or
launches, sampling, copy of the sampled ids; the engine launches the next
step's kernels while the host waits for the ids, so a window of K steps holds the
device work of K steps, the first of them launched just before the window and the
one after the last inside it). The default run has the layer
sizes of the Qwen3-4B configuration with seeded random weights, bfloat16, a
batch of 8 requests whose prompts are 2,048 uniform-random ids, context limit
8,192, pages of 16 tokens. W untimed steps, then windows of exactly K timed
steps between device synchronisations: three windows, the median one is
reported and the spread of the three beside it (the reference's method: one
warm-up and three trials, median and spread, bench/run_bench.py:164-182,
bench/metrics.py:10-30). Prints one JSON line: ``value`` is decoded tokens per
second at batch 8; ``points`` adds batch 1 and 64 (``point_rooflines`` their
step times and fractions); ``prefill`` is one 2,048-token prompt in one step;
``roofline`` is the decode step's bytes (every weight once plus the cache of
the live requests) over its time, against the published HBM peak, with the
bandwidth and the MFMA rate this device delivered in a microbenchmark beside
the published figures (``measured_peak``).

Other workloads: ``--workload mix`` (continuous batching of ``--requests``
requests with prompts of 128 to 4,096 tokens, portions of 2,048, 256 outputs
each) and any closed batch by ``--preset/--batch/--prompt-len/--context``.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
# the reference's own steady decode rate at batch 8 (RTX 4090, 256-token prompts), for orientation
REFERENCE_4090_B8_TOK_S = 740.0
TRIALS = 3


def say(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def spread(values) -> float:
    """(max - min) / median, as the reference flags unstable trials (bench/metrics.py:10-30)."""
    med = statistics.median(values)
    return round((max(values) - min(values)) / med, 4) if med > 0 else 0.0


def measure_device_peaks(device) -> dict:
    """What this device delivers: GB/s reading 4 GiB once (far beyond every cache), and TFLOP/s
    of bfloat16 32x32x16 MFMA instructions on registers with every SIMD busy. Best of five each."""
    import ctypes

    import torch

    from qwen3_runtime_amd.ops import hip

    lib = hip.load_library("peaks")
    stream = hip.current_stream
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    nbytes = 4 << 30
    buf = torch.zeros(nbytes, dtype=torch.uint8, device=device)

    def timed(launch) -> float:
        best = float("inf")
        for i in range(7):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            code = launch()
            b.record()
            b.synchronize()
            if code != 0:
                raise RuntimeError(lib.qrt_last_error().decode())
            if i >= 2:
                best = min(best, a.elapsed_time(b) * 1e-3)
        return best

    t_read = timed(lambda: lib.qrt_peak_read(ctypes.c_void_p(buf.data_ptr()), ctypes.c_size_t(nbytes),
                                             ctypes.c_void_p(sink.data_ptr()), ctypes.c_int(256 * 64), stream()))
    del buf
    blocks, iters = 256 * 2, 20000
    t_mfma = timed(lambda: lib.qrt_peak_mfma_bf16(ctypes.c_void_p(sink.data_ptr()), ctypes.c_int(blocks),
                                                  ctypes.c_int(iters), stream()))
    torch.cuda.empty_cache()
    return {"hbm_gbs": round(nbytes / t_read / 1e9, 1),
            "mfma_bf16_tflops": round(blocks * 4 * iters * 4 * 32768 / t_mfma / 1e12, 1)}


def sizes_of(raw: dict, limit: int = 12) -> dict:
    """The sizes and switches of a config.json: its integer and boolean entries, without the
    ids of special tokens and the position limit (no sizes of the computation)."""
    skip = ("token_id", "max_position", "max_window", "seed")
    out = {k: v for k, v in raw.items()
           if isinstance(v, (bool, int)) and not any(s in k for s in skip) and (v is not False or k.startswith("tie"))}
    return dict(list(out.items())[:limit])


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default=None, help="default: qwen3_4b (mix: qwen3_8b; capacity: qwen3_32b)")
    ap.add_argument("--batch", type=int, default=None, help="default 8 (capacity: 32)")
    ap.add_argument("--prompt-len", type=int, default=None, help="default 2048 (capacity: 16384)")
    ap.add_argument("--context", type=int, default=None, help="default 8192 (capacity: 32768)")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill measurement")
    ap.add_argument("--no-peaks", action="store_true", help="skip the microbenchmark of the device's own peaks")
    ap.add_argument("--trials", type=int, default=TRIALS, help="timed windows of --steps steps each")
    ap.add_argument("--workload", default="decode", choices=["decode", "mix", "capacity"],
                    help="decode: the closed batch (default). mix: --requests requests with prompts of 128 to 4,096 "
                         "tokens and 256 output tokens each through the scheduler, prompts read in portions of 2,048 "
                         "(the 8B shape unless --preset says otherwise). capacity: the closed batch at the 32B shape, "
                         "32 prompts of 16,384 tokens with room for 512 outputs each in a context of 32,768, decode "
                         "steps only (no batch 1 / 64, no single-prompt prefill; the prompts' reading is prompt_phase)")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--budget", type=int, default=2048, help="tokens per step (max_num_batched_tokens); the workloads "
                                                             "name 2,048")
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure only the 2,048-token prefill (for profiling); prints a reduced line")
    args = ap.parse_args()
    by_workload = {"decode": ("qwen3_4b", 8, 2048, 8192), "mix": ("qwen3_8b", 8, 2048, 8192),
                   "capacity": ("qwen3_32b", 32, 16384, 32768)}[args.workload]
    for name, value in zip(("preset", "batch", "prompt_len", "context"), by_workload):
        if getattr(args, name) is None:
            setattr(args, name, value)
    if args.workload == "capacity":
        args.no_points = True
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine is single-GPU)")
        return 2

    import torch

    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.llm import build_engine
    from qwen3_runtime_amd.registry import preset_config
    from qwen3_runtime_amd.sampling.params import SamplingParams

    # the configuration is a config.json as a dict; nothing below knows which architecture it names:
    # bytes and operations of a step come from the model's parts and the cache manager
    raw_full = preset_config(args.preset)
    raw = dict(raw_full)
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    steps, warmup, trials = args.steps, args.warmup, max(1, args.trials)
    page = 16
    max_batch = args.batch if (args.no_points or args.prefill_only) else max(args.batch, 64)
    mix = args.workload == "mix"
    if mix:
        max_batch = args.requests
    budget = args.budget  # tokens per step
    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    dev_name = "cuda:0"

    peaks = None
    if not args.no_peaks and not args.prefill_only:
        peaks = measure_device_peaks(dev_name)
        say(f"this device: {peaks['hbm_gbs']:.0f} GB/s read, {peaks['mfma_bf16_tflops']:.0f} TFLOP/s bf16 MFMA "
            f"(published: {HBM_PEAK_GBS:.0f} GB/s, {MFMA_PEAK['bf16'] / 1e12:.0f} TFLOP/s)")

    # a request decodes while later ones are still read in: up to this many steps before the timed ones
    lead = lambda batch: batch * -(-args.prompt_len // budget)
    per_req_tokens = args.prompt_len + trials * steps + warmup + lead(max_batch) + 10
    pages = max_batch * (-(-min(per_req_tokens, args.context) // page) + 1)
    if mix:
        pages = max_batch * (-(-(4096 + 256) // page) + 1)
    t0 = time.time()
    engine = build_engine(
        None, config=raw, seed=20260825, dtype=args.dtype, block_size=page, num_kv_blocks=pages,
        max_num_seqs=max_batch, max_num_batched_tokens=budget, max_model_len=args.context,
        cuda_graph=not args.no_graph,
    )
    say(f"model on device in {time.time() - t0:.1f} s, {engine.loaded.weight_bytes / 1e9:.2f} GB of weights, "
        f"{pages} pages")
    dev = engine.runner.device
    gen = torch.Generator().manual_seed(20260825)
    bytes_el = 2 if args.dtype == "bfloat16" else 4
    model, vocab = engine.loaded.model, engine.loaded.model.plan.vocab_size

    def step_bytes_and_flop(spans, rows):
        """What a step over ``spans`` = (tokens of the step, tokens in the cache after it) has to
        read (every weight it uses once: a table that is only looked up counts its rows; and the
        cache of its requests) and to compute, as the model's parts and the cache manager say."""
        cost = model.step_cost(spans, rows, bytes_el)
        return cost.total_weight_bytes + engine.cache.bytes_read([kv for _, kv in spans], bytes_el), cost.flop

    def roofline(step_seconds: float, kv_lens) -> dict:
        nbytes, _ = step_bytes_and_flop([(1, round(kv)) for kv in kv_lens], len(kv_lens))
        achieved = nbytes / step_seconds / 1e9
        out = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": round(achieved / HBM_PEAK_GBS, 4)}
        if peaks:
            out["measured_peak"] = peaks["hbm_gbs"]
            out["frac_of_measured"] = round(achieved / peaks["hbm_gbs"], 4)
        return out

    def decode_run(batch: int, k: int, w: int, n_trials: int):
        """Read ``batch`` prompts in, then ``n_trials`` windows of ``k`` timed decode steps after ``w``
        warm-up steps. Returns the windows as (seconds, tokens each request holds at the window's
        middle), and the time the prompts took."""
        prompts = torch.randint(0, vocab, (batch, args.prompt_len), generator=gen).tolist()
        reqs = [engine.request(engine.add_request(p, max_tokens=n_trials * k + w + lead(batch) + 8,
                                                  sampling=SamplingParams())) for p in prompts]
        torch.cuda.synchronize(dev)
        t = time.perf_counter()
        while any(len(r.token_ids) == r.prompt_len for r in reqs):
            engine.step()  # prompt portions until every request has its first token
        torch.cuda.synchronize(dev)
        fill = time.perf_counter() - t
        for _ in range(w):
            engine.step()
        windows = []
        for _ in range(n_trials):
            torch.cuda.synchronize(dev)
            kv_before = [engine.cache.length(r.request_id) for r in reqs]
            t = time.perf_counter()
            for _ in range(k):
                out = engine.step()
                assert len(out) == batch and all(tok is not None for _, tok, _ in out)
            torch.cuda.synchronize(dev)
            dt = time.perf_counter() - t
            kv_after = [engine.cache.length(r.request_id) for r in reqs]
            windows.append((dt, [(a + b) / 2 for a, b in zip(kv_before, kv_after)]))
        for r in reqs:
            engine.finish_request(r.request_id)
        return windows, fill

    def median_window(windows):
        return sorted(windows)[len(windows) // 2]

    def prefill_run():
        """One 2,048-token prompt through the step function, logits at its last token."""
        tokens = 2048
        ids = torch.randint(0, vocab, (tokens,), generator=gen).tolist()
        times = []
        for i in range(1 + trials):
            rid = f"prefill{i}"
            engine.cache.admit(rid)
            torch.cuda.synchronize(dev)
            t = time.perf_counter()
            engine.runner.step([StepEntry(rid, ids, [tokens - 1])])
            torch.cuda.synchronize(dev)
            times.append(time.perf_counter() - t)
            engine.cache.release(rid)
        timed = times[1:]  # the first is the warm-up
        pt = statistics.median(timed)
        _, flop = step_bytes_and_flop([(tokens, tokens)], 1)
        peak = MFMA_PEAK[dtype_key]
        out = {"value": round(tokens / pt, 1), "tokens": tokens, "ms": round(pt * 1e3, 3),
               "frac": round(flop / pt / peak, 4), "trials": len(timed), "spread": spread(timed)}
        if peaks and dtype_key == "bf16":
            out["measured_peak_tflops"] = peaks["mfma_bf16_tflops"]
            out["frac_of_measured"] = round(flop / pt / (peaks["mfma_bf16_tflops"] * 1e12), 4)
        return out

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s, one 2,048-token prompt", "prefill": prefill_run()}), flush=True)
        return 0

    if mix:
        # continuous batching: every request queued at once, prompts read in portions beside the
        # decoding of those already in
        lengths = torch.randint(128, 4097, (args.requests,), generator=gen).tolist()
        prompts = [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in lengths]
        engine.generate_batch(prompts[:2], max_tokens=8)  # warm-up: libraries, allocator
        torch.cuda.synchronize(dev)
        t = time.perf_counter()
        reqs = [engine.request(engine.add_request(p, max_tokens=256, sampling=SamplingParams())) for p in prompts]
        n_steps = 0
        ran = []  # per step: its spans and the rows it sampled for, priced after the clock stops
        stamps: dict[int, list[float]] = {r.request_id: [] for r in reqs}  # arrival time of every token
        while not engine.is_finished():
            out = engine.step()
            now = time.perf_counter() - t
            ran.append((engine.last_step_stats["spans"], sum(tok is not None for _, tok, _ in out)))
            for rid, tok, _done in out:
                if tok is not None:
                    stamps[rid].append(now)
            n_steps += 1
        torch.cuda.synchronize(dev)
        dt = time.perf_counter() - t
        out_tokens = sum(len(r.output_tokens) for r in reqs)
        floor_s = 0.0  # what the steps that ran would take at the published peaks
        for spans, rows in ran:
            nbytes, flop = step_bytes_and_flop(spans, rows)
            floor_s += max(nbytes / (HBM_PEAK_GBS * 1e9), flop / MFMA_PEAK[dtype_key])
        # the reference's closed-batch figures (qwen3_runtime/serving/slo_harness.py:47-87): time to
        # the first token, time per output token after it, gaps between consecutive tokens
        ttft = sorted(ts[0] for ts in stamps.values())
        tpot = sorted((ts[-1] - ts[0]) / (len(ts) - 1) for ts in stamps.values() if len(ts) > 1)
        itl = sorted(b - a for ts in stamps.values() for a, b in zip(ts, ts[1:]))
        pick = lambda xs, q: round(xs[min(len(xs) - 1, int(q * len(xs)))] * 1e3, 2) if xs else None
        print(json.dumps({
            "metric": f"output tok/s, {args.requests} requests with 128-4,096-token prompts and 256 output tokens each, "
                      f"continuous batching ({args.preset} shape)",
            "value": round(out_tokens / dt, 1), "unit": "tok/s", "n_gpus": 1, "seconds": round(dt, 3),
            "engine_steps": n_steps, "prompt_tokens": sum(lengths), "output_tokens": out_tokens,
            "total_tok_per_s": round((sum(lengths) + out_tokens) / dt, 1),
            "ttft_ms": {"p50": pick(ttft, 0.5), "p99": pick(ttft, 0.99)},
            "tpot_ms": {"p50": pick(tpot, 0.5), "p99": pick(tpot, 0.99)},
            "itl_ms": {"p50": pick(itl, 0.5), "p99": pick(itl, 0.99)},
            # each step priced at max(bytes / HBM peak, flop / MFMA peak), summed, over the time taken
            "roofline": {"bound": "per step: hbm or mfma", "floor_s": round(floor_s, 3), "frac": round(floor_s / dt, 4)},
            "measured_peak": peaks,
            "preemptions": engine.scheduler.num_preemptions, "dtype": dtype_key,
            "data": "synthetic: uniform-random token ids and lengths, seeded random weights",
            "config": {"model": f"{args.preset} shape", "layers": len(model.plan.order), "max_num_seqs": max_batch,
                       "max_num_batched_tokens": budget, "page_size": page, "hip_graph": not args.no_graph},
        }), flush=True)
        return 0

    windows, fill_s = decode_run(args.batch, steps, warmup, trials)
    dt, kv_tokens = median_window(windows)
    ms_per_step = dt / steps * 1e3
    value = args.batch * steps / dt

    points, point_rooflines, prefill = {}, {}, None
    if not args.no_points:
        for b in (1, 64):
            k = min(steps, 64)
            w, _ = decode_run(b, k, min(warmup, 8), trials)
            d, kv = median_window(w)
            points[f"decode_b{b}"] = round(b * k / d, 1)
            r = roofline(d / k, kv)
            point_rooflines[f"decode_b{b}"] = {"ms_per_step": round(d / k * 1e3, 4), "frac": r["frac"],
                                               "achieved_gbs": r["achieved"],
                                               "spread": spread([x[0] for x in w])}
        prefill = prefill_run()

    shape_name = {"qwen3_4b": "Qwen3-4B", "qwen3_8b": "Qwen3-8B", "qwen3_32b": "Qwen3-32B"}.get(args.preset, args.preset)
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({shape_name} shape, {args.prompt_len:,}-token prompts)",
        "value": round(value, 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_key,
        "data": "synthetic: uniform-random token ids, seeded random weights N(0, 0.02), norms 1.0",
        "config": {
            "model": f"{args.preset} shape",
            # every size of the configuration, under config.json's own names
            **sizes_of(raw),
            "layers_of_full_model": raw_full.get("num_hidden_layers", len(model.plan.order)),
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "context_limit": args.context,
            "page_size": page,
            "hip_graph": not args.no_graph,
            "parallelism": "single GPU",
        },
        "trials": {"windows": trials, "steps_each": steps, "reported": "median window",
                   "ms_per_step": [round(w[0] / steps * 1e3, 4) for w in windows],
                   "spread": spread([w[0] for w in windows])},
        "roofline": roofline(dt / steps, kv_tokens),
        # reading the prompts in, portions of 2,048 tokens beside the decoding of those already in
        "prompt_phase": {"tokens": args.batch * args.prompt_len, "seconds": round(fill_s, 3),
                         "tok_s": round(args.batch * args.prompt_len / fill_s, 1)},
        "env": {"gpu": torch.cuda.get_device_name(dev), "torch": torch.__version__, "hip": torch.version.hip,
                "hbm_gib": round(torch.cuda.get_device_properties(dev).total_memory / 2**30, 1)},
    }
    if peaks:
        line["measured_peak"] = peaks
    if args.preset == "qwen3_4b" and args.batch == 8 and args.prompt_len == 2048:
        line["vs_reference_rtx4090_batch8"] = round(value / REFERENCE_4090_B8_TOK_S, 2)
    if prefill is not None:
        line["prefill"] = prefill
        line["points"] = points
        line["point_rooflines"] = point_rooflines
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
