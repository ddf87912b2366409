#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-4B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (schedule, graph replay or
launches, sampling, copy of the sampled ids). The default run has the layer
sizes of the Qwen3-4B configuration with seeded random weights, bfloat16, a
batch of 8 requests whose prompts are 2,048 uniform-random ids, context limit
8,192, pages of 16 tokens. W untimed steps, then exactly K timed steps between
device synchronisations. Prints one JSON line: ``value`` is decoded tokens per
second at batch 8; ``points`` adds batch 1 and 64; ``prefill`` is one
2,048-token prompt in one step; ``roofline`` is the decode step's bytes (every
weight once plus the cache of the live requests) over its time, against the
published HBM peak.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
# the reference's own steady decode rate at batch 8 (RTX 4090, 256-token prompts), for orientation
REFERENCE_4090_B8_TOK_S = 740.0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default="qwen3_4b")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill measurement")
    ap.add_argument("--workload", default="decode", choices=["decode", "mix"],
                    help="decode: the closed batch (default). mix: --requests requests with prompts of 128 to 4,096 "
                         "tokens and 256 output tokens each through the scheduler, prompts read in portions of 2,048")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure only the 2,048-token prefill (for profiling); prints a reduced line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine is single-GPU)")
        return 2

    import dataclasses

    import torch

    from qwen3_runtime_amd.config.presets import preset
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.llm import build_engine
    from qwen3_runtime_amd.sampling.params import SamplingParams

    cfg_full = preset(args.preset)
    cfg = cfg_full if args.layers is None else dataclasses.replace(cfg_full, num_hidden_layers=args.layers)
    steps, warmup = args.steps, args.warmup
    page = 16
    max_batch = args.batch if (args.no_points or args.prefill_only) else max(args.batch, 64)
    mix = args.workload == "mix"
    if mix:
        max_batch = args.requests
    budget = 2048  # tokens per step
    # a request decodes while later ones are still read in: up to this many steps before the timed ones
    lead = lambda batch: batch * -(-args.prompt_len // budget)
    per_req_tokens = args.prompt_len + steps + warmup + lead(max_batch) + 10
    pages = max_batch * (-(-per_req_tokens // page) + 1)
    if mix:
        pages = max_batch * (-(-(4096 + 256) // page) + 1)
    t0 = time.time()
    engine = build_engine(
        None, config=cfg, seed=20260825, dtype=args.dtype, block_size=page, num_kv_blocks=pages,
        max_num_seqs=max_batch, max_num_batched_tokens=budget, max_model_len=args.context,
        cuda_graph=not args.no_graph,
    )
    print(f"[bench] model on device in {time.time() - t0:.1f} s, {engine.loaded.weight_bytes / 1e9:.2f} GB of weights",
          file=sys.stderr, flush=True)
    dev = engine.runner.device
    gen = torch.Generator().manual_seed(20260825)
    bytes_el = 2 if args.dtype == "bfloat16" else 4

    def decode_run(batch: int, k: int, w: int):
        """Prefill ``batch`` prompts, then time ``k`` decode steps after ``w`` warm-up steps."""
        prompts = torch.randint(0, cfg.vocab_size, (batch, args.prompt_len), generator=gen).tolist()
        reqs = [engine.request(engine.add_request(p, max_tokens=k + w + lead(batch) + 8, sampling=SamplingParams()))
                for p in prompts]
        while any(len(r.token_ids) == r.prompt_len for r in reqs):
            engine.step()  # prompt portions until every request has its first token
        for _ in range(w):
            engine.step()
        torch.cuda.synchronize(dev)
        kv_tokens = sum(engine.cache.length(r.request_id) for r in reqs)
        t = time.perf_counter()
        for _ in range(k):
            out = engine.step()
            assert len(out) == batch and all(tok is not None for _, tok, _ in out)
        torch.cuda.synchronize(dev)
        dt = time.perf_counter() - t
        kv_tokens = (kv_tokens + sum(engine.cache.length(r.request_id) for r in reqs)) / 2
        for r in reqs:
            engine.finish_request(r.request_id)
        return dt, kv_tokens

    def prefill_run():
        """One 2,048-token prompt through the step function, logits at its last token."""
        tokens = 2048
        ids = torch.randint(0, cfg.vocab_size, (tokens,), generator=gen).tolist()
        times = []
        for i in range(4):
            rid = f"prefill{i}"
            engine.cache.admit(rid)
            torch.cuda.synchronize(dev)
            t = time.perf_counter()
            engine.runner.step([StepEntry(rid, ids, [tokens - 1])])
            torch.cuda.synchronize(dev)
            times.append(time.perf_counter() - t)
            engine.cache.release(rid)
        pt = min(times[1:])
        lin = 2 * tokens * cfg.num_hidden_layers * (
            cfg.hidden_size * (cfg.q_width + 2 * cfg.kv_width) + cfg.q_width * cfg.hidden_size
            + 3 * cfg.hidden_size * cfg.intermediate_size)
        attn = 2 * cfg.q_width * tokens * tokens * cfg.num_hidden_layers
        head = 2 * cfg.vocab_size * cfg.hidden_size
        peak = MFMA_PEAK["bf16" if args.dtype == "bfloat16" else "fp32"]
        return {"value": round(tokens / pt, 1), "tokens": tokens, "ms": round(pt * 1e3, 3),
                "frac": round((lin + attn + head) / pt / peak, 4)}

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s, one 2,048-token prompt", "prefill": prefill_run()}), flush=True)
        return 0

    if mix:
        # continuous batching: every request queued at once, prompts read in portions beside the
        # decoding of those already in
        lengths = torch.randint(128, 4097, (args.requests,), generator=gen).tolist()
        prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]
        engine.generate_batch(prompts[:2], max_tokens=8)  # warm-up: libraries, allocator
        torch.cuda.synchronize(dev)
        t = time.perf_counter()
        reqs = [engine.request(engine.add_request(p, max_tokens=256, sampling=SamplingParams())) for p in prompts]
        n_steps = 0
        stamps: dict[int, list[float]] = {r.request_id: [] for r in reqs}  # arrival time of every token
        while not engine.is_finished():
            out = engine.step()
            now = time.perf_counter() - t
            for rid, tok, _done in out:
                if tok is not None:
                    stamps[rid].append(now)
            n_steps += 1
        torch.cuda.synchronize(dev)
        dt = time.perf_counter() - t
        out_tokens = sum(len(r.output_tokens) for r in reqs)
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
            "preemptions": engine.scheduler.num_preemptions, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: uniform-random token ids and lengths, seeded random weights",
            "config": {"model": f"{args.preset} shape", "layers": cfg.num_hidden_layers, "max_num_seqs": max_batch,
                       "max_num_batched_tokens": budget, "page_size": page, "hip_graph": not args.no_graph},
        }), flush=True)
        return 0

    dt, kv_tokens = decode_run(args.batch, steps, warmup)
    ms_per_step = dt / steps * 1e3
    value = args.batch * steps / dt
    kv_bytes_per_token = 2 * cfg.num_hidden_layers * cfg.kv_width * bytes_el
    # every weight the step uses, once: the tied table is read once, as the head
    head_bytes = cfg.vocab_size * cfg.hidden_size * bytes_el
    step_weight_bytes = engine.loaded.weight_bytes if cfg.tie_word_embeddings else engine.loaded.weight_bytes - head_bytes
    step_bytes = step_weight_bytes + kv_tokens * kv_bytes_per_token
    achieved = step_bytes / (dt / steps) / 1e9

    points, prefill = {}, None
    if not args.no_points:
        for b in (1, 64):
            k = min(steps, 64)
            d, _ = decode_run(b, k, min(warmup, 8))
            points[f"decode_b{b}"] = round(b * k / d, 1)
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
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform-random token ids, seeded random weights N(0, 0.02), norms 1.0",
        "config": {
            "model": f"{args.preset} shape",
            "layers": cfg.num_hidden_layers,
            "layers_of_full_model": cfg_full.num_hidden_layers,
            "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "tied_head": cfg.tie_word_embeddings,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "context_limit": args.context,
            "page_size": page,
            "hip_graph": not args.no_graph,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if args.preset == "qwen3_4b" and args.batch == 8 and args.prompt_len == 2048:
        line["vs_reference_rtx4090_batch8"] = round(value / REFERENCE_4090_B8_TOK_S, 2)
    if prefill is not None:
        line["prefill"] = prefill
        line["points"] = points
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
