"""Trace replay: feed given token ids through the model step by step, write logits.

Reads one JSON object per line from standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry brings a request's next tokens; all entries of a step run as one
batch through the engine's own step function, cache manager and kernels. For a
step that wants logits, ``<out>/<step>.f32`` receives them as little-endian
float32 ``[wanted, vocab]`` in the order of the entries and of ``want``. After
each step a line ``done <step>`` is printed and flushed. Requests named in
``end`` give back what they hold after the step. Nothing is sampled.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

import numpy as np

# a request's tokens are counted in units of this many when --max-tokens is given
CAPACITY_UNIT = 64
MAX_LIVE = 4


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", default=None, help="folder with config.json and model.safetensors")
    ap.add_argument("--preset", default=None,
                    help="instead of --model: seeded random weights of a registered configuration")
    ap.add_argument("--seed", type=int, default=0, help="seed of --preset's weights")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, default=None,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--num-pages", type=int, default=None, help="instead of --max-tokens: pages per cache group")
    ap.add_argument("--page-size", type=int, default=16)
    args = ap.parse_args(argv)

    import torch

    from .config.engine import EngineConfig
    from .engine.batch import StepEntry
    from .engine.factory import load

    if args.page_size < 1 or CAPACITY_UNIT % args.page_size:
        ap.error(f"--page-size must divide {CAPACITY_UNIT}")
    out = Path(args.out)
    out.mkdir(parents=True, exist_ok=True)
    if (args.model is None) == (args.preset is None):
        ap.error("give --model DIR or --preset NAME")
    if (args.max_tokens is None) == (args.num_pages is None):
        ap.error("give --max-tokens N or --num-pages N")
    if args.num_pages is not None:
        num_pages = args.num_pages
    else:
        num_pages = max(1, -(-args.max_tokens // CAPACITY_UNIT)) * (CAPACITY_UNIT // args.page_size)
    engine = EngineConfig(page_size=args.page_size, num_pages=num_pages, max_num_seqs=MAX_LIVE,
                          dtype=args.dtype, device="cuda:0", hip_graph=False)
    print(f"[trace_run] loading {args.model or args.preset} ({args.dtype}, {num_pages} pages of {args.page_size})",
          file=sys.stderr, flush=True)
    if args.preset is not None:
        from .engine.factory import build_model
        from .registry import preset_config
        from .weights import RandomSource

        raw = preset_config(args.preset)
        source = RandomSource(build_model(raw)[1].tensor_decls(), args.seed, norm_jitter=0.1)
        loaded = load(None, engine, source=source, raw_config=raw)
    else:
        loaded = load(args.model, engine)
    runner, cache = loaded.runner, loaded.cache

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = []
        for e in step.get("entries", []):
            rid = e["id"]
            if not cache.has(rid):
                cache.admit(rid)
            entries.append(StepEntry(rid, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                np.ascontiguousarray(arr).tofile(out / f"{step['step']}.f32")
        for rid in step.get("end", []):
            if cache.has(rid):
                cache.release(rid)
        print(f"done {step['step']}", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
