"""Command line: generate token ids from a model folder or a random-weight preset.

    python -m qwen3_runtime_amd.cli --model DIR --prompt-tokens 151643 8948 198 2610 --max-tokens 8

``--model`` (or ``QWEN3_RUNTIME_MODEL``), ``--max-tokens``, ``--prompt-tokens``,
``--backend`` and ``--cuda-graph/--no-cuda-graph`` keep the reference's names
and meanings (qwen3_runtime/reference/cli.py:18-38); there is one backend,
``hip``. The output lines ``runtime``, ``bytes_per_block``, ``device``,
``backend``, ``cuda_graph`` are the reference's too (cli.py:51-56). There is no
comparison with another library's model here.
"""

from __future__ import annotations

import argparse
import os


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="qwen3_runtime_amd.cli")
    ap.add_argument("--model", default=os.environ.get("QWEN3_RUNTIME_MODEL"))
    ap.add_argument("--preset", default=None, help="random weights of a named configuration instead of --model")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--write-model", default=None, metavar="DIR",
                    help="with --preset: write config.json and model.safetensors there and exit")
    ap.add_argument("--max-tokens", type=int, default=8)
    ap.add_argument("--prompt-tokens", type=int, nargs="+", default=[151643, 8948, 198, 2610])
    ap.add_argument("--prompt-len", type=int, default=None, help="a random prompt of this length instead")
    ap.add_argument("--backend", default="hip", choices=["hip"], help="attention backend; there is one")
    ap.add_argument("--cuda-graph", action=argparse.BooleanOptionalAction, default=None,
                    help="replay decode steps from captured (HIP) graphs; default on")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--sample-seed", type=int, default=None)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-kv-blocks", type=int, default=None)
    ap.add_argument("--max-num-seqs", type=int, default=1)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    args = ap.parse_args(argv)

    from .registry import preset_config
    from .sampling.params import SamplingParams

    if args.write_model:
        if not args.preset:
            ap.error("--write-model needs --preset")
        from .weights import write_model_folder

        print("wrote", write_model_folder(args.write_model, preset_config(args.preset), args.seed))
        return 0
    if not args.model and not args.preset:
        raise SystemExit("set --model or QWEN3_RUNTIME_MODEL (or --preset for random weights)")

    from .cache import CacheManager
    from .llm import build_engine

    engine = build_engine(
        args.model if not args.preset else None,
        config=preset_config(args.preset) if args.preset else None, seed=args.seed,
        max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
        block_size=args.block_size, num_kv_blocks=args.num_kv_blocks, dtype=args.dtype,
        cuda_graph=args.cuda_graph,
    )
    prompt = args.prompt_tokens
    vocab = engine.runner.vocab_size
    if args.prompt_len is not None:
        import random

        rng = random.Random(args.seed)
        prompt = [rng.randrange(vocab) for _ in range(args.prompt_len)]
    elif max(prompt) >= vocab:
        prompt = [t % vocab for t in prompt]
    sampling = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                              min_p=args.min_p, seed=args.sample_seed)
    out = engine.generate(prompt, max_tokens=args.max_tokens, sampling=sampling)
    bytes_per = 2 if args.dtype == "bfloat16" else 4
    print("runtime", out)
    print("bytes_per_block", CacheManager.bytes_per_page(engine.loaded.model.plan.caches, args.block_size, bytes_per))
    print("device", engine.runner.device)
    print("backend", args.backend)
    print("cuda_graph", engine.runner.hip_graph)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
