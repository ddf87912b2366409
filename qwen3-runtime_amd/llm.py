"""Python entry point: ``LLM(model).generate(prompts, sampling, max_tokens)``.

Construction, as in the reference's facade (qwen3_runtime/llm.py:87-129):
a path to a model folder loads it; ``None`` builds a tiny model with seeded
random weights (optionally of a given ``config``). ``generate`` takes a list of
token ids and returns the new token ids; a list of such lists is submitted
together and batched continuously (the reference runs them one after another,
qwen3_runtime/llm.py:156-157); a string needs a tokenizer, or falls back to the
reference's toy character map (qwen3_runtime/llm.py:131-140).
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Sequence

import torch

from .config.engine import EngineConfig
from .config.model import Qwen3Config
from .config.presets import preset
from .engine.engine import Engine
from .engine.factory import build_model, load
from .sampling.params import SamplingParams
from .weights import RandomSource


def build_engine(
    model_dir: str | Path | None,
    *,
    max_num_seqs: int = 8,
    max_num_batched_tokens: int = 2048,
    block_size: int = 16,
    num_kv_blocks: int | None = None,
    dtype: str = "bfloat16",
    device: str = "cuda:0",
    cuda_graph: bool | None = None,
    max_model_len: int | None = None,
    config: Any = None,
    seed: int = 0,
    norm_jitter: float = 0.0,
    ops=None,
) -> Engine:
    """Engine over a model folder, or over random weights of ``config`` when the folder is None.

    Option names follow the reference's factory (qwen3_runtime/engine/factory.py:110-186):
    ``block_size`` is the page size, ``num_kv_blocks`` the number of pages, ``cuda_graph``
    switches the replay of decode steps from captured graphs (HIP graphs here).
    """
    raw = source = None
    if model_dir is None:
        cfg = config or preset("tiny_a")
        raw = cfg.to_dict()
        _, model = build_model(raw)
        source = RandomSource(model.tensor_decls(), seed, norm_jitter=norm_jitter)
    eos = None
    if raw is None:
        from .config.model import read_config_json

        eos = read_config_json(model_dir).get("eos_token_id")
    else:
        eos = raw.get("eos_token_id")
    if isinstance(eos, (list, tuple)):
        eos = eos[0] if eos else None
    engine_cfg = EngineConfig(
        page_size=block_size, num_pages=num_kv_blocks, max_num_seqs=max_num_seqs,
        max_num_batched_tokens=max_num_batched_tokens, eos_token_id=eos, dtype=dtype, device=device,
        max_model_len=max_model_len, hip_graph=True if cuda_graph is None else bool(cuda_graph),
    )
    loaded = load(model_dir, engine_cfg, source=source, raw_config=raw, ops=ops)
    return Engine(engine_cfg, loaded)


class LLM:
    def __init__(
        self,
        model: str | Path | None = None,
        *,
        tokenizer: Any = None,
        config: Qwen3Config | None = None,
        max_num_seqs: int = 4,
        max_num_batched_tokens: int = 256,
        **factory_kwargs,
    ):
        self.tokenizer = tokenizer
        if model is None:
            factory_kwargs.setdefault("num_kv_blocks", 64)
            factory_kwargs.setdefault("norm_jitter", 0.1)
        self.engine = build_engine(
            model, config=config, max_num_seqs=max_num_seqs,
            max_num_batched_tokens=max_num_batched_tokens, **factory_kwargs,
        )
        self.vocab_size = self.engine.runner.vocab_size

    def encode(self, prompt) -> list[int]:
        if isinstance(prompt, list) and prompt and isinstance(prompt[0], int):
            return [int(x) for x in prompt]
        if self.tokenizer is None:
            if isinstance(prompt, str):
                top = min(31, self.vocab_size - 1)
                return [min(top, (ord(ch) % 30) + 1) for ch in prompt] or [1]
            raise TypeError("prompt must be token ids or a string")
        ids = self.tokenizer.encode(prompt)
        return [int(x) for x in (ids.tolist() if hasattr(ids, "tolist") else ids)]

    def decode(self, tokens: Sequence[int]) -> str:
        if self.tokenizer is None:
            return " ".join(str(t) for t in tokens)
        return self.tokenizer.decode(list(tokens), skip_special_tokens=True)

    def generate(self, prompts, sampling: SamplingParams | None = None, max_tokens: int = 16):
        sampling = sampling or SamplingParams()
        if isinstance(prompts, list) and prompts and isinstance(prompts[0], (list, tuple)):
            return self.engine.generate_batch(prompts, max_tokens=max_tokens, sampling=sampling)
        if isinstance(prompts, list) and prompts and isinstance(prompts[0], int):
            return self.engine.generate(prompts, max_tokens=max_tokens, sampling=sampling)
        ids = self.encode(prompts)
        return self.decode(self.engine.generate(ids, max_tokens=max_tokens, sampling=sampling))
