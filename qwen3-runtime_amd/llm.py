"""Python entry point: ``LLM(model).generate(prompts, sampling, max_tokens)``.

Construction, as in the reference's facade (qwen3_runtime/llm.py:87-129):
a path to a model folder loads it; ``None`` builds a small model with seeded
random weights (of a given ``config``, or of the first registered preset).
``generate`` takes a list of token ids and returns the new token ids; a list of
such lists is submitted together and batched continuously (the reference runs
them one after another, qwen3_runtime/llm.py:156-157); a string needs a
tokenizer, or falls back to a character map with the reference's values
(qwen3_runtime/llm.py:131-140). Nothing here names an architecture: a
configuration is a config.json as a dict (or anything with ``to_dict()``), and
the registry finds its model.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Mapping, Sequence

from . import registry
from .config.engine import EngineConfig
from .config.model import read_config_json
from .engine.engine import Engine
from .engine.factory import build_model, load
from .sampling.params import SamplingParams
from .weights import RandomSource


def raw_config_of(config: Any) -> dict:
    """A config.json dict from what a caller may pass as ``config``: None (the first
    registered preset), a preset's name, a dict, or a typed configuration with ``to_dict()``."""
    if config is None or isinstance(config, str):
        return registry.preset_config(config)
    if isinstance(config, Mapping):
        return dict(config)
    if hasattr(config, "to_dict"):
        return dict(config.to_dict())
    raise TypeError(f"config must be a preset name, a dict or have to_dict(); got {type(config).__name__}")


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
        raw = raw_config_of(config)
        _, model = build_model(raw)
        source = RandomSource(model.tensor_decls(), seed, norm_jitter=norm_jitter)
    eos = (raw if raw is not None else read_config_json(model_dir)).get("eos_token_id")
    if isinstance(eos, (list, tuple)):
        eos = eos[0] if eos else None
    engine_cfg = EngineConfig(
        page_size=block_size, num_pages=num_kv_blocks, max_num_seqs=max_num_seqs,
        max_num_batched_tokens=max_num_batched_tokens, eos_token_id=eos, dtype=dtype, device=device,
        max_model_len=max_model_len, hip_graph=True if cuda_graph is None else bool(cuda_graph),
    )
    loaded = load(model_dir, engine_cfg, source=source, raw_config=raw, ops=ops)
    return Engine(engine_cfg, loaded)


def character_ids(text: str, vocab_size: int) -> list[int]:
    """Without a tokenizer a string still has to become ids: character ``c`` becomes
    ``1 + ord(c) % 30``, kept below 32 and below the vocabulary; an empty string is ``[1]``
    (the values of the reference's stand-in, qwen3_runtime/llm.py:131-140)."""
    ceiling = min(31, vocab_size - 1)
    ids = [min(ceiling, 1 + ord(c) % 30) for c in text]
    return ids if ids else [1]


def _is_id_list(x) -> bool:
    return isinstance(x, (list, tuple)) and len(x) > 0 and all(isinstance(t, int) for t in x)


class LLM:
    def __init__(
        self,
        model: str | Path | None = None,
        *,
        tokenizer: Any = None,
        config: Any = None,
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
        """Token ids of one prompt: ids pass through, text goes to the tokenizer or the character map."""
        if _is_id_list(prompt):
            return list(map(int, prompt))
        if not isinstance(prompt, str):
            raise TypeError("prompt must be token ids or a string")
        if self.tokenizer is None:
            return character_ids(prompt, self.vocab_size)
        ids = self.tokenizer.encode(prompt)
        return list(map(int, getattr(ids, "tolist", lambda: ids)()))

    def decode(self, tokens: Sequence[int]) -> str:
        """Text of generated ids; without a tokenizer, the ids themselves, space-separated."""
        if self.tokenizer is not None:
            return self.tokenizer.decode(list(tokens), skip_special_tokens=True)
        return " ".join(map(str, tokens))

    def generate(self, prompts, sampling: SamplingParams | None = None, max_tokens: int = 16):
        """Ids in, ids out; a list of id lists in, a list of id lists out (one batch); text in, text out."""
        options = dict(max_tokens=max_tokens, sampling=sampling if sampling is not None else SamplingParams())
        if isinstance(prompts, (list, tuple)) and prompts and all(_is_id_list(p) for p in prompts):
            return self.engine.generate_batch(prompts, **options)
        if _is_id_list(prompts):
            return self.engine.generate(list(prompts), **options)
        return self.decode(self.engine.generate(self.encode(prompts), **options))
