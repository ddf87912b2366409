"""Run-time settings of an engine, apart from the model's own sizes.

Names and defaults follow the reference's ``Config`` where it has them
(qwen3_runtime/config.py:16-23: ``block_size`` 16, ``max_num_seqs`` 8,
``max_num_batched_tokens`` 2048, ``eos_token_id``); there is no backend switch.
"""

from __future__ import annotations

from dataclasses import dataclass

DTYPES = ("bfloat16", "float32")


@dataclass(frozen=True)
class EngineConfig:
    page_size: int = 16
    # pages per cache group; None sizes the pools from free device memory
    num_pages: int | None = None
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 2048
    eos_token_id: int | None = None
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    # longest sequence a request may reach; None takes the model's position limit
    max_model_len: int | None = None
    # share of the memory free after loading that the cache pools may take
    # (reference: qwen3_runtime/engine/factory.py:94-107 uses 0.85)
    memory_fraction: float = 0.85
    # replay pure-decode steps from captured HIP graphs
    hip_graph: bool = True

    def __post_init__(self) -> None:
        if self.page_size < 1:
            raise ValueError("page_size must be positive")
        if self.num_pages is not None and self.num_pages < 1:
            raise ValueError("num_pages must be positive")
        if self.max_num_seqs < 1:
            raise ValueError("max_num_seqs must be positive")
        if self.max_num_batched_tokens < 1:
            raise ValueError("max_num_batched_tokens must be positive")
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if not 0.0 < self.memory_fraction <= 1.0:
            raise ValueError("memory_fraction must be in (0, 1]")
