"""Single-GPU inference engine for the Qwen3 dense decoder on AMD MI355X (gfx950).

From a model folder (``config.json`` + ``model.safetensors``) to next tokens:
typed configuration and registry, weights by tensor name, layers assembled
from parts, a paged cache manager, one step function over mixed batches, a
continuous-batching scheduler, sampling, and hand-written HIP kernels.
"""

from .config import EngineConfig, Qwen3Config, preset  # noqa: F401
from .sampling.params import SamplingParams  # noqa: F401

__all__ = ["EngineConfig", "LLM", "Qwen3Config", "SamplingParams", "preset"]


def __getattr__(name):
    if name == "LLM":
        from .llm import LLM

        return LLM
    raise AttributeError(name)
