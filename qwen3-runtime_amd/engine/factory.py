"""From a model folder to a model on the device with its cache and step function.

The architecture named in ``config.json`` picks the configuration class and
the plan; nothing here knows which model it builds. The number of pages is
either given or derived from the memory that is free once the weights are
loaded (reference: qwen3_runtime/engine/factory.py:75-107, 85 % of free
memory, at least 32 pages).
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path

import torch

from ..cache import CacheManager
from ..config.engine import EngineConfig
from ..config.model import read_config_json
from ..parts.model import DecoderModel
from ..registry import architecture_for
from ..weights import SafetensorsSource, load_model
from .runner import ModelRunner

TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class LoadedModel:
    config: object
    model: DecoderModel
    cache: CacheManager
    runner: ModelRunner
    weight_bytes: int


def build_model(raw_config: dict) -> tuple[object, DecoderModel]:
    arch = architecture_for(raw_config)
    cfg = arch.read_config(raw_config)
    return cfg, DecoderModel(arch.make_plan(cfg))


def pages_for_memory(model: DecoderModel, engine: EngineConfig, dtype: torch.dtype, device) -> int:
    """Pages per group when none were asked for: what ``memory_fraction`` of the free device
    memory holds, but never more than the engine can use. ``max_num_seqs`` requests can be
    resident, each at most ``max_model_len`` tokens long, so more pages than that (plus one
    spare page per request) would only be memory taken from everything else: a small model
    would otherwise claim most of the device, and the host lists with one entry per page
    would have millions of entries. At least 32 pages, as the reference
    (qwen3_runtime/engine/factory.py:94-107)."""
    per_page = CacheManager.bytes_per_page(model.plan.caches, engine.page_size, torch.finfo(dtype).bits // 8)
    if per_page == 0:
        return 32
    max_len = min(engine.max_model_len or model.plan.max_positions, model.plan.max_positions)
    useful = engine.max_num_seqs * (-(-max_len // engine.page_size) + 1)
    free, _total = torch.cuda.mem_get_info(device)
    return max(32, min(useful, int(free * engine.memory_fraction) // per_page))


def load(model_dir: str | Path | None, engine: EngineConfig, *, source=None, raw_config: dict | None = None,
         ops=None) -> LoadedModel:
    """Build, load and wire up. ``source``/``raw_config`` replace the folder (random weights on
    the device); ``ops`` replaces the HIP ops (host-side tests only)."""
    dtype = TORCH_DTYPE[engine.dtype]
    device = torch.device(engine.device)
    if raw_config is None:
        raw_config = read_config_json(model_dir)
    cfg, model = build_model(raw_config)
    if source is None:
        source = SafetensorsSource(model_dir)
    if ops is None:
        from ..ops.hip import HipOps

        if device.type != "cuda":
            raise RuntimeError("the engine runs on a GPU only; there is no CPU path")
        ops = HipOps()
    loader = load_model(model, source, device, dtype, where=f" in {model_dir}" if model_dir else "")
    num_pages = engine.num_pages or pages_for_memory(model, engine, dtype, device)
    cache = CacheManager(
        model.plan.caches, page_size=engine.page_size, num_pages=num_pages,
        max_requests=engine.max_num_seqs, device=device, dtype=dtype,
    )
    max_len = min(engine.max_model_len or model.plan.max_positions, model.plan.max_positions)
    runner = ModelRunner(model, cache, ops, dtype=dtype, device=device, max_model_len=max_len,
                         hip_graph=engine.hip_graph)
    return LoadedModel(cfg, model, cache, runner, loader.num_bytes)
