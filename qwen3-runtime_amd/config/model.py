"""Typed model configuration read from a model folder's ``config.json``.

``Qwen3Config`` reads the keys the Qwen3 dense decoder defines and rejects the
options the architecture does not implement, with the same conditions as
``Qwen3ModelConfig.from_hf_config`` (reference: qwen3_runtime/models/qwen3.py:33-59).
It adds the consistency checks the reference leaves out (head counts that do
not divide, an odd head size, sizes below one).

Nothing outside this file knows a size: parts receive their numbers as
constructor arguments, taken from an instance of this class.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json the engine cannot run: says which key and why."""


_REQUIRED = (
    "vocab_size",
    "hidden_size",
    "num_hidden_layers",
    "num_attention_heads",
    "num_key_value_heads",
    "intermediate_size",
    "rms_norm_eps",
    "rope_theta",
    "max_position_embeddings",
    "tie_word_embeddings",
)


@dataclass(frozen=True)
class Qwen3Config:
    """Sizes and constants of one Qwen3 dense decoder.

    Field meanings follow config.json (reference: qwen3_runtime/models/qwen3.py:19-31):
    ``head_dim`` defaults to ``hidden_size // num_attention_heads`` and may make
    ``num_attention_heads * head_dim`` differ from ``hidden_size``; ``rms_norm_eps``
    is the one eps of every RMSNorm, including the per-head q/k norms;
    ``max_position_embeddings`` bounds the positions a request may reach.
    """

    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_id: int | None = None

    architecture = "Qwen3ForCausalLM"

    def __post_init__(self) -> None:
        for key in (
            "vocab_size",
            "hidden_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "intermediate_size",
            "max_position_embeddings",
        ):
            if int(getattr(self, key)) < 1:
                raise ConfigError(f"{key} must be positive, got {getattr(self, key)!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for rotary position encoding")
        if not self.rms_norm_eps > 0.0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not self.rope_theta > 0.0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        """Validate and read config.json's keys (reference: qwen3_runtime/models/qwen3.py:33-59)."""
        arch = raw.get("architectures") or []
        if cls.architecture not in arch:
            raise ConfigError(f"unsupported architectures: {arch}")
        if raw.get("hidden_act") != "silu":
            raise ConfigError(f"unsupported hidden_act: {raw.get('hidden_act')!r}")
        if raw.get("use_sliding_window"):
            raise ConfigError("use_sliding_window is set: the Qwen3 dense decoder here has no window")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"unsupported rope_scaling: {raw.get('rope_scaling')!r}")
        if raw.get("attention_bias"):
            raise ConfigError("attention_bias is set: q/k/v/o projections here have no bias")
        missing = [k for k in _REQUIRED if k not in raw]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {missing}")
        head_dim = raw.get("head_dim") or int(raw["hidden_size"]) // int(raw["num_attention_heads"])
        eos = raw.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            # a list of stop ids takes its first (reference: qwen3_runtime/engine/factory.py:64-72)
            eos = eos[0] if eos else None
        return cls(
            vocab_size=int(raw["vocab_size"]),
            hidden_size=int(raw["hidden_size"]),
            num_hidden_layers=int(raw["num_hidden_layers"]),
            num_attention_heads=int(raw["num_attention_heads"]),
            num_key_value_heads=int(raw["num_key_value_heads"]),
            head_dim=int(head_dim),
            intermediate_size=int(raw["intermediate_size"]),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=float(raw["rope_theta"]),
            max_position_embeddings=int(raw["max_position_embeddings"]),
            tie_word_embeddings=bool(raw["tie_word_embeddings"]),
            eos_token_id=None if eos is None else int(eos),
        )

    def to_dict(self) -> dict[str, Any]:
        """The config.json a model folder of this configuration carries."""
        raw = asdict(self)
        raw.update(
            architectures=[self.architecture],
            model_type="qwen3",
            hidden_act="silu",
            attention_bias=False,
            use_sliding_window=False,
            rope_scaling=None,
            torch_dtype="bfloat16",
        )
        if raw["eos_token_id"] is None:
            del raw["eos_token_id"]
        return raw

    # Derived widths, so no caller multiplies sizes itself.
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim


def read_config_json(folder: str | Path) -> dict[str, Any]:
    path = Path(folder) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in {Path(folder)}")
    return json.loads(path.read_text())
