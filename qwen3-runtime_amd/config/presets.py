"""Named configurations used by tests and measurements.

The two tiny ones differ in every size and option; the large ones carry the
published sizes of the Qwen3 dense family (4B: reference docs/pins/Qwen3-4B/config.json).
"""

from __future__ import annotations

from .model import Qwen3Config

PRESETS: dict[str, Qwen3Config] = {
    "tiny_a": Qwen3Config(
        vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=16, intermediate_size=128, rms_norm_eps=1e-6,
        rope_theta=10000.0, max_position_embeddings=512, tie_word_embeddings=True,
    ),
    "tiny_b": Qwen3Config(
        vocab_size=384, hidden_size=96, num_hidden_layers=3, num_attention_heads=6,
        num_key_value_heads=2, head_dim=32, intermediate_size=272, rms_norm_eps=1e-5,
        rope_theta=1000000.0, max_position_embeddings=1024, tie_word_embeddings=False,
    ),
    "qwen3_4b": Qwen3Config(
        vocab_size=151936, hidden_size=2560, num_hidden_layers=36, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=9728, rms_norm_eps=1e-6,
        rope_theta=1000000.0, max_position_embeddings=40960, tie_word_embeddings=True,
        eos_token_id=151645,
    ),
    "qwen3_8b": Qwen3Config(
        vocab_size=151936, hidden_size=4096, num_hidden_layers=36, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
        rope_theta=1000000.0, max_position_embeddings=40960, tie_word_embeddings=False,
        eos_token_id=151645,
    ),
    "qwen3_32b": Qwen3Config(
        vocab_size=151936, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64,
        num_key_value_heads=8, head_dim=128, intermediate_size=25600, rms_norm_eps=1e-6,
        rope_theta=1000000.0, max_position_embeddings=40960, tie_word_embeddings=False,
        eos_token_id=151645,
    ),
}

# page size each preset is run with by default
PRESET_PAGE_SIZE = {"tiny_a": 16, "tiny_b": 8}


def preset(name: str) -> Qwen3Config:
    try:
        return PRESETS[name]
    except KeyError:
        raise ValueError(f"unknown preset {name!r}; presets: {sorted(PRESETS)}") from None
