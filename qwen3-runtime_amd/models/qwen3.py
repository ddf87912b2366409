"""The Qwen3 dense decoder as a plan of parts.

Every layer is the same pre-norm block: grouped-query attention with per-head
q/k RMSNorm and NeoX rotary encoding, then a SwiGLU feed-forward; a final
RMSNorm and a head that is tied to the embedding or not
(reference: qwen3_runtime/models/qwen3.py:62-208). Tensor names are those of
the model file (reference: qwen3_runtime/utils/loader.py:33-54).
"""

from __future__ import annotations

from ..config.model import Qwen3Config
from ..config.presets import PRESET_PAGE_SIZE, PRESETS
from ..parts.plan import CacheSpec, LayerSpec, ModelPlan, PartSpec, RunStep
from ..registry import register_architecture, register_preset


def plan_qwen3(cfg: Qwen3Config) -> ModelPlan:
    rope = PartSpec("rope_neox", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta})
    layers, caches, order = [], [], []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        mixer = PartSpec(
            "gqa_attention",
            {
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "qk_norm_eps": cfg.rms_norm_eps,
                "position": rope,
                "window": None,
            },
            {
                "q": f"{p}.self_attn.q_proj.weight",
                "k": f"{p}.self_attn.k_proj.weight",
                "v": f"{p}.self_attn.v_proj.weight",
                "o": f"{p}.self_attn.o_proj.weight",
                "q_norm": f"{p}.self_attn.q_norm.weight",
                "k_norm": f"{p}.self_attn.k_norm.weight",
            },
        )
        ff = PartSpec(
            "swiglu",
            {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size},
            {
                "gate": f"{p}.mlp.gate_proj.weight",
                "up": f"{p}.mlp.up_proj.weight",
                "down": f"{p}.mlp.down_proj.weight",
            },
        )
        norms = {
            "input": _rmsnorm(cfg, f"{p}.input_layernorm.weight"),
            "post_mixer": _rmsnorm(cfg, f"{p}.post_attention_layernorm.weight"),
        }
        layers.append(LayerSpec(PartSpec("pre_norm"), mixer, ff, norms))
        caches.append(CacheSpec("paged_kv", heads=cfg.num_key_value_heads, head_dim=cfg.head_dim))
        order.append(RunStep(layer=i, cache=i))
    embed_name = "model.embed_tokens.weight"
    head_name = embed_name if cfg.tie_word_embeddings else "lm_head.weight"
    sizes = {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}
    return ModelPlan(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", sizes, {"weight": embed_name}),
        layers=layers,
        caches=caches,
        order=order,
        final_norm=_rmsnorm(cfg, "model.norm.weight"),
        head=PartSpec("linear_head", sizes, {"weight": head_name}),
        # a tied model file may still carry the head's copy; it is not read
        # (reference: qwen3_runtime/utils/loader.py:38-39)
        ignorable=("lm_head.weight",) if cfg.tie_word_embeddings else (),
        eos_token_id=cfg.eos_token_id,
    )


def _rmsnorm(cfg: Qwen3Config, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps}, {"weight": name})


register_architecture(Qwen3Config.architecture, Qwen3Config.from_dict, plan_qwen3)
for _name, _cfg in PRESETS.items():
    register_preset(_name, _cfg.to_dict(), PRESET_PAGE_SIZE.get(_name, 16))
