"""Configuration, registry, weight loading errors and the random-weights mode (no GPU)."""

import json

import pytest
import torch

from qwen3_runtime_amd.config.model import ConfigError, Qwen3Config
from qwen3_runtime_amd.config.presets import preset
from qwen3_runtime_amd.parts.model import DecoderModel
from qwen3_runtime_amd.registry import architecture_for, architecture_names
from qwen3_runtime_amd.weights import (RandomSource, SafetensorsSource, WeightError, check_source, load_model,
                                       write_model_folder)


def raw_4b():
    # the reference's pinned Qwen3-4B config.json (docs/pins/Qwen3-4B/config.json)
    return {
        "architectures": ["Qwen3ForCausalLM"], "attention_bias": False, "attention_dropout": 0.0,
        "bos_token_id": 151643, "eos_token_id": 151645, "head_dim": 128, "hidden_act": "silu",
        "hidden_size": 2560, "initializer_range": 0.02, "intermediate_size": 9728,
        "max_position_embeddings": 40960, "max_window_layers": 36, "model_type": "qwen3",
        "num_attention_heads": 32, "num_hidden_layers": 36, "num_key_value_heads": 8, "rms_norm_eps": 1e-06,
        "rope_scaling": None, "rope_theta": 1000000, "sliding_window": None, "tie_word_embeddings": True,
        "torch_dtype": "bfloat16", "use_cache": True, "use_sliding_window": False, "vocab_size": 151936,
    }


def test_pinned_4b_config_values():
    # reference: tests/cpu/test_model_config.py:9-32
    cfg = Qwen3Config.from_dict(raw_4b())
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads) == (2560, 36, 32, 8)
    assert cfg.head_dim == 128 and cfg.q_width == 4096 != cfg.hidden_size
    assert cfg.intermediate_size == 9728 and cfg.vocab_size == 151936
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-6 and cfg.tie_word_embeddings
    assert cfg.eos_token_id == 151645
    assert cfg == preset("qwen3_4b")


def test_head_dim_defaults_to_hidden_over_heads():
    raw = raw_4b()
    del raw["head_dim"]
    assert Qwen3Config.from_dict(raw).head_dim == 2560 // 32


@pytest.mark.parametrize("key,value,match", [
    ("architectures", ["LlamaForCausalLM"], "unsupported architectures"),
    ("hidden_act", "gelu", "hidden_act"),
    ("use_sliding_window", True, "sliding"),
    ("rope_scaling", {"type": "yarn", "factor": 4}, "rope_scaling"),
    ("attention_bias", True, "bias"),
    ("num_key_value_heads", 5, "multiple"),
    ("head_dim", 33, "even"),
    ("rms_norm_eps", 0.0, "rms_norm_eps"),
    ("vocab_size", 0, "vocab_size"),
])
def test_config_rejects(key, value, match):
    raw = raw_4b()
    raw[key] = value
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict(raw)


def test_config_names_missing_keys():
    raw = raw_4b()
    del raw["rope_theta"], raw["intermediate_size"]
    with pytest.raises(ConfigError, match=r"rope_theta.*|intermediate_size"):
        Qwen3Config.from_dict(raw)


def test_eos_list_takes_first():
    raw = raw_4b()
    raw["eos_token_id"] = [7, 8]
    assert Qwen3Config.from_dict(raw).eos_token_id == 7


def test_config_round_trips_through_config_json():
    for name in ("tiny_a", "tiny_b"):
        cfg = preset(name)
        assert Qwen3Config.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg


def test_registry_picks_by_architecture_name():
    assert "Qwen3ForCausalLM" in architecture_names()
    arch = architecture_for(raw_4b())
    assert arch.name == "Qwen3ForCausalLM"
    with pytest.raises(ValueError, match="registered.*Qwen3ForCausalLM"):
        architecture_for({"architectures": ["NoSuchModel"]})


def test_tiny_presets_differ_in_every_size_and_option():
    a, b = preset("tiny_a"), preset("tiny_b")
    for field in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "head_dim",
                  "intermediate_size", "rms_norm_eps", "rope_theta", "tie_word_embeddings"):
        assert getattr(a, field) != getattr(b, field), field
    assert a.num_attention_heads // a.num_key_value_heads != b.num_attention_heads // b.num_key_value_heads
    assert a.q_width == a.hidden_size and b.q_width != b.hidden_size


def model_of(cfg):
    arch = architecture_for(cfg.to_dict())
    return DecoderModel(arch.make_plan(cfg))


def test_plan_declares_the_model_files_tensors():
    names = {d.file_name: d.shape for d in model_of(preset("tiny_b")).tensor_decls()}
    assert names["model.layers.2.self_attn.q_proj.weight"] == (6 * 32, 96)
    assert names["model.layers.0.self_attn.k_proj.weight"] == (2 * 32, 96)
    assert names["model.layers.1.self_attn.q_norm.weight"] == (32,)
    assert names["model.layers.1.mlp.down_proj.weight"] == (96, 272)
    assert names["lm_head.weight"] == (384, 96)
    assert "lm_head.weight" not in {d.file_name for d in model_of(preset("tiny_a")).tensor_decls()}
    assert len(names) == 3 * 11 + 3


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    from safetensors.torch import load_file, save_file

    cfg = preset("tiny_a")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=1)
    tensors = load_file(str(folder / "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_norm.weight"] = torch.ones(17)
    tensors["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(64, 65)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as err:
        load_model(model_of(cfg), SafetensorsSource(folder), "cpu", torch.float32)
    e = err.value
    assert sorted(e.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert sorted(n for n, _, _ in e.wrong_shape) == [
        "model.layers.0.self_attn.k_norm.weight", "model.layers.0.self_attn.o_proj.weight"]
    text = str(e)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "[17]", "[16]", "[64, 65]"):
        assert piece in text


def test_an_integer_tensor_where_a_matrix_is_read_is_an_error(tmp_path):
    """A tensor of the right name and shape but stored as integers (a quantised file, say) must
    not be cast silently into weights; it is named in the same single error."""
    from safetensors.torch import load_file, save_file

    cfg = preset("tiny_a")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=1)
    tensors = load_file(str(folder / "model.safetensors"))
    name = "model.layers.1.self_attn.q_proj.weight"
    tensors[name] = torch.zeros(tensors[name].shape, dtype=torch.int8)
    del tensors["model.norm.weight"]
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as err:
        load_model(model_of(cfg), SafetensorsSource(folder), "cpu", torch.float32)
    assert err.value.wrong_dtype == [(name, "int8", "bfloat16, float32 or float16")]
    assert err.value.missing == ["model.norm.weight"]
    assert "wrong types (1)" in str(err.value) and "stored as int8" in str(err.value)


def test_integer_tables_are_declared_drawn_and_kept_as_int32():
    """A part may declare an integer table: it is drawn as integers, stored as int32, loaded
    as int32 in both engine types, and a floating tensor in its place is an error."""
    from qwen3_runtime_amd.parts.plan import TensorDecl
    from qwen3_runtime_amd.weights.loader import WeightLoader

    decls = [TensorDecl("perm", (7,), init="index:5", storage="int"), TensorDecl("w", (3, 4))]
    src = RandomSource(decls, 3)
    assert src.dtype("perm") == torch.int32 and src.dtype("w") == torch.bfloat16
    perm = src.get("perm")
    assert perm.dtype == torch.int32 and 0 <= int(perm.min()) and int(perm.max()) < 5
    check_source(src, decls)
    for engine_dtype in (torch.bfloat16, torch.float32):
        assert WeightLoader(src, "cpu", engine_dtype).table_i32("perm").dtype == torch.int32
    swapped = RandomSource([TensorDecl("perm", (7,)), TensorDecl("w", (3, 4))], 3)
    with pytest.raises(WeightError, match="perm is stored as bfloat16, expected an integer type"):
        check_source(swapped, decls)


def test_tied_model_may_carry_an_unused_head(tmp_path):
    from safetensors.torch import load_file, save_file

    cfg = preset("tiny_a")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=1)
    tensors = load_file(str(folder / "model.safetensors"))
    tensors["lm_head.weight"] = torch.zeros(cfg.vocab_size, cfg.hidden_size)
    save_file(tensors, str(folder / "model.safetensors"))
    model = model_of(cfg)
    load_model(model, SafetensorsSource(folder), "cpu", torch.float32)
    assert model.head.weight is model.embedding.weight  # one tensor serves both


def test_no_safetensors_and_no_config(tmp_path):
    from qwen3_runtime_amd.config.model import read_config_json

    with pytest.raises(FileNotFoundError):
        SafetensorsSource(tmp_path)
    with pytest.raises(FileNotFoundError):
        read_config_json(tmp_path)


def test_sharded_folder_reads_through_the_index(tmp_path):
    from safetensors.torch import load_file, save_file

    cfg = preset("tiny_a")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=1)
    tensors = load_file(str(folder / "model.safetensors"))
    (folder / "model.safetensors").unlink()
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    weight_map = {}
    for fname, keys in shards.items():
        save_file({k: tensors[k] for k in keys}, str(folder / fname))
        weight_map.update({k: fname for k in keys})
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    src = SafetensorsSource(folder)
    check_source(src, model_of(cfg).tensor_decls())
    assert torch.equal(src.get("model.norm.weight"), tensors["model.norm.weight"])


def test_placement_keeps_bfloat16_and_float32_as_stored(tmp_path):
    cfg = preset("tiny_a")
    f32 = ("model.norm.weight", "model.layers.0.mlp.down_proj.weight")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=1, f32_names=f32)
    model = model_of(cfg)
    load_model(model, SafetensorsSource(folder), "cpu", torch.bfloat16)
    assert model.embedding.weight.dtype == torch.bfloat16
    assert model.blocks[0].feed_forward.down.dtype == torch.float32   # stored in 32-bit: stays so
    assert model.blocks[1].feed_forward.down.dtype == torch.bfloat16
    assert model.blocks[0].mixer.qkv.dtype == torch.bfloat16
    assert model.final_norm.weight.dtype == torch.float32              # norm weights are held in float32
    model32 = model_of(cfg)
    load_model(model32, SafetensorsSource(folder), "cpu", torch.float32)
    assert model32.blocks[0].mixer.qkv.dtype == torch.float32
    # upcasting the stored bfloat16 is exact
    assert torch.equal(model32.blocks[1].feed_forward.down, model.blocks[1].feed_forward.down.float())


def test_fused_rows_are_q_then_k_then_v_and_gate_then_up(tmp_path):
    # reference: qwen3_runtime/utils/loader.py:42-53
    from safetensors.torch import load_file

    cfg = preset("tiny_b")
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=2)
    t = load_file(str(folder / "model.safetensors"))
    model = model_of(cfg)
    load_model(model, SafetensorsSource(folder), "cpu", torch.float32)
    p = "model.layers.1"
    want = torch.cat([t[f"{p}.self_attn.q_proj.weight"], t[f"{p}.self_attn.k_proj.weight"],
                      t[f"{p}.self_attn.v_proj.weight"]]).float()
    assert torch.equal(model.blocks[1].mixer.qkv, want)
    want = torch.cat([t[f"{p}.mlp.gate_proj.weight"], t[f"{p}.mlp.up_proj.weight"]]).float()
    assert torch.equal(model.blocks[1].feed_forward.gate_up, want)


def test_random_weights_are_seeded_by_name_and_have_the_stated_moments(tmp_path):
    cfg = preset("tiny_b")
    decls = model_of(cfg).tensor_decls()
    a, b = RandomSource(decls, 5), RandomSource(list(reversed(decls)), 5)
    name = "model.layers.2.mlp.gate_proj.weight"
    assert torch.equal(a.get(name), b.get(name))            # order of asking does not matter
    assert not torch.equal(a.get(name), RandomSource(decls, 6).get(name))
    w = RandomSource(decls, 5, store_dtype=torch.float32).get(name)
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = RandomSource(decls, 5, store_dtype=torch.float32).get("model.layers.0.input_layernorm.weight")
    assert abs(float(n.mean()) - 1.0) < 0.05 and 0.05 < float(n.std()) < 0.15
    ones = RandomSource(decls, 5, norm_jitter=0.0).get("model.norm.weight")
    assert torch.equal(ones.float(), torch.ones(cfg.hidden_size))
    folder = write_model_folder(tmp_path / "m", cfg.to_dict(), seed=5)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    src = SafetensorsSource(folder)
    assert src.dtype(name) == torch.bfloat16 and src.shape(name) == (272, 96)
    assert torch.equal(src.get(name), a.get(name))
