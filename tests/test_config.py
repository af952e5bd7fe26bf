"""Configuration and the architecture registry (no GPU)."""
import json

import pytest

import tiny
from palm_infra_amd.config import (ConfigError, Qwen3Config, config_from_dict, config_from_dir, registered_architectures)


def test_reads_the_reference_keys_and_defaults():
    # models/qwen3.py:175-184: kv heads default to heads, head_dim to hidden/heads, eps 1e-6, theta 1e6
    cfg = config_from_dict(dict(architectures=["Qwen3ForCausalLM"], vocab_size=100, hidden_size=48, num_hidden_layers=1,
                                num_attention_heads=6, intermediate_size=64))
    assert isinstance(cfg, Qwen3Config)
    assert (cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps, cfg.rope_theta) == (6, 8, 1e-6, 1000000.0)
    assert cfg.tie_word_embeddings is None


def test_model_type_is_a_second_way_in():
    raw = dict(tiny.CONFIGS["A"])
    raw.pop("architectures")
    assert isinstance(config_from_dict(raw), Qwen3Config)


def test_unknown_architecture_lists_the_registered_ones():
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(architectures=["LlamaForCausalLM"], model_type="llama"))
    assert "LlamaForCausalLM" in str(e.value) and "Qwen3ForCausalLM" in str(e.value)
    assert "Qwen3ForCausalLM" in registered_architectures()


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size"])
def test_missing_required_key(key):
    raw = dict(tiny.CONFIGS["A"])
    raw.pop(key)
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


@pytest.mark.parametrize("change,word", [
    (dict(num_key_value_heads=3), "divisible"),            # models/qwen3.py:186-190
    (dict(head_dim=15), "even"),
    (dict(num_hidden_layers=0), "positive"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(use_sliding_window=True, sliding_window=128), "sliding window"),
    (dict(rope_scaling={"type": "yarn", "factor": 4.0}), "rope_scaling"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
])
def test_values_the_architecture_cannot_run_with(change, word):
    with pytest.raises(ConfigError, match=word):
        config_from_dict(dict(tiny.CONFIGS["A"], **change))


def test_a_window_that_is_switched_off_is_accepted():
    # Qwen3 checkpoints carry sliding_window with use_sliding_window=false
    config_from_dict(dict(tiny.CONFIGS["A"], use_sliding_window=False, sliding_window=4096, rope_scaling=None))


def test_round_trip_through_config_json(tmp_path):
    for name, raw in tiny.CONFIGS.items():
        cfg = config_from_dict(raw)
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        assert config_from_dir(tmp_path) == cfg, name


def test_stop_tokens_come_from_eos_token_id():
    assert config_from_dict(tiny.CONFIGS["A"]).spec().stop_token_ids == (7,)
    assert config_from_dict(tiny.CONFIGS["B"]).spec().stop_token_ids == (3, 11)
    assert config_from_dict(tiny.CONFIGS["C"]).spec().stop_token_ids == ()


def test_description_names_every_checkpoint_tensor_with_its_shape():
    cfg = config_from_dict(tiny.CONFIGS["B"])
    exp = cfg.spec().expected_tensors()
    # the names of the reference's fixture (tests/run_tiny_qwen3_cpu_e2e.py:79-94)
    for n in ("model.embed_tokens.weight", "lm_head.weight", "model.norm.weight",
              "model.layers.0.input_layernorm.weight", "model.layers.0.post_attention_layernorm.weight",
              "model.layers.2.self_attn.q_proj.weight", "model.layers.2.self_attn.k_proj.weight",
              "model.layers.2.self_attn.v_proj.weight", "model.layers.2.self_attn.q_norm.weight",
              "model.layers.2.self_attn.k_norm.weight", "model.layers.2.self_attn.o_proj.weight",
              "model.layers.2.mlp.gate_proj.weight", "model.layers.2.mlp.up_proj.weight", "model.layers.2.mlp.down_proj.weight"):
        assert n in exp, n
    assert len(exp) == 3 + 11 * 3
    assert exp["model.layers.1.self_attn.q_proj.weight"][0] == (8 * 32, 96)       # heads*head_dim != hidden
    assert exp["model.layers.1.self_attn.k_proj.weight"][0] == (1 * 32, 96)
    assert exp["model.layers.1.self_attn.o_proj.weight"][0] == (96, 256)
    assert exp["model.layers.1.self_attn.q_norm.weight"] == ((32,), "vector")
    assert exp["model.layers.1.mlp.down_proj.weight"][0] == (96, 224)


def test_joined_projections_keep_the_reference_order():
    # q rows, then k, then v (models/qwen3.py:125-142); gate rows, then up (models/qwen3.py:144-160)
    spec = config_from_dict(tiny.CONFIGS["A"]).spec()
    mixer = spec.layers[0].parts["mixer"]
    assert [n.split(".")[-2] for n in mixer.tensors["qkv"].names] == ["q_proj", "k_proj", "v_proj"]
    assert mixer.tensors["qkv"].shape == (4 * 16 + 2 * 2 * 16, 64)          # as tests/test_qwen3_graph.py:43-51
    ff = spec.layers[0].parts["feed_forward"]
    assert [n.split(".")[-2] for n in ff.tensors["gate_up"].names] == ["gate_proj", "up_proj"]
    assert ff.tensors["gate_up"].shape == (256, 64)


def test_head_is_tied_by_key_or_by_what_the_checkpoint_holds():
    raw = dict(tiny.CONFIGS["A"])
    assert "lm_head.weight" not in config_from_dict(raw).spec().expected_tensors()
    raw["tie_word_embeddings"] = False
    assert "lm_head.weight" in config_from_dict(raw).spec().expected_tensors()
    # models/qwen3.py:89-95, 162-165: lm_head.weight if the file has it, else the embedding, whatever the key says
    for tie in (True, False, None):
        cfg = config_from_dict({k: v for k, v in dict(raw, tie_word_embeddings=tie).items() if v is not None})
        assert "lm_head.weight" in cfg.spec(["lm_head.weight", "model.embed_tokens.weight"]).expected_tensors()
        assert "lm_head.weight" not in cfg.spec(["model.embed_tokens.weight"]).expected_tensors()


def test_run_order_is_data_and_is_checked():
    from palm_infra_amd.config import LayerCall
    spec = config_from_dict(tiny.CONFIGS["A"]).spec()
    import dataclasses
    twice = dataclasses.replace(spec, order=(LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(1, cache_of=1)))
    assert len(twice.order) == 4
    with pytest.raises(ValueError, match="does not run before"):
        dataclasses.replace(spec, order=(LayerCall(0, cache_of=1), LayerCall(1)))
    with pytest.raises(ValueError, match="names layer"):
        dataclasses.replace(spec, order=(LayerCall(5),))
    with pytest.raises(ValueError, match="holds none"):
        dataclasses.replace(spec, order=(LayerCall(0), LayerCall(1, cache_of=0), LayerCall(0, cache_of=1)))


def test_named_sizes_are_data_and_load():
    from palm_infra_amd.config import ConfigError, config_source, preset_dict, preset_names
    assert {"tiny-a", "tiny-b", "qwen3-8b", "qwen3-14b", "qwen3-32b"} <= set(preset_names())
    for name in preset_names():
        cfg = config_from_dict(preset_dict(name))
        assert cfg.spec().vocab_size == preset_dict(name)["vocab_size"]
    assert config_source("tiny-b")["head_dim"] == 32
    with pytest.raises(ConfigError, match="unknown size 'qwen9'.*tiny-a"):
        config_source("qwen9")


def test_config_source_reads_a_file_or_a_folder(tmp_path):
    import json
    from palm_infra_amd.config import config_source
    (tmp_path / "config.json").write_text(json.dumps(tiny.CONFIGS["A"]))
    assert config_source(tmp_path) == tiny.CONFIGS["A"] == config_source(tmp_path / "config.json")


def test_rotation_base_in_a_rope_parameters_table():
    raw = {k: v for k, v in tiny.CONFIGS["B"].items() if k != "rope_theta"}
    assert config_from_dict(dict(raw, rope_parameters={"rope_type": "default", "rope_theta": 12345.0})).rope_theta == 12345.0
    assert config_from_dict(dict(raw, rope_theta=7.0, rope_parameters={"rope_theta": 12345.0})).rope_theta == 7.0
    assert config_from_dict(raw).rope_theta == 1000000.0
    with pytest.raises(ConfigError, match="plain rotation only"):
        config_from_dict(dict(raw, rope_parameters={"rope_type": "yarn", "rope_theta": 1e6, "factor": 4.0}))


def test_stop_tokens_of_generation_config_join_those_of_config(tmp_path):
    import json
    (tmp_path / "config.json").write_text(json.dumps(dict(tiny.CONFIGS["A"], eos_token_id=7)))
    assert config_from_dir(tmp_path).eos_token_ids == (7,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [9, 7], "temperature": 0.6}))
    assert config_from_dir(tmp_path).eos_token_ids == (7, 9)
    assert config_from_dir(tmp_path).spec().stop_token_ids == (7, 9)
    (tmp_path / "generation_config.json").write_text(json.dumps({"top_k": 20}))
    assert config_from_dir(tmp_path).eos_token_ids == (7,)
