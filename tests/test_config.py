"""Configuration and registry (CPU)."""
import copy
import json

import pytest

import pytriton_llama_amd  # noqa: F401
from pytriton_llama_amd.config import (ConfigError, LlamaConfig, MODEL_REGISTRY, build_model,
                                       config_from_dict, config_from_folder)
from tiny_configs import TINY_A, TINY_B, TINY_C


def test_reads_every_size_from_the_file():
    c = config_from_dict(TINY_B)
    assert isinstance(c, LlamaConfig)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads,
            c.head_dim, c.intermediate_size, c.vocab_size) == (3, 128, 4, 1, 32, 320, 384)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and not c.tie_word_embeddings
    rs = c.rope_scaling
    assert (rs.rope_type, rs.factor, rs.low_freq_factor, rs.high_freq_factor,
            rs.original_max_position_embeddings) == ("llama3", 8.0, 1.0, 4.0, 64)
    assert c.group_size == 4 and c.q_size == 128 and c.kv_size == 32


def test_head_dim_is_honoured_when_given():
    # the reference always overwrites it with hidden/heads (model_config.py:41-45)
    c = config_from_dict(TINY_C)
    assert c.head_dim == 64 and c.q_size == 6 * 64 != c.hidden_size
    assert c.rope_scaling.rope_type == "llama3"          # through the legacy key "type"
    assert config_from_dict(TINY_A).head_dim == 8


def test_kv_heads_default_to_heads():
    d = copy.deepcopy(TINY_A)
    del d["num_key_value_heads"]
    assert config_from_dict(d).num_key_value_heads == 8


@pytest.mark.parametrize("change, word", [
    ({"num_key_value_heads": 3}, "multiple"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "lacks"),
    ({"head_dim": 7}, "even"),
    ({"vocab_size": None}, "vocab_size"),
    ({"hidden_size": 60, "num_attention_heads": 7}, "head_dim"),
    ({"architectures": ["GPT2LMHeadModel"]}, "not supported"),
    ({"architectures": [], "model_type": "other"}, "architectures"),
])
def test_rejects_what_it_cannot_run(change, word):
    d = copy.deepcopy(TINY_A)
    d.update(change)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_model_type_stands_in_for_a_missing_architectures_entry():
    d = copy.deepcopy(TINY_A)
    del d["architectures"]
    assert isinstance(config_from_dict(d), LlamaConfig)
    d["model_type"] = "gpt2"
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict(d)


def test_registry_maps_name_to_model():
    assert "LlamaForCausalLM" in MODEL_REGISTRY
    m = build_model(TINY_B)
    assert len(m.blocks) == 3 and len(m.schedule) == 3 and len(m.cache_layers) == 3
    names = set(m.expected_tensors())
    assert "lm_head.weight" in names and "model.layers.2.mlp.down_proj.weight" in names
    assert len(names) == 3 + 9 * 3
    tied = build_model(TINY_A)
    assert "lm_head.weight" not in tied.expected_tensors()
    assert tied.head.tied_to is tied.embedding


def test_parameter_count_of_the_1b_shape():
    cfg = dict(TINY_A, num_hidden_layers=16, hidden_size=2048, num_attention_heads=32,
               num_key_value_heads=8, intermediate_size=8192, vocab_size=128256)
    m = build_model(cfg)
    total = 0
    for _, (_, src) in m.expected_tensors().items():
        n = 1
        for s in src.shape:
            n *= s
        total += n
    assert total == 1_235_814_400


def test_round_trip_through_a_folder(tmp_path):
    c = config_from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert config_from_folder(str(tmp_path)) == c
    with pytest.raises(ConfigError, match="config.json"):
        config_from_folder(str(tmp_path / "nowhere"))


def test_parts_take_their_numbers_as_parameters():
    a, b = build_model(TINY_A), build_model(TINY_B)
    assert a.blocks[0].input_norm.eps == 1e-5 and b.blocks[0].input_norm.eps == 1e-6
    assert a.blocks[0].mixer.num_kv_heads == 2 and b.blocks[0].mixer.num_kv_heads == 1
    assert abs(a.blocks[0].mixer.scale - 8 ** -0.5) < 1e-12 and abs(b.blocks[0].mixer.scale - 32 ** -0.5) < 1e-12
    assert b.blocks[0].feed_forward.intermediate_size == 320
