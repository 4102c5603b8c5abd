"""Configuration and registry (CPU)."""
import copy

import pytest

import cpmcu_amd
from cpmcu_amd.config import ConfigError, MiniCPMConfig
from cpmcu_amd.registry import get_architecture

import tiny


def test_reads_every_key_of_tiny_configs():
    a = MiniCPMConfig.from_dict(tiny.tiny_a())
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (2, 64, 4, 2, 16)
    assert (a.intermediate_size, a.vocab_size, a.rms_norm_eps, a.rope_theta) == (160, 512, 1e-6, 10000.0)
    assert a.tie_word_embeddings is True and a.sparse_config is None and a.eos_token_ids == (2,)
    assert a.residual_scale == pytest.approx(1.4 / 2 ** 0.5) and a.head_scale == pytest.approx(32 / 64)
    b = MiniCPMConfig.from_dict(tiny.tiny_b())
    assert b.head_dim == 32 and b.num_key_value_heads == 1 and b.eos_token_ids == (1, 7)
    assert b.sparse_config.window_blocks == 2 and b.sparse_config.dense_len == 64
    assert b.rope_scaling.original_max_position_embeddings == 128 and len(b.rope_scaling.long_factor) == 16


def test_defaults_when_keys_are_absent():
    raw = tiny.tiny_a()
    for k in ("scale_emb", "dim_model_base", "scale_depth", "num_key_value_heads", "rope_scaling", "tie_word_embeddings",
              "eos_token_id", "rope_theta"):
        raw.pop(k)
    c = MiniCPMConfig.from_dict(raw)
    assert c.scale_emb == 1.0 and c.residual_scale == 1.0 and c.head_scale == 1.0
    assert c.num_key_value_heads == c.num_attention_heads and c.head_dim == 16
    assert c.rope_scaling is None and c.tie_word_embeddings is None and c.eos_token_ids == () and c.rope_theta == 10000.0


def test_round_trip_through_to_dict():
    for raw in (tiny.tiny_a(), tiny.tiny_b()):
        c = MiniCPMConfig.from_dict(raw)
        assert MiniCPMConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change,needle", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"head_dim": 15}, "head_dim"),
    ({"eos_token_id": 99999}, "outside the vocabulary"),
])
def test_bad_values_are_refused(change, needle):
    raw = tiny.tiny_a()
    raw.update(change)
    with pytest.raises(ConfigError, match=needle):
        MiniCPMConfig.from_dict(raw)


def test_factor_list_of_wrong_length():
    raw = tiny.tiny_a()
    raw["rope_scaling"]["long_factor"] = [1.0] * 7
    with pytest.raises(ConfigError, match="long_factor.*7 entries.*8"):
        MiniCPMConfig.from_dict(raw)
    raw = tiny.tiny_a()
    raw["rope_scaling"]["rope_type"] = "yarn"
    with pytest.raises(ConfigError, match="yarn"):
        MiniCPMConfig.from_dict(raw)


@pytest.mark.parametrize("change,needle", [
    ({"block_size": 18}, "multiple of kernel_stride"),
    ({"kernel_size": 2}, "kernel_size"),
    ({"window_size": 40}, "window_size"),
    ({"init_blocks": 9}, "init_blocks"),
])
def test_sparse_config_is_validated(change, needle):
    raw = tiny.tiny_b()
    raw["sparse_config"].update(change)
    with pytest.raises(ConfigError, match=needle):
        MiniCPMConfig.from_dict(raw)


def test_registry_names_what_it_knows():
    assert "MiniCPMForCausalLM" in cpmcu_amd.architectures()
    with pytest.raises(KeyError, match="MiniCPMForCausalLM"):
        get_architecture("NoSuchModelForCausalLM")


def test_model_is_built_from_the_configuration_layer_by_layer():
    from cpmcu_amd.parts import GQAAttention, InfLLMv2Attention
    a = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_a()))
    b = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_b()))
    assert len(a.layers) == 2 and len(b.layers) == 3
    assert all(type(l.mixer) is GQAAttention for l in a.layers)
    assert all(type(l.mixer) is InfLLMv2Attention for l in b.layers)
    assert b.layers[0].mixer.bs == 16 and b.layers[0].mixer.window_blocks == 2
    assert a.head.tied_to is a.embedding and b.head.tied_to is None
    names = {s.name for s in b.all_weight_specs()}
    assert "lm_head.weight" in names and "model.layers.2.mlp.down_proj.weight" in names
    assert "lm_head.weight" not in {s.name for s in a.all_weight_specs()}
    # sparse attention can be switched off without touching the configuration
    d = get_architecture("MiniCPMForCausalLM").build(MiniCPMConfig.from_dict(tiny.tiny_b()), sparse=False)
    assert all(type(l.mixer) is GQAAttention for l in d.layers)
