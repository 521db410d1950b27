"""The typed configuration and the registry."""

import json

import pytest

from conftest import TINY_A, TINY_B
from mini_llm_amd.config import (ConfigError, GPT2Config, config_from_dict, get_architecture, load_config,
                                 register_architecture, registered_architectures)


def test_reads_its_own_keys():
    c = config_from_dict(TINY_B)
    assert isinstance(c, GPT2Config)
    assert (c.n_layer, c.n_embd, c.n_head, c.n_inner, c.vocab_size, c.n_positions) == (3, 96, 3, 320, 1000, 64)
    assert c.layer_norm_epsilon == 1e-6 and c.activation_function == "gelu" and c.head_size == 32


def test_n_inner_null_or_absent_is_four_times_the_width():
    assert config_from_dict(TINY_A).n_inner == 256
    raw = {k: v for k, v in TINY_A.items() if k != "n_inner"}
    assert config_from_dict(raw).n_inner == 256


def test_defaults_are_gpt2_small():
    c = config_from_dict({"architectures": ["GPT2LMHeadModel"]})
    assert (c.n_layer, c.n_embd, c.n_head, c.n_inner, c.vocab_size, c.n_positions) == (12, 768, 12, 3072, 50257, 1024)
    assert c.layer_norm_epsilon == 1e-5 and c.activation_function == "gelu_new"


def test_roundtrip_through_to_dict(tmp_path):
    c = config_from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert load_config(tmp_path) == c


@pytest.mark.parametrize(
    "change,word",
    [
        ({"n_head": 5}, "divisible"),
        ({"activation_function": "relu"}, "activation_function"),
        ({"n_layer": 0}, "n_layer"),
        ({"n_embd": "64"}, "n_embd"),
        ({"vocab_size": -3}, "vocab_size"),
        ({"layer_norm_epsilon": 0}, "layer_norm_epsilon"),
        ({"tie_word_embeddings": False}, "tie_word_embeddings"),
        ({"scale_attn_by_inverse_layer_idx": True}, "scale_attn_by_inverse_layer_idx"),
        ({"reorder_and_upcast_attn": True}, "reorder_and_upcast_attn"),
        ({"scale_attn_weights": False}, "scale_attn_weights"),
    ],
)
def test_refuses_what_it_cannot_run(change, word):
    with pytest.raises(ConfigError, match=word):
        config_from_dict(dict(TINY_A, **change))


def test_unknown_architecture_names_the_registered_ones():
    with pytest.raises(ConfigError, match="GPT2LMHeadModel"):
        config_from_dict(dict(TINY_A, architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_missing_or_broken_config_json(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(tmp_path)


def test_registry_builds_the_model_from_parts():
    from mini_llm_amd.precision import Precision

    assert "GPT2LMHeadModel" in registered_architectures()
    config = config_from_dict(TINY_B)
    model = get_architecture("GPT2LMHeadModel").build(config, Precision.from_name("float32"))
    specs = model.named_tensor_specs()
    assert specs["h.2.attn.c_attn.weight"].shape == (96, 288) and specs["h.0.mlp.c_fc.weight"].shape == (96, 320)
    assert specs["wte.weight"].shape == (1000, 96) and specs["wpe.weight"].shape == (64, 96)
    assert len(specs) == 2 + 12 * 3 + 2
    assert [(c.block, c.cache, c.write_cache) for c in model.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True)]
    (group,) = model.cache_groups()
    assert (group.layers, group.n_kv_heads, group.head_size, group.window) == ((0, 1, 2), 3, 32, None)
    assert model.max_positions() == 64 and model.vocab_size == 1000


def test_another_architecture_can_be_registered():
    calls = []
    register_architecture("ToyForTests", GPT2Config, lambda config, precision: calls.append(config) or "model")
    config = config_from_dict(dict(TINY_A, architectures=["ToyForTests"]))
    assert get_architecture(config.architecture).build(config, None) == "model" and calls == [config]


def test_any_head_size_the_kernels_take_is_a_valid_configuration():
    # the reference takes every width that its heads divide (pytorch/src/mini_llm/vector_addition_extension.cpp:180)
    for n_embd, n_head in ((40, 4), (42, 3), (72, 3), (256, 1), (7, 7)):
        assert config_from_dict(dict(TINY_A, n_embd=n_embd, n_head=n_head)).head_size == n_embd // n_head
    with pytest.raises(ConfigError, match="wider than the attention kernels take"):
        config_from_dict(dict(TINY_A, n_embd=514, n_head=2))
    with pytest.raises(ConfigError, match="not divisible"):
        config_from_dict(dict(TINY_A, n_embd=42, n_head=4))
