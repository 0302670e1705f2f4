"""Configuration: keys, defaults, validation errors that name key and value, the registry."""
import json

import pytest

from helpers import CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D

import vipera_rs_amd  # noqa: F401
from vipera_rs_amd import models  # noqa: F401  (registers architectures)
from vipera_rs_amd.config import (Qwen2Config, architecture_names, config_from_dict, load_config,
                                  lookup_architecture, register_architecture, unregister_architecture)
from vipera_rs_amd.errors import InvalidArgumentError, IoError, ParseError, UnsupportedError


def test_reads_every_size_from_the_file():
    cfg = config_from_dict(CONFIG_B)
    assert isinstance(cfg, Qwen2Config)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
            cfg.intermediate_size, cfg.vocab_size) == (3, 96, 3, 1, 32, 200, 300)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    assert cfg.context_limit == 256 and not cfg.use_sliding_window


def test_defaults_follow_the_reference():
    minimal = {"architectures": ["Qwen2ForCausalLM"], "vocab_size": 10, "hidden_size": 24, "intermediate_size": 8,
               "num_hidden_layers": 1, "num_attention_heads": 4}
    cfg = config_from_dict(minimal)
    assert cfg.num_key_value_heads == 4          # model.rs:1352
    assert cfg.head_dim == 6                      # hidden / heads, model.rs:1367-1377
    assert cfg.rms_norm_eps == 1e-6               # model.rs:1397
    assert cfg.rope_theta == 10000.0              # model.rs:1398
    assert cfg.tie_word_embeddings is False and cfg.use_sliding_window is False


def test_head_dim_need_not_be_hidden_over_heads():
    cfg = config_from_dict(CONFIG_C)
    assert cfg.head_dim == 48 and cfg.head_dim * cfg.num_attention_heads != cfg.hidden_size
    assert config_from_dict(cfg.to_dict()).head_dim == 48


@pytest.mark.parametrize("change,needle", [
    ({"num_attention_heads": 5, "num_key_value_heads": 2, "hidden_size": 80}, "num_key_value_heads"),
    ({"head_dim": 15}, "head_dim"),
    ({"hidden_size": 70}, "hidden_size"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"rms_norm_eps": -1.0}, "rms_norm_eps"),
    ({"num_hidden_layers": -2}, "num_hidden_layers"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
])
def test_errors_name_the_key(change, needle):
    data = dict(CONFIG_A, **change)
    with pytest.raises((InvalidArgumentError, UnsupportedError)) as err:
        config_from_dict(data)
    assert needle in str(err.value)


def test_a_missing_required_key_is_named():
    data = dict(CONFIG_A)
    del data["intermediate_size"]
    with pytest.raises(InvalidArgumentError, match="intermediate_size"):
        config_from_dict(data)


def test_unknown_architecture_lists_the_registered_ones():
    with pytest.raises(UnsupportedError) as err:
        config_from_dict(dict(CONFIG_A, architectures=["LlamaForCausalLM"]))
    assert "LlamaForCausalLM" in str(err.value) and "Qwen2ForCausalLM" in str(err.value)
    with pytest.raises(InvalidArgumentError, match="architectures"):
        config_from_dict({"vocab_size": 3})


def test_registry_is_open():
    class Other(Qwen2Config):
        architecture = "OtherForCausalLM"

    register_architecture("OtherForCausalLM", Other, lambda config, runtime: None)
    try:
        assert "OtherForCausalLM" in architecture_names()
        assert lookup_architecture("OtherForCausalLM")[0] is Other
        assert isinstance(config_from_dict(dict(CONFIG_A, architectures=["OtherForCausalLM"])), Other)
    finally:
        unregister_architecture("OtherForCausalLM")
    assert "OtherForCausalLM" not in architecture_names()


def test_layers_are_described_one_by_one_with_their_windows():
    cfg = config_from_dict(CONFIG_D)
    specs = cfg.layer_specs()
    assert [s.mixer.params["window"] for s in specs] == [0, 21, 21]   # the first max_window_layers see everything
    assert all(s.mixer.kind == "attention" and s.ffn.kind == "gated_mlp" and s.block == "prenorm" for s in specs)
    assert specs[2].prefix == "model.layers.2." and specs[0].position.params["base"] == 1e6
    assert [e.layer for e in cfg.schedule()] == [0, 1, 2] and all(e.cache_of is None for e in cfg.schedule())
    assert [s.mixer.params["window"] for s in config_from_dict(CONFIG_A).layer_specs()] == [0, 0]
    assert [s.mixer.params["window"] for s in config_from_dict(CONFIG_B).layer_specs()] == [0, 0, 0]   # switched off


def test_round_trip_through_a_folder(tmp_path):
    cfg = config_from_dict(CONFIG_B)
    cfg.save(str(tmp_path))
    again = load_config(str(tmp_path))
    assert again == cfg
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ParseError):
        load_config(str(tmp_path))
    with pytest.raises(IoError):
        load_config(str(tmp_path / "absent"))


def test_eos_ids_from_the_file():
    assert config_from_dict(dict(CONFIG_A, eos_token_id=7)).eos_token_ids == (7,)
    assert config_from_dict(dict(CONFIG_A, eos_token_id=[7, 9])).eos_token_ids == (7, 9)
    with pytest.raises(InvalidArgumentError, match="eos_token_id"):
        config_from_dict(dict(CONFIG_A, eos_token_id="</s>"))
