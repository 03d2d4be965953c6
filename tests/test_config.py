"""Configuration and registry: typed reading of config.json, defaults, errors."""
import json

import pytest

from infernum_amd.config import (ConfigError, LlamaConfig, UnsupportedModelError, config_from_dict, load_config,
                                 register_architecture, registered_architectures)

import tiny_models as TM

MIN = dict(vocab_size=100, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4)


def test_defaults_follow_the_reference():
    # infernum-llama/src/config.rs:104-126: kv heads = heads, eps 1e-5, theta 1e4, 2048 positions, bos 1, eos 2
    c = LlamaConfig.from_dict(MIN)
    assert c.model_type == "llama"
    assert c.num_kv_heads == 4 and c.head_dim == 16 and c.num_heads_per_kv == 1
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0 and c.max_position_embeddings == 2048
    assert c.bos_token_id == 1 and c.eos_token_id == 2 and c.tie_word_embeddings is False
    assert c.rope_scaling is None and c.effective_sliding_window(0) is None


def test_every_key_is_read():
    c = TM.tiny_config("B")
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_kv_heads) == (3, 128, 4, 1)
    assert (c.head_dim, c.intermediate_size, c.vocab_size) == (32, 352, 384)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.max_position_embeddings == 256
    s = c.rope_scaling
    assert (s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == (8.0, 1.0, 4.0, 64)


def test_eos_list_takes_first():
    # infernum-llama/src/config.rs:64-68
    assert LlamaConfig.from_dict(dict(MIN, eos_token_id=[7, 8, 9])).eos_token_id == 7


def test_explicit_head_dim_and_window():
    c = TM.tiny_config("C")
    assert c.head_dim == 48 and c.hidden_size // c.num_attention_heads == 16
    assert [c.effective_sliding_window(i) for i in range(3)] == [24, 24, None]
    assert LlamaConfig.from_dict(dict(MIN, sliding_window=8)).effective_sliding_window(0) is None   # flag is off


def test_round_trip_through_config_json(tmp_path):
    for name in ("A", "B", "C"):
        c = TM.tiny_config(name)
        (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
        assert load_config(str(tmp_path)) == c


@pytest.mark.parametrize("key", sorted(MIN))
def test_missing_required_key(key):
    raw = dict(MIN)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(raw)


@pytest.mark.parametrize("patch,needle", [
    (dict(hidden_size="64"), "hidden_size"),
    (dict(hidden_size=0), "hidden_size"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(rms_norm_eps="tiny"), "rms_norm_eps"),
    (dict(rope_theta=-1.0), "rope_theta"),
    (dict(tie_word_embeddings="yes"), "tie_word_embeddings"),
    (dict(num_attention_heads=3), "multiple of num_attention_heads"),
    (dict(num_key_value_heads=3), "multiple of num_key_value_heads"),
    (dict(head_dim=15), "even"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(use_sliding_window=True), "sliding_window"),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), "yarn"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=4.0, high_freq_factor=1.0,
                            original_max_position_embeddings=64)), "high_freq_factor"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=8.0)), "low_freq_factor"),
    (dict(rope_scaling=[1, 2]), "rope_scaling"),
])
def test_bad_values_name_their_key(patch, needle):
    with pytest.raises(ConfigError, match=needle):
        LlamaConfig.from_dict(dict(MIN, **patch))


def test_unknown_model_type_lists_the_supported():
    # infernum-llama/src/config.rs:148-157
    with pytest.raises(UnsupportedModelError, match='Unsupported model_type: "gpt9"') as e:
        config_from_dict(dict(MIN, model_type="gpt9"))
    assert "llama" in str(e.value)
    with pytest.raises(UnsupportedModelError, match="expert"):
        config_from_dict(dict(MIN, model_type="llama", num_local_experts=8))
    with pytest.raises(UnsupportedModelError, match="mixtral"):
        config_from_dict(dict(MIN, model_type="mixtral"))


def test_model_type_defaults_to_llama_and_unknown_keys_are_ignored():
    c = config_from_dict(dict(MIN, some_future_key=[1, 2, 3], torch_dtype="bfloat16"))
    assert isinstance(c, LlamaConfig)


def test_files(tmp_path):
    with pytest.raises(ConfigError, match="cannot read"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(ConfigError, match="object"):
        load_config(str(tmp_path))


def test_registry_takes_another_architecture():
    class ToyConfig:
        model_type = "toy-arch"

        @staticmethod
        def from_dict(raw, where="config.json"):
            c = ToyConfig()
            c.width = raw["width"]
            return c

    register_architecture("toy-arch", ToyConfig, lambda cfg: ("spec of width", cfg.width), replace=True)
    assert "toy-arch" in registered_architectures() and "llama" in registered_architectures()
    from infernum_amd.config import model_spec_for
    c = config_from_dict({"model_type": "toy-arch", "width": 5})
    assert model_spec_for(c) == ("spec of width", 5)
    with pytest.raises(ValueError, match="registered already"):
        register_architecture("llama", ToyConfig, lambda cfg: None)
