"""Configuration and registry: every size comes from config.json; required keys,
defaults (src/arch/llama.rs:118-123), unsupported options and unknown
architectures give clear errors."""
import json

import pytest

from llm_rs_amd import ConfigError, LlamaConfig, config_from_dict, load_config, register_architecture
from llm_rs_amd.config import architectures
from tiny_configs import TINY_A, TINY_B


def test_tiny_configs_differ_in_every_size_and_option():
    a, b = LlamaConfig.from_dict(TINY_A), LlamaConfig.from_dict(TINY_B)
    for key in ("num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                "intermediate_size", "vocab_size", "rope_theta", "rope_scaling", "max_position_embeddings",
                "rms_norm_eps", "tie_word_embeddings"):
        assert getattr(a, key) != getattr(b, key), key
    assert a.num_attention_heads // a.num_key_value_heads != b.num_attention_heads // b.num_key_value_heads
    assert b.hidden_size & (b.hidden_size - 1) and b.intermediate_size & (b.intermediate_size - 1) and b.vocab_size & (b.vocab_size - 1)


def test_defaults_follow_the_reference():
    d = dict(architectures=["LlamaForCausalLM"], vocab_size=100, hidden_size=48, intermediate_size=64,
             num_hidden_layers=1, num_attention_heads=4, max_position_embeddings=32)
    c = config_from_dict(d)
    assert c.num_key_value_heads == 4 and c.head_dim == 12          # llama.rs:118-119
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0       # llama.rs:122-123
    assert c.rope_scaling is None and c.tie_word_embeddings is False


@pytest.mark.parametrize("key", LlamaConfig.REQUIRED)
def test_missing_required_key(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=f"missing config key: {key}"):
        config_from_dict(d)


@pytest.mark.parametrize("change,message", [
    (dict(num_key_value_heads=2), "no multiple"), (dict(head_dim=15), "even"), (dict(hidden_act="gelu"), "hidden_act"),
    (dict(attention_bias=True), "attention_bias"), (dict(mlp_bias=True), "mlp_bias"),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), "rope_scaling"), (dict(num_hidden_layers=0), "positive"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=2.0)), "rope_scaling.low_freq_factor"),
    (dict(architectures=["MambaForCausalLM"]), "unsupported architecture: MambaForCausalLM"),
    (dict(architectures=None), "architectures"),
])
def test_rejected(change, message):
    with pytest.raises(ConfigError, match=message):
        config_from_dict({**TINY_B, **change})


def test_round_trip_through_config_json(tmp_path):
    c = LlamaConfig.from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert load_config(str(tmp_path)) == c
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(str(tmp_path / "nowhere"))


def test_model_spec_holds_the_sizes_layer_by_layer():
    c = LlamaConfig.from_dict(TINY_B)
    spec = c.model_spec()
    assert len(spec.layers) == 3 and [r.layer for r in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "attention" and m.prefix == "model.layers.1.self_attn"
    assert m.params["num_heads"] == 3 and m.params["num_kv_heads"] == 1 and m.params["head_dim"] == 32
    assert m.params["position"]["theta"] == 500000.0 and m.params["position"]["scaling"]["factor"] == 8.0
    assert spec.layers[2].feed_forward.params == {"hidden_size": 96, "intermediate_size": 320}
    assert spec.final_norm.params["eps"] == 1e-6 and spec.head_name == "lm_head.weight"
    assert LlamaConfig.from_dict(TINY_A).model_spec().head_name is None


def test_another_architecture_can_be_registered():
    class Cfg:
        def __init__(self, d):
            self.d = d
    register_architecture("TestOnlyForCausalLM", Cfg)
    assert "TestOnlyForCausalLM" in architectures()
    assert isinstance(config_from_dict({"architectures": ["TestOnlyForCausalLM"]}), Cfg)
