"""Configuration: reading the architecture's own config.json keys, the registry, and what the spec says."""
import json

import pytest

from conftest import TINY_A, TINY_B, TINY_W
from vt_transformer_amd.config import (ConfigError, ModelSpec, PartSpec, Qwen2Config, ScheduleEntry,
                                       config_from_dict, load_config, register_architecture)
from vt_transformer_amd.config.base import LayerSpec, ModelConfig


def test_qwen2_keys_are_read():
    c = config_from_dict(dict(TINY_B))
    assert isinstance(c, Qwen2Config)
    assert (c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (320, 96, 200, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 3, 32)
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-5 and c.tie_word_embeddings is False


def test_defaults_of_absent_keys():
    d = dict(architectures=["Qwen2ForCausalLM"], vocab_size=10, hidden_size=32, intermediate_size=8,
             num_hidden_layers=1, num_attention_heads=4)
    c = config_from_dict(d)
    assert c.num_key_value_heads == 4          # = heads
    assert c.head_dim == 8                     # = hidden / heads
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 1e6 and c.tie_word_embeddings is False
    assert c.eos_token_id == []


def test_head_dim_need_not_divide_hidden():
    d = dict(TINY_A, head_dim=48)
    c = config_from_dict(d)
    spec = c.to_spec()
    assert spec.layers[0].mixer.params["head_dim"] == 48


@pytest.mark.parametrize("change,word", [
    ({"vocab_size": None}, "vocab_size"),
    ({"hidden_size": "64"}, "hidden_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"architectures": ["LlamaForCausalLM"]}, "not registered"),
    ({"architectures": []}, "architectures"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"head_dim": 15}, "head_dim"),
])
def test_bad_configs_are_refused_with_the_key_named(change, word):
    d = dict(TINY_A)
    d.update(change)
    d = {k: v for k, v in d.items() if v is not None or k in ("sliding_window",)}
    with pytest.raises(ConfigError) as e:
        config_from_dict(d)
    assert word in str(e.value)


def test_eos_may_be_a_list():
    assert config_from_dict(dict(TINY_A, eos_token_id=[5, 7])).to_spec().eos_token_ids == [5, 7]
    assert config_from_dict(dict(TINY_A, eos_token_id=9)).to_spec().eos_token_ids == [9]


def test_spec_of_qwen2():
    spec = config_from_dict(dict(TINY_W)).to_spec()
    assert len(spec.layers) == 4 and [e.layer for e in spec.schedule] == [0, 1, 2, 3]
    assert [l.mixer.params["window"] for l in spec.layers] == [0, 0, 40, 40]   # window from max_window_layers on
    m = spec.layers[1].mixer.params
    assert (m["num_heads"], m["num_kv_heads"], m["head_dim"], m["qkv_bias"], m["out_bias"]) == (5, 1, 48, True, False)
    assert m["position"].kind == "rotary" and m["position"].params == {"theta": 50000.0, "dim": 48}
    assert spec.layers[0].norms["input"].params["eps"] == 3e-6
    assert spec.layers[2].prefix == "model.layers.2."
    assert spec.head.params["tied_to"] is None
    assert config_from_dict(dict(TINY_A)).to_spec().head.params["tied_to"] == "model.embed_tokens.weight"


def test_roundtrip_through_a_folder(tmp_path):
    c = config_from_dict(dict(TINY_W))
    c.save(str(tmp_path))
    c2 = load_config(str(tmp_path))
    assert c2 == c
    with open(tmp_path / "config.json") as f:
        assert json.load(f)["architectures"] == ["Qwen2ForCausalLM"]
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "nothing"))


def test_schedule_is_checked():
    spec = config_from_dict(dict(TINY_A)).to_spec()
    ok = ModelSpec(**{**spec.__dict__, "schedule": [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, cache_from=1),
                                                    ScheduleEntry(0)]})
    ok.validate()     # a layer may run twice, and an entry may read an earlier entry's cache
    for bad in ([ScheduleEntry(2)], [ScheduleEntry(0, cache_from=0)], [ScheduleEntry(0), ScheduleEntry(1, cache_from=2)],
                [ScheduleEntry(0), ScheduleEntry(1, cache_from=0), ScheduleEntry(0, cache_from=1)]):
        with pytest.raises(ConfigError):
            ModelSpec(**{**spec.__dict__, "schedule": bad}).validate()


def test_another_architecture_can_be_registered():
    class ToyConfig(ModelConfig):
        architecture = "ToyForCausalLM"

        def __init__(self, n):
            self.n = n

        @classmethod
        def from_dict(cls, d):
            return cls(d["n_layer"])

    register_architecture("ToyForCausalLM", ToyConfig)
    c = config_from_dict({"architectures": ["ToyForCausalLM"], "n_layer": 3})
    assert isinstance(c, ToyConfig) and c.n == 3
