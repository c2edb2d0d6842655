"""Configuration and registry (no GPU)."""
import json

import pytest

from torchless_rs_amd.config import (ConfigError, MistralConfig, config_from_dict, load_config,
                                     register_architecture, registered_architectures,
                                     unregister_architecture)
from torchless_rs_amd.models import model_spec_for
from util import TINY_A, TINY_B


def test_every_key_is_read():
    c = config_from_dict(dict(TINY_B, bos_token_id=1, eos_token_id=2, torch_dtype="bfloat16"))
    assert isinstance(c, MistralConfig)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads) == (3, 96, 6, 1)
    assert (c.head_dim, c.intermediate_size, c.vocab_size) == (32, 224, 384)
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-6 and c.sliding_window is None
    assert c.max_position_embeddings == 128 and c.tie_word_embeddings is False
    assert c.bos_token_id == 1 and c.eos_token_ids == [2] and c.torch_dtype == "bfloat16"


def test_defaults_and_derived():
    # the parse of the reference's own test: 4096/14336/32/32/8/32000 (safetensors.rs:843-870)
    c = config_from_dict({"architectures": ["MistralForCausalLM"], "hidden_size": 4096,
                          "intermediate_size": 14336, "num_hidden_layers": 32,
                          "num_attention_heads": 32, "num_key_value_heads": 8, "vocab_size": 32000,
                          "max_position_embeddings": 4096, "rope_theta": 10000.0, "rms_norm_eps": 1e-5})
    assert c.head_dim == 128 and c.sliding_window is None and c.eos_token_ids == []
    c = config_from_dict({"architectures": ["MistralForCausalLM"], "hidden_size": 64,
                          "intermediate_size": 8, "num_hidden_layers": 1, "num_attention_heads": 4,
                          "vocab_size": 10, "rms_norm_eps": 1e-5})
    assert c.num_key_value_heads == 4 and c.rope_theta == 10000.0       # KV heads default to heads
    assert config_from_dict(dict(TINY_A, sliding_window=0)).sliding_window is None
    assert config_from_dict(dict(TINY_A, eos_token_id=[2, 7])).eos_token_ids == [2, 7]
    assert config_from_dict(dict(TINY_A, foo=3)).extra == {"foo": 3}


def test_round_trip_through_dict():
    c = config_from_dict(dict(TINY_B, eos_token_id=2))
    assert config_from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change, word", [
    ({"hidden_size": None}, "hidden_size"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"num_attention_heads": 5}, "head_dim"),                 # 64 / 5 and no head_dim
    ({"num_key_value_heads": 3}, "num_key_value_heads"),       # 4 % 3
    ({"head_dim": 15}, "even"),
    ({"head_dim": 258}, "up to 256"),                           # beyond what the attention kernels take
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "linear", "factor": 2}}, "rope_scaling"),
    ({"quantization_config": {"quant_method": "gptq"}}, "quantized"),
    ({"rms_norm_eps": -1.0}, "rms_norm_eps"),
    ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
    ({"sliding_window": -4}, "sliding_window"),
    ({"eos_token_id": "two"}, "eos_token_id"),
])
def test_errors(change, word):
    d = dict(TINY_A)
    for k, v in change.items():
        if v is None:
            d.pop(k)
        else:
            d[k] = v
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_unknown_architecture_lists_the_known():
    with pytest.raises(ConfigError, match="MistralForCausalLM"):
        config_from_dict(dict(TINY_A, architectures=["NopeForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_load_config_from_folder(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert load_config(str(tmp_path)).sliding_window == 8


def test_registry_takes_a_new_architecture():
    from torchless_rs_amd.config.base import ModelConfig

    class C(ModelConfig):
        @classmethod
        def from_dict(cls, d):
            return cls(architecture="ToyForCausalLM")

    register_architecture("ToyForCausalLM", C, lambda cfg: "spec")
    try:
        assert "ToyForCausalLM" in registered_architectures()
        c = config_from_dict({"architectures": ["ToyForCausalLM"]})
        assert model_spec_for(c) == "spec"
    finally:
        unregister_architecture("ToyForCausalLM")


def test_spec_follows_the_configuration():
    for cfgd in (TINY_A, TINY_B):
        c = config_from_dict(cfgd)
        spec = model_spec_for(c)
        ws = spec.weight_specs()
        assert len(ws) == 3 + 9 * c.num_hidden_layers                    # src/model/mod.rs:360-369, 392-414
        assert ws["model.layers.0.self_attn.q_proj.weight"].shape == (
            c.num_attention_heads * c.head_dim, c.hidden_size)
        assert ws["model.layers.0.self_attn.o_proj.weight"].shape == (
            c.hidden_size, c.num_attention_heads * c.head_dim)
        assert ws["model.layers.0.self_attn.k_proj.weight"].shape == (
            c.num_key_value_heads * c.head_dim, c.hidden_size)
        assert ws["lm_head.weight"].shape == (c.vocab_size, c.hidden_size)
        assert [r.layer for r in spec.schedule] == list(range(c.num_hidden_layers))
        assert spec.layers[0].mixer.params["window"] == c.sliding_window
    tied = model_spec_for(config_from_dict(dict(TINY_A, tie_word_embeddings=True))).weight_specs()
    assert "lm_head.weight" not in tied
