"""Typed configuration and the architecture registry."""
import json

import pytest

from libllm_amd import ConfigError
from libllm_amd.config import (LlamaConfig, ScheduleEntry, architectures, config_from_dict,
                               config_from_dir, register_architecture, validate_schedule)
from libllm_amd.engine import DecoderModel
from tiny import LLAMA3_MIDDLE_BAND, TINY_A, TINY_B, TINY_C


def test_every_key_is_read():
    for d in (TINY_A, TINY_B, TINY_C):
        c = config_from_dict(d)
        assert isinstance(c, LlamaConfig)
        assert (c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (
            d["hidden_size"], d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"])
        assert (c.intermediate_size, c.num_hidden_layers, c.vocab_size) == (
            d["intermediate_size"], d["num_hidden_layers"], d["vocab_size"])
        assert c.rms_norm_eps == d["rms_norm_eps"] and c.rope_theta == d["rope_theta"]
        assert c.rope_scaling == d["rope_scaling"] and c.tie_word_embeddings == d["tie_word_embeddings"]
        assert c.max_position_embeddings == d["max_position_embeddings"]
        assert config_from_dict(c.to_dict()) == c                       # config.json round trip
    assert config_from_dict(TINY_B).eos_token_ids == (7, 9)            # a list of stop tokens
    assert config_from_dict(TINY_A).eos_token_ids == (2,)


def test_defaults():
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "rope_theta",
                                                      "rope_scaling", "tie_word_embeddings", "eos_token_id",
                                                      "hidden_act", "bos_token_id")}
    c = config_from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads               # src/libllm/llama.cc:64-68
    assert c.head_dim == c.hidden_size // c.num_attention_heads         # src/libllm/llama.cc:120
    assert c.rope_theta == 10000.0 and c.rope_scaling is None
    assert c.tie_word_embeddings is False and c.attention_bias is False and c.eos_token_ids == ()


@pytest.mark.parametrize("change, word", [
    ({"model_type": "gpt2"}, "unexpected model type: gpt2"),            # src/libllm/model_for_generation.cc:45-49
    ({"model_type": None}, "model_type"),
    ({"hidden_size": None}, "hidden_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"head_dim": None, "hidden_size": 66}, "multiple"),                # src/libllm/llama.cc:117-118
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"eos_token_id": "x"}, "eos_token_id"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_scaling"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "low_freq_factor"),
])
def test_errors_name_the_key(change, word):
    d = dict(TINY_A)
    d.update(change)
    d = {k: v for k, v in d.items() if v is not None or k == "rope_scaling"}
    with pytest.raises(ConfigError) as e:
        DecoderModel(config_from_dict(d).to_spec()).blocks[0].mixer.position.inv_freq()
    assert word in str(e.value)


@pytest.mark.parametrize("params,want", LLAMA3_MIDDLE_BAND)
def test_llama3_middle_band_values(params, want):
    """The engine's frequency table at the pairs of the middle band, against numbers worked out
    apart from it (see tiny.LLAMA3_MIDDLE_BAND)."""
    from libllm_amd.parts.rope import scaled_inv_freq
    factor, low, high, orig, theta, hd = params
    got = scaled_inv_freq(hd, theta, {"rope_type": "llama3", "factor": factor, "low_freq_factor": low,
                                      "high_freq_factor": high, "original_max_position_embeddings": orig})
    for j, value in want.items():
        assert abs(float(got[j]) / value - 1.0) < 1e-12, (j, float(got[j]), value)


def test_config_from_dir(tmp_path):
    with pytest.raises(ConfigError):
        config_from_dir(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        config_from_dir(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    assert config_from_dir(str(tmp_path)).vocab_size == 1000


def test_registry_takes_another_architecture():
    class Other(LlamaConfig):
        pass
    register_architecture("other-llama", Other)
    assert "other-llama" in architectures() and "llama" in architectures()
    assert isinstance(config_from_dict(dict(TINY_A, model_type="other-llama")), Other)


def test_spec_is_data():
    spec = config_from_dict(TINY_B).to_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert (m.kind, m.n_heads, m.n_kv_heads, m.head_dim, m.window) == ("attention", 6, 1, 32, 0)
    assert m.position.kind == "rotary" and m.position.theta == 500000.0 and m.position.scaling["factor"] == 8.0
    assert spec.layers[1].feed_forward.intermediate == 512 and spec.layers[1].norms[0].eps == 1e-6
    assert spec.head.tied is False and spec.head.tensor == "lm_head.weight" and spec.stop_tokens == (7, 9)
    tied = config_from_dict(TINY_A).to_spec()
    assert tied.head.tied and tied.head.tensor == tied.embedding.tensor
    decl = DecoderModel(spec).declared()
    assert decl["model.layers.2.self_attn.k_proj.weight"].shape == (32, 192)
    assert decl["model.layers.0.mlp.down_proj.weight"].shape == (192, 512)
    assert decl["model.norm.weight"].role == "vector" and "lm_head.weight" in decl
    assert "lm_head.weight" not in DecoderModel(tied).declared()


def test_schedule_validation():
    spec = config_from_dict(TINY_A).to_spec()
    spec.schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2), ScheduleEntry(1, 1, writes=False)]
    validate_schedule(spec)                                              # a layer twice, a shared cache entry
    for bad in ([ScheduleEntry(2, 0)], [ScheduleEntry(0, 0), ScheduleEntry(1, 0)],
                [ScheduleEntry(0, 1, writes=False)], [ScheduleEntry(0, -1)]):
        spec.schedule = bad
        with pytest.raises(ConfigError):
            validate_schedule(spec)
