"""Configuration: typed parsing of config.json keys, validation, the registry."""
import json
import os

import pytest

import tiny
from zinfer_amd import ConfigError, UnsupportedModelType
from zinfer_amd.config import (Qwen3Config, entry_for, load_config, register_architecture,
                               registered_architectures, unregister_architecture)


def test_qwen3_keys_are_typed_and_required():
    cfg = Qwen3Config.from_dict(tiny.TINY_B)
    assert cfg.head_dim == 32 and cfg.num_attention_heads * cfg.head_dim != cfg.hidden_size
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    for key in ("head_dim", "hidden_size", "intermediate_size", "max_position_embeddings",
                "model_type", "num_attention_heads", "num_hidden_layers", "num_key_value_heads",
                "rms_norm_eps", "rope_theta", "tie_word_embeddings", "torch_dtype", "vocab_size"):
        raw = dict(tiny.TINY_B)
        del raw[key]
        with pytest.raises(ConfigError, match=key):
            Qwen3Config.from_dict(raw)           # no default, as in the reference's struct
    raw = dict(tiny.TINY_B, some_unknown_key=1)
    Qwen3Config.from_dict(raw)                    # unknown keys are ignored


@pytest.mark.parametrize("key,value", [
    ("hidden_size", "64"), ("hidden_size", 1.5), ("head_dim", -16), ("vocab_size", True),
    ("rms_norm_eps", "tiny"), ("tie_word_embeddings", 1), ("architectures", "Qwen3ForCausalLM")])
def test_wrong_types_are_refused(key, value):
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(dict(tiny.TINY_A, **{key: value}))


@pytest.mark.parametrize("change,word", [
    (dict(num_key_value_heads=3), "InvalidGrouping"), (dict(head_dim=15), "InvalidHeadDim"),
    (dict(hidden_size=0), "InvalidDimensions"), (dict(num_attention_heads=0), "InvalidDimensions"),
    (dict(use_sliding_window=True), "use_sliding_window"), (dict(attention_bias=True), "bias"),
    (dict(hidden_act="gelu"), "hidden_act"), (dict(rope_scaling={"type": "yarn"}), "rope_scaling"),
    (dict(rope_theta=0.0), "rope_theta")])
def test_values_the_formulas_do_not_cover_are_refused(change, word):
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(dict(tiny.TINY_A, **change))


def test_model_spec_carries_every_size():
    spec = Qwen3Config.from_dict(tiny.TINY_C).model_spec()
    assert len(spec.layers) == 2 and [e.layer for e in spec.schedule] == [0, 1]
    attn = spec.layers[0].mixer
    assert (attn.n_heads, attn.n_kv_heads, attn.head_dim, attn.window) == (3, 1, 48, None)
    assert attn.qk_norm_eps == 3e-6 and attn.position.theta == 50000.0
    assert attn.position.max_positions == 384
    assert spec.layers[0].feed_forward.intermediate_size == 112
    assert spec.final_norm.eps == 3e-6 and spec.vocab_size == 777
    assert spec.eos_token_ids == (151645, 151643)   # families/qwen3/generation_policy.zig:3-6


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert entry_for({"model_type": "qwen3"}).config_type is Qwen3Config
    assert entry_for({"architectures": ["Qwen3ForCausalLM"]}).config_type is Qwen3Config
    with pytest.raises(ConfigError, match="MissingModelType"):
        entry_for({})
    with pytest.raises(ConfigError, match="InvalidModelType"):
        entry_for({"model_type": 3})
    with pytest.raises(UnsupportedModelType):
        entry_for({"model_type": "llama"})
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    assert load_config(str(tmp_path)).hidden_size == 64
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "nowhere"))

    class Other:
        @classmethod
        def from_dict(cls, raw):
            return cls()
    register_architecture("OtherForCausalLM", Other, model_type="other")
    try:
        assert entry_for({"model_type": "other"}).config_type is Other
    finally:
        unregister_architecture("OtherForCausalLM")
    with pytest.raises(UnsupportedModelType):
        entry_for({"model_type": "other"})


def test_to_dict_round_trip():
    cfg = Qwen3Config.from_dict(tiny.TINY_B)
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
