"""Configuration and registry (CPU)."""
import json

import pytest

import return_amd.models  # noqa: F401
from return_amd.config import (ConfigError, EngineConfig, Qwen3Config, load_config, lookup_architecture,
                               registered_architectures)
from tests.conftest import TINY_A, TINY_B


def test_reads_every_size_from_config_json():
    a, b = Qwen3Config.from_dict(TINY_A), Qwen3Config.from_dict(TINY_B)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)
    assert (b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (96, 6, 1, 32)
    assert b.q_width == 192 != b.hidden_size and b.kv_width == 32
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert a.rms_norm_eps == 1e-6 and b.rms_norm_eps == 1e-5
    assert a.rope_theta == 10000.0 and b.rope_theta == 1e6


def test_defaults_of_optional_keys():
    raw = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "num_key_value_heads", "tie_word_embeddings")}
    c = Qwen3Config.from_dict(raw)
    assert c.head_dim == 64 // 4                      # rollout/monkey_patch/qwen3.py:117
    assert c.num_key_value_heads == 4
    assert c.tie_word_embeddings is False


def test_constants_of_the_model_have_no_stand_in():
    """The norms' eps and the rotation's base are the model's own: a config.json without them is refused."""
    for key in ("rms_norm_eps", "rope_theta"):
        with pytest.raises(ConfigError, match=key):
            Qwen3Config.from_dict({k: v for k, v in TINY_A.items() if k != key})


def test_rotation_base_in_either_layout():
    """rope_theta at the top level, or inside rope_parameters as newer config.json files have it; a
    config.json of the second kind must not run with another base, and its rope_type is checked too."""
    base = {k: v for k, v in TINY_B.items() if k != "rope_theta"}
    new = Qwen3Config.from_dict(dict(base, rope_parameters={"rope_theta": 1000000.0, "rope_type": "default"}))
    assert new.rope_theta == TINY_B["rope_theta"] == 1e6
    assert new == Qwen3Config.from_dict(TINY_B)
    both = Qwen3Config.from_dict(dict(TINY_B, rope_parameters={"rope_theta": 1e6, "rope_type": "default"}))
    assert both.rope_theta == 1e6
    with pytest.raises(ConfigError, match="rope_theta"):
        Qwen3Config.from_dict(dict(TINY_B, rope_parameters={"rope_theta": 5e5}))          # two different bases
    with pytest.raises(ConfigError, match="rope_theta"):
        Qwen3Config.from_dict(dict(base, rope_parameters={"rope_type": "default"}))       # none at all
    with pytest.raises(ConfigError, match="rope_parameters"):
        Qwen3Config.from_dict(dict(base, rope_parameters={"rope_theta": 1e6, "rope_type": "yarn", "factor": 4.0}))
    with pytest.raises(ConfigError, match="rope_parameters"):
        Qwen3Config.from_dict(dict(base, rope_parameters="default"))


def test_json_numbers_are_coerced():
    c = Qwen3Config.from_dict(dict(TINY_B, rope_theta=1000000, vocab_size=384.0))
    assert isinstance(c.rope_theta, float) and isinstance(c.vocab_size, int)
    with pytest.raises(ConfigError, match="vocab_size"):
        Qwen3Config.from_dict(dict(TINY_B, vocab_size=38.5))


@pytest.mark.parametrize("change,word", [
    (dict(use_sliding_window=True), "sliding"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 4.0}), "rope_scaling"),
    (dict(num_key_value_heads=3), "multiple"),
    (dict(head_dim=15), "even"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(model_type="llama"), "model_type"),
    (dict(num_hidden_layers=0), "num_hidden_layers"),
])
def test_unsupported_options_are_refused(change, word):
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(dict(TINY_A, **change))


def test_default_rope_scaling_is_accepted():
    Qwen3Config.from_dict(dict(TINY_A, rope_scaling=None))
    Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"rope_type": "default"}))


def test_missing_keys_are_listed_together():
    raw = {k: v for k, v in TINY_A.items() if k not in ("vocab_size", "intermediate_size")}
    with pytest.raises(ConfigError) as e:
        Qwen3Config.from_dict(raw)
    assert "vocab_size" in str(e.value) and "intermediate_size" in str(e.value)


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    cls, build_spec = lookup_architecture("Qwen3ForCausalLM")
    assert cls is Qwen3Config
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):      # the error names what is registered
        lookup_architecture("LlamaForCausalLM")
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    cfg = load_config(str(tmp_path))
    assert isinstance(cfg, Qwen3Config) and cfg.num_hidden_layers == 3
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_B, architectures=["Nope"])))
    with pytest.raises(ConfigError, match="Nope"):
        load_config(str(tmp_path))


def test_round_trip(tmp_path):
    c = Qwen3Config.from_dict(TINY_B)
    c.save(str(tmp_path))
    assert load_config(str(tmp_path)) == c


def test_spec_follows_the_configuration():
    _, build_spec = lookup_architecture("Qwen3ForCausalLM")
    for raw in (TINY_A, TINY_B):
        cfg = Qwen3Config.from_dict(raw)
        spec = build_spec(cfg)
        assert len(spec.blocks) == cfg.num_hidden_layers == len(spec.schedule)
        m = spec.blocks[0].part("mixer").params
        assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == (
            cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim)
        assert spec.blocks[0].part("mixer_norm").params["eps"] == cfg.rms_norm_eps
        assert spec.positions["rotary"].params["theta"] == cfg.rope_theta
        tied = spec.head.tensors["weight"] == spec.embedding.tensors["weight"]
        assert tied == cfg.tie_word_embeddings
        names = spec.expected_tensors()
        assert ("lm_head.weight" in names) == (not cfg.tie_word_embeddings)
        assert names["model.layers.0.self_attn.q_proj.weight"][0] == (cfg.q_width, cfg.hidden_size)
        assert names["model.layers.0.self_attn.k_norm.weight"][0] == (cfg.head_dim,)


def test_engine_config():
    ec = EngineConfig(dtype="bf16", page_size=16, max_token=100)
    assert ec.dtype == "bfloat16" and ec.num_pages == 6
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(page_size=32, max_token=16)
