"""Weight loading by name, its one error, and the random-weights mode (CPU)."""
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import return_amd.models  # noqa: F401
from return_amd.config import Qwen3Config, lookup_architecture
from return_amd.weights import WeightError, load_weights, random_weights, write_model_folder
from tests.conftest import TINY_A, TINY_A_INIT, TINY_B, TINY_B_INIT


def spec_of(raw):
    cfg = Qwen3Config.from_dict(raw)
    return cfg, lookup_architecture(cfg.architecture)[1](cfg)


def test_folder_round_trip(tmp_path):
    cfg, spec = spec_of(TINY_B)
    write_model_folder(str(tmp_path), cfg, **TINY_B_INIT)
    assert sorted(os.listdir(tmp_path)) == ["config.json", "model.safetensors"]
    w = load_weights(str(tmp_path), spec)
    want = random_weights(spec, **TINY_B_INIT)
    assert set(w) == set(want) == set(spec.expected_tensors())
    for k in w:
        assert w[k].dtype == torch.bfloat16 and torch.equal(w[k], want[k])
    assert w["model.layers.2.self_attn.q_proj.weight"].shape == (192, 96)
    assert w["lm_head.weight"].shape == (384, 96)


def test_seed_decides_everything():
    _, spec = spec_of(TINY_A)
    a, b, c = random_weights(spec, seed=5), random_weights(spec, seed=5), random_weights(spec, seed=6)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert any(not torch.equal(a[k], c[k]) for k in a)


def test_distributions():
    _, spec = spec_of(TINY_B)
    w = random_weights(spec, seed=1, std=0.03, embedding_std=0.05, norm_jitter=0.02, dtype="float32")
    assert abs(w["model.layers.0.mlp.gate_proj.weight"].std().item() - 0.03) < 0.003
    assert abs(w["model.embed_tokens.weight"].std().item() - 0.05) < 0.004
    n = w["model.layers.1.input_layernorm.weight"]
    assert abs(n.mean().item() - 1.0) < 0.01 and 0.005 < n.std().item() < 0.04


def test_one_error_lists_missing_unexpected_and_misshaped(tmp_path):
    cfg, spec = spec_of(TINY_A)
    write_model_folder(str(tmp_path), cfg, **TINY_A_INIT)
    path = os.path.join(tmp_path, "model.safetensors")
    t = load_file(path)
    del t["model.layers.1.mlp.down_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path), spec)
    msg = str(e.value)
    assert e.value.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert e.value.misshaped[0][0] == "model.layers.0.self_attn.k_proj.weight"
    for word in ("missing", "unexpected", "wrong shape", "(16, 64)", "(32, 64)", "down_proj", "inv_freq"):
        assert word in msg


def test_tied_model_accepts_a_stored_head_and_untied_needs_it(tmp_path):
    cfg, spec = spec_of(TINY_A)                      # tied
    write_model_folder(str(tmp_path), cfg, **TINY_A_INIT)
    path = os.path.join(tmp_path, "model.safetensors")
    t = load_file(path)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, path)
    w = load_weights(str(tmp_path), spec)
    assert "lm_head.weight" not in w
    cfg_b, spec_b = spec_of(dict(TINY_A, tie_word_embeddings=False))
    del t["lm_head.weight"]
    save_file(t, path)
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(str(tmp_path), spec_b)


def test_stored_precision_is_kept(tmp_path):
    cfg, spec = spec_of(TINY_A)
    write_model_folder(str(tmp_path), cfg, **TINY_A_INIT)
    path = os.path.join(tmp_path, "model.safetensors")
    t = load_file(path)
    t["model.norm.weight"] = t["model.norm.weight"].float() + 1e-4          # not a bf16 value
    t["model.layers.0.self_attn.q_norm.weight"] = t["model.layers.0.self_attn.q_norm.weight"].to(torch.float16)
    save_file(t, path)
    w = load_weights(str(tmp_path), spec)
    assert w["model.norm.weight"].dtype == torch.float32
    assert torch.equal(w["model.norm.weight"], t["model.norm.weight"])
    assert w["model.layers.0.self_attn.q_norm.weight"].dtype == torch.float32
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_sharded_checkpoint(tmp_path):
    import json
    cfg, spec = spec_of(TINY_A)
    write_model_folder(str(tmp_path), cfg, **TINY_A_INIT)
    path = os.path.join(tmp_path, "model.safetensors")
    t = load_file(path)
    os.remove(path)
    names = sorted(t)
    halves = {"model-00001-of-00002.safetensors": names[:len(names) // 2],
              "model-00002-of-00002.safetensors": names[len(names) // 2:]}
    for f, ns in halves.items():
        save_file({n: t[n] for n in ns}, os.path.join(tmp_path, f))
    with open(os.path.join(tmp_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {n: fn for fn, ns in halves.items() for n in ns}}, f)
    w = load_weights(str(tmp_path), spec)
    assert all(torch.equal(w[k], t[k]) for k in t)


def test_missing_files(tmp_path):
    _, spec = spec_of(TINY_A)
    with pytest.raises(FileNotFoundError):
        load_weights(str(tmp_path), spec)
