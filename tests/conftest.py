import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny Qwen3 configurations that differ in every size and option.
TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=256, hidden_size=64,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, max_position_embeddings=256, rms_norm_eps=1e-6, rope_theta=10000.0,
    tie_word_embeddings=True, attention_bias=False, hidden_act="silu", use_sliding_window=False)
TINY_A_INIT = dict(seed=0, std=0.02, embedding_std=0.02, norm_jitter=0.01)
TINY_A_PAGE = 16

TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=384, hidden_size=96,
    num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    intermediate_size=160, max_position_embeddings=512, rms_norm_eps=1e-5, rope_theta=1000000.0,
    tie_word_embeddings=False, attention_bias=False, hidden_act="silu", use_sliding_window=False)
TINY_B_INIT = dict(seed=1, std=0.03, embedding_std=0.05, norm_jitter=0.02)
TINY_B_PAGE = 32

# sizes that are no power of two anywhere: 5 heads over 5 kv heads (no grouping), head size 48
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=331, hidden_size=120,
    num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5, head_dim=48,
    intermediate_size=200, max_position_embeddings=320, rms_norm_eps=3e-6, rope_theta=50000.0,
    tie_word_embeddings=False)
TINY_C_INIT = dict(seed=2, std=0.04, embedding_std=0.04, norm_jitter=0.05)


def make_folder(tmp_path_factory, name, raw, init, dtype="bfloat16"):
    import return_amd.models  # noqa: F401
    from return_amd.config import lookup_architecture
    from return_amd.weights import write_model_folder
    cls, _ = lookup_architecture(raw["architectures"][0])
    cfg = cls.from_dict(raw)
    folder = str(tmp_path_factory.mktemp(name))
    write_model_folder(folder, cfg, dtype=dtype, **init)
    return folder


@pytest.fixture(scope="session")
def folder_a(tmp_path_factory):
    return make_folder(tmp_path_factory, "tiny_a", TINY_A, TINY_A_INIT)


@pytest.fixture(scope="session")
def folder_b(tmp_path_factory):
    return make_folder(tmp_path_factory, "tiny_b", TINY_B, TINY_B_INIT)


@pytest.fixture(scope="session")
def folder_c(tmp_path_factory):
    return make_folder(tmp_path_factory, "tiny_c", TINY_C, TINY_C_INIT)
