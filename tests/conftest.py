import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real GPU (run on the MI355X box)")


# Two tiny configurations that differ in every size and option, and a third with a window.
TINY_A = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=256, hidden_size=64, intermediate_size=128,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16, rope_theta=10000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=1024, hidden_act="silu",
    use_sliding_window=False, torch_dtype="bfloat16")
TINY_B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=320, hidden_size=96, intermediate_size=200,
    num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=3, head_dim=32, rope_theta=1000000.0,
    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=2048, hidden_act="silu",
    use_sliding_window=False, torch_dtype="bfloat16")
# window on the upper layers only, odd group of 5 query heads per kv head, width that is no multiple of 64
TINY_W = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=203, hidden_size=80, intermediate_size=112,
    num_hidden_layers=4, num_attention_heads=5, num_key_value_heads=1, head_dim=48, rope_theta=50000.0,
    rms_norm_eps=3e-6, tie_word_embeddings=False, max_position_embeddings=1024, hidden_act="silu",
    use_sliding_window=True, sliding_window=40, max_window_layers=2, torch_dtype="bfloat16")

TINY = {"A": TINY_A, "B": TINY_B, "W": TINY_W}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders with random weights, written once per session into a temporary place."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("models")
    out = {}
    for i, (name, cfg) in enumerate(TINY.items()):
        folder = str(root / name)
        write_random_model(config_from_dict(dict(cfg)), folder, seed=100 + i)
        out[name] = folder
    return out
