import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


# Two tiny configurations that differ in every size and option.
TINY_A = dict(
    architectures=["LlamaForCausalLM"], model_type="llama",
    vocab_size=256, hidden_size=64, intermediate_size=176, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128,
    rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY_B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama",
    vocab_size=333, hidden_size=96, intermediate_size=256, num_hidden_layers=3,
    num_attention_heads=3, num_key_value_heads=1, max_position_embeddings=256,
    rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=True)
TINY = {"a": (TINY_A, 16), "b": (TINY_B, 8)}  # name -> (config.json, cache page size)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> model folder with seeded random weights (stored in 32-bit)."""
    from llmserve.weights import write_random_model

    dirs = {}
    for i, (name, (cfg, _bs)) in enumerate(TINY.items()):
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(d, cfg, seed=11 + i)
        dirs[name] = d
    return dirs
