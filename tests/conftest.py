import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Tiny configurations that differ in every size and option.
TINY = {
    # 2 layers, 4 q / 2 kv heads, head 16 (q width = hidden), tied
    "A": dict(architectures=["Qwen3ForCausalLM"], hidden_size=64, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128,
              vocab_size=256, max_position_embeddings=1024, rms_norm_eps=1e-6, rope_theta=10000.0,
              tie_word_embeddings=True),
    # 3 layers, 4 q / 1 kv head, head 32 (q width 128 != hidden 80), untied, odd vocabulary
    "B": dict(architectures=["Qwen3ForCausalLM"], hidden_size=80, num_hidden_layers=3,
              num_attention_heads=4, num_key_value_heads=1, head_dim=32, intermediate_size=208,
              vocab_size=311, max_position_embeddings=2048, rms_norm_eps=1e-5, rope_theta=1000000.0,
              tie_word_embeddings=False),
    # 2 layers, 6 q / 3 kv heads, head 48, widths that are no multiple of 8, untied
    "C": dict(architectures=["Qwen3ForCausalLM"], hidden_size=76, num_hidden_layers=2,
              num_attention_heads=6, num_key_value_heads=3, head_dim=48, intermediate_size=100,
              vocab_size=517, max_position_embeddings=4096, rms_norm_eps=3e-6, rope_theta=500000.0,
              tie_word_embeddings=False, eos_token_id=5),
    # 2 layers, 5 q / 5 kv heads (no sharing), head 20: an even head size that is no multiple of 16, which
    # the matrix-core kernels do not take (both engines run it on the scalar kernels); pages of 4
    "D": dict(architectures=["Qwen3ForCausalLM"], hidden_size=100, num_hidden_layers=2,
              num_attention_heads=5, num_key_value_heads=5, head_dim=20, intermediate_size=70,
              vocab_size=97, max_position_embeddings=512, rms_norm_eps=2e-5, rope_theta=20000.0,
              tie_word_embeddings=True),
}
PAGE_SIZE = {"A": 16, "B": 8, "C": 32, "D": 4}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """{name: folder} of random models, written once per test session into a temporary folder."""
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model
    out = {}
    for i, (name, cfg) in enumerate(TINY.items()):
        folder = str(tmp_path_factory.mktemp(f"tiny{name}"))
        # a larger spread than N(0, 0.02) so that at these widths the layers, not the embedding,
        # decide the logits
        write_random_model(folder, config_from_dict(cfg), seed=i, matrix_std=0.12, norm_std=0.2)
        out[name] = folder
    return out


@pytest.fixture(scope="session")
def plain_models(model_folders):
    from plain.qwen3_plain import PlainQwen3
    return {name: PlainQwen3(folder) for name, folder in model_folders.items()}
