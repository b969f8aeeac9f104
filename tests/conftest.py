"""Shared fixtures: the two tiny configurations and model folders made in temporary directories."""

import os
import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (run with -m gpu on an MI355X)")


# Two configurations that differ in every size and option: layers, width, head counts and
# grouping, head size, feed-forward width (200 is no multiple of 16), vocabulary, rope theta,
# norm eps, tied or separate head, context length.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 128,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 200, "vocab_size": 384, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 256,
}
TINY = {"A": TINY_A, "B": TINY_B}
BLOCK_SIZE = {"A": 4, "B": 16}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> (folder, config) for tiny A and B with float32 weights, written once per session."""
    from tie_amd.weights.random_init import write_random_model

    out = {}
    for name, cfg in TINY.items():
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(folder, cfg, seed=11 + len(out), dtype="float32")
        out[name] = (str(folder), cfg)
    return out


@pytest.fixture(scope="session")
def model_folders_bf16(tmp_path_factory):
    from tie_amd.weights.random_init import write_random_model

    out = {}
    for name, cfg in TINY.items():
        folder = tmp_path_factory.mktemp(f"tiny_{name}_bf16")
        write_random_model(folder, cfg, seed=21 + len(out), dtype="bfloat16")
        out[name] = (str(folder), cfg)
    return out


def load_plain_weights(folder):
    """The tensors of a model folder as float64 CPU tensors, read with the safetensors package."""
    import torch
    from safetensors import safe_open

    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64)
    return weights
