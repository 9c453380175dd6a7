import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 512, "attention_bias": False, "hidden_act": "silu",
    "eos_token_id": 3,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 160, "vocab_size": 389, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 640, "attention_bias": False, "hidden_act": "silu",
    "eos_token_id": 7,
}
# a third one with projection biases (and therefore no q/k norms) and a head size that is no power of two
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "intermediate_size": 112, "vocab_size": 301, "rope_theta": 50000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 384, "attention_bias": True, "hidden_act": "silu",
}
# the head size and group size of the real family (128, 4 query heads per key/value head), otherwise small
SMALL_D = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 512, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 128, "intermediate_size": 1536, "vocab_size": 2048, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 1024, "attention_bias": False, "hidden_act": "silu",
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (SMALL_D, 3)}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder with config.json and model.safetensors (bfloat16 random weights)."""
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    out = {}
    for name, (cfg, seed) in TINY.items():
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(str(folder), cfg, seed)
        out[name] = str(folder)
    return out


@pytest.fixture()
def emulated_kernels():
    """Installs the CPU stand-in for the kernel library for one test."""
    from nanohybrid_vlm_amd.native import ops
    from emulated_kernels import EmulatedBackend
    old = ops._backend
    ops.set_backend(EmulatedBackend())
    yield
    ops.set_backend(old)


def require_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU here")
