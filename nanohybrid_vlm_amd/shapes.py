"""Named configurations for measurements and examples: config.json contents of the
Qwen3 sizes that the benchmarks use, and two tiny ones. Only the command line and
``bench.py`` read these; the engine itself takes every size from a config.json."""
from __future__ import annotations


def _qwen3(layers, hidden, heads, kv_heads, head_dim, inter, vocab=151936, theta=1000000.0, eps=1e-6, tie=False,
           max_pos=40960):
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": layers,
        "hidden_size": hidden, "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
        "intermediate_size": inter, "vocab_size": vocab, "rope_theta": theta, "rms_norm_eps": eps,
        "tie_word_embeddings": tie, "max_position_embeddings": max_pos, "attention_bias": False, "hidden_act": "silu",
        "eos_token_id": 151645 if vocab > 151645 else 0, "torch_dtype": "bfloat16",
    }


SHAPES = {
    "tinyA": _qwen3(2, 64, 4, 2, 16, 128, vocab=256, theta=10000.0, eps=1e-6, tie=True, max_pos=128),
    "tinyB": _qwen3(3, 96, 6, 1, 32, 160, vocab=389, theta=1000000.0, eps=1e-5, tie=False, max_pos=256),
    "8b": _qwen3(36, 4096, 32, 8, 128, 12288),
    "14b": _qwen3(40, 5120, 40, 8, 128, 17408),
    "32b": _qwen3(64, 5120, 64, 8, 128, 25600),
}
