"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B, TINY_C
from nanohybrid_vlm_amd.config.engine_config import EngineConfig
from nanohybrid_vlm_amd.architectures.qwen3 import Qwen3Config
from nanohybrid_vlm_amd.config.model_config import ConfigError, read_config_json
from nanohybrid_vlm_amd.config.registry import (Architecture, UnknownArchitecture, register_architecture,
                                                resolve_architecture, unregister_architecture)
from nanohybrid_vlm_amd.parts.model import DecoderModel
from nanohybrid_vlm_amd.weights.loader import WeightsError, load_weights
from nanohybrid_vlm_amd.weights.random_init import write_random_model


def test_config_reads_every_size_and_the_reference_defaults():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
            cfg.intermediate_size, cfg.vocab_size) == (3, 96, 6, 1, 32, 160, 389)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    raw = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "attention_bias", "rope_theta", "num_key_value_heads")}
    cfg = Qwen3Config.from_dict(raw)
    assert cfg.head_dim == 64 // 4            # hidden_size // heads
    assert cfg.attention_bias is True         # absent key means bias
    assert cfg.rope_theta == 1000000
    assert cfg.num_key_value_heads == 4
    # of rope_scaling only its own rope_theta is read
    cfg = Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"rope_type": "yarn", "factor": 4.0, "rope_theta": 777.0}))
    assert cfg.rope_theta == 777.0


@pytest.mark.parametrize("change,match", [
    ({"hidden_size": None}, "hidden_size"), ({"vocab_size": "many"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "multiple"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"head_dim": 15}, "even"), ({"num_hidden_layers": 0}, "positive"), ({"eos_token_id": [1, 2]}, "eos_token_id"),
])
def test_config_errors_name_the_key(change, match):
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict(dict(TINY_A, **change))


def test_registry():
    assert resolve_architecture(TINY_A).name == "Qwen3ForCausalLM"
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"          # no architectures listed
    with pytest.raises(UnknownArchitecture, match="registered"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(UnknownArchitecture, match="lists"):
        resolve_architecture({"architectures": ["SomethingElse"], "model_type": "qwen3"})
    with pytest.raises(UnknownArchitecture, match="does not go with"):
        resolve_architecture({"architectures": ["Qwen3ForCausalLM"], "model_type": "llama"})
    toy = Architecture("ToyLM", ("toy",), dict, lambda c: None, lambda c: {})
    register_architecture(toy)
    try:
        assert resolve_architecture({"architectures": ["ToyLM"]}) is toy
        with pytest.raises(ValueError, match="already"):
            register_architecture(toy)
    finally:
        unregister_architecture("ToyLM")


def test_engine_config_checks():
    assert EngineConfig(model="x", dtype="bf16").dtype == "bfloat16"
    assert EngineConfig(model="x", kvcache_block_size=4).kvcache_block_size == 4
    for bad in [dict(dtype="float16"), dict(scheduler_policy="fifo"), dict(max_prefill_wait_ms=-1),
                dict(max_num_seqs=0), dict(gpu_memory_utilization=1.5), dict(kvcache_block_size=0),
                dict(num_kvcache_blocks=0), dict(num_state_slots=-2), dict(max_graph_batch=0)]:
        with pytest.raises(ValueError):
            EngineConfig(model="x", **bad)


def _load(folder, dtype=torch.float32):
    raw = read_config_json(folder)
    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    model = DecoderModel(arch.build_spec(cfg))
    return model, load_weights(model, arch, cfg, folder, dtype, "cpu")


def test_random_model_folder_and_packing(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_B, seed=1)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    stored = load_file(os.path.join(folder, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    assert "lm_head.weight" in stored
    # the same seed gives the same file, another seed another
    again = write_random_model(str(tmp_path / "m2"), TINY_B, seed=1)
    other = write_random_model(str(tmp_path / "m3"), TINY_B, seed=2)
    k = "model.layers.1.mlp.up_proj.weight"
    assert torch.equal(load_file(os.path.join(again, "model.safetensors"))[k], stored[k])
    assert not torch.equal(load_file(os.path.join(other, "model.safetensors"))[k], stored[k])
    # distributions: matrices N(0, 0.02^2), norm weights 1 + N(0, 0.1^2)
    assert abs(stored[k].float().std().item() - 0.02) < 2e-3
    nw = stored["model.layers.0.input_layernorm.weight"].float()
    assert abs(nw.mean().item() - 1) < 0.05 and 0.05 < nw.std().item() < 0.15
    # loading packs q | k | v and gate | up by rows
    model, params = _load(folder, torch.bfloat16)
    assert all(p.dtype == torch.bfloat16 for p in params.values())
    q, kv = 6 * 32, 1 * 32
    qkv = params["layers.2.mixer.qkv.weight"]
    assert qkv.shape == (q + 2 * kv, 96)
    assert torch.equal(qkv[:q], stored["model.layers.2.self_attn.q_proj.weight"])
    assert torch.equal(qkv[q:q + kv], stored["model.layers.2.self_attn.k_proj.weight"])
    assert torch.equal(qkv[q + kv:], stored["model.layers.2.self_attn.v_proj.weight"])
    gu = params["layers.0.feed_forward.gate_up.weight"]
    assert torch.equal(gu[:160], stored["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(gu[160:], stored["model.layers.0.mlp.up_proj.weight"])
    assert model.head_weight is params["head.weight"]


def test_tied_head_and_bias(tmp_path):
    folder = write_random_model(str(tmp_path / "a"), TINY_A, seed=0)
    stored = load_file(os.path.join(folder, "model.safetensors"))
    assert "lm_head.weight" not in stored                      # tied: the file holds the embedding only
    model, params = _load(folder)
    assert model.head_weight is model.embed_weight
    # a tied checkpoint that repeats the embedding as lm_head.weight is accepted too
    stored["lm_head.weight"] = stored["model.embed_tokens.weight"].clone()
    save_file(stored, os.path.join(folder, "model.safetensors"))
    model, params = _load(folder)
    assert model.head_weight is model.embed_weight and torch.equal(params["embed.weight"], stored["model.embed_tokens.weight"].float())
    # but a copy that differs from the embedding is an error, not a silent choice between the two
    # (the reference copies it over the shared storage, nanovllm/models/qwen3.py:202-203)
    stored["lm_head.weight"][3, 5] += 0.25
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError, match="lm_head.weight is not equal to model.embed_tokens.weight") as info:
        _load(folder)
    assert info.value.differing and not info.value.missing and not info.value.unexpected
    stored["lm_head.weight"] = torch.zeros(7, 64, dtype=torch.bfloat16)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError, match="wrong shapes"):
        _load(folder)
    folder = write_random_model(str(tmp_path / "c"), TINY_C, seed=2)
    model, params = _load(folder)
    assert "layers.0.mixer.qkv.bias" in params and "layers.0.mixer.q_norm.weight" not in params


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_A, seed=0)
    path = os.path.join(folder, "model.safetensors")
    stored = load_file(path)
    stored["model.norm.weight"] = stored["model.norm.weight"].float()
    stored["model.layers.0.self_attn.q_norm.weight"] = stored["model.layers.0.self_attn.q_norm.weight"].float()
    save_file(stored, path)
    _, params = _load(folder, torch.bfloat16)
    assert params["final_norm.weight"].dtype == torch.float32
    assert params["layers.0.mixer.q_norm.weight"].dtype == torch.float32
    assert params["layers.0.mixer.k_norm.weight"].dtype == torch.bfloat16
    assert params["embed.weight"].dtype == torch.bfloat16
    _, params = _load(folder, torch.float32)
    assert all(p.dtype == torch.float32 for p in params.values())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_B, seed=1)
    path = os.path.join(folder, "model.safetensors")
    stored = load_file(path)
    del stored["model.layers.1.self_attn.k_proj.weight"]               # one shard of a packed parameter
    del stored["lm_head.weight"]
    stored["model.layers.0.mlp.extra_proj.weight"] = torch.zeros(2, 2)
    stored["model.layers.7.input_layernorm.weight"] = torch.zeros(96)  # a layer the model does not have
    stored["model.layers.2.mlp.down_proj.weight"] = torch.zeros(96, 161, dtype=torch.bfloat16)
    stored["model.norm.weight"] = torch.zeros(95, dtype=torch.bfloat16)
    save_file(stored, path)
    with pytest.raises(WeightsError) as info:
        _load(folder)
    e = info.value
    assert e.missing == ["lm_head.weight", "model.layers.1.self_attn.k_proj.weight"] or \
        sorted(e.missing) == ["lm_head.weight", "model.layers.1.self_attn.k_proj.weight"]
    assert e.unexpected == ["model.layers.0.mlp.extra_proj.weight", "model.layers.7.input_layernorm.weight"]
    assert len(e.wrong_shape) == 2 and "down_proj" in " ".join(e.wrong_shape) and "[96, 161]" in " ".join(e.wrong_shape)
    msg = str(e)
    for piece in ("missing", "unexpected", "wrong shapes", "k_proj", "extra_proj", "needed [96, 160]"):
        assert piece in msg


def test_ignored_prefixes_are_skipped(tmp_path):
    """Tensors under a prefix that the architecture declares ignored (a vision tower beside the decoder, say) are
    neither loaded nor reported (nanovllm/utils/loader.py:27-31,85-93)."""
    import dataclasses
    from nanohybrid_vlm_amd.architectures.qwen3 import QWEN3
    from nanohybrid_vlm_amd.parts.model import DecoderModel
    from nanohybrid_vlm_amd.weights.loader import load_weights
    folder = write_random_model(str(tmp_path / "m"), TINY_A, seed=0)
    path = os.path.join(folder, "model.safetensors")
    stored = load_file(path)
    stored["visual.blocks.0.weight"] = torch.zeros(3, 3)
    stored["mtp.head.weight"] = torch.zeros(2)
    save_file(stored, path)
    with pytest.raises(WeightsError) as info:
        _load(folder)
    assert info.value.unexpected == ["mtp.head.weight", "visual.blocks.0.weight"]
    arch = dataclasses.replace(QWEN3, ignored_prefixes=("visual.", "mtp."))
    cfg = arch.parse_config(TINY_A)
    model = DecoderModel(arch.build_spec(cfg))
    params = load_weights(model, arch, cfg, folder, torch.float32, "cpu")
    assert "embed.weight" in params and not any("visual" in n or "mtp" in n for n in params)


def test_a_nested_text_config_is_read(tmp_path):
    """A multimodal checkpoint nests the decoder's keys under text_config (nanovllm/config.py:318-322)."""
    nested = {"architectures": ["Qwen3ForCausalLM"], "vision_config": {"hidden_size": 11},
              "text_config": {k: v for k, v in TINY_B.items() if k != "architectures"}}
    with open(tmp_path / "config.json", "w") as f:
        json.dump(nested, f)
    raw = read_config_json(str(tmp_path))
    cfg = Qwen3Config.from_dict(raw)
    assert cfg.hidden_size == 96 and cfg.architectures == ("Qwen3ForCausalLM",) and cfg.model_type == "qwen3"
    # keys at the top level win: a plain config.json that happens to carry a text_config is read as it is
    with open(tmp_path / "config.json", "w") as f:
        json.dump(dict(TINY_A, text_config={"hidden_size": 1}), f)
    assert Qwen3Config.from_dict(read_config_json(str(tmp_path))).hidden_size == 64


def test_random_weights_on_the_device_keep_float32_tensors():
    """Weights drawn in place of a checkpoint: what a checkpoint would keep in 32-bit (norm weights) is float32,
    the matrices have the run's element type."""
    from nanohybrid_vlm_amd.weights.random_init import build_random_model
    arch, cfg, model = build_random_model(TINY_B, seed=5, dtype="bfloat16", device="cpu")
    specs = model.all_param_specs()
    for name, t in model.parameters.items():
        assert t.dtype == (torch.float32 if specs[name].keeps_float32 else torch.bfloat16), name
    assert abs(model.parameters["final_norm.weight"].mean().item() - 1.0) < 0.1
    assert model.parameters["embed.weight"].float().std().item() == pytest.approx(0.02, rel=0.1)


def test_missing_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        read_config_json(str(tmp_path))
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_A, f)
    with pytest.raises(FileNotFoundError, match="safetensors"):
        _load(str(tmp_path))
