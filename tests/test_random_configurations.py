"""Configurations drawn at random (seeded): every size and option of the architecture at values that the fixed tiny
configurations do not take, replayed in portions and mixed on few pages of a size drawn with them, against the plain
implementation."""
import random

import pytest
import torch

import plain_qwen3 as plain
import replay_cases as rc
from helpers import max_abs_diff, tolerance_for
from test_replay import _check, _poisoned


def random_configuration(seed: int):
    rnd = random.Random(seed)
    kv_heads = rnd.choice([1, 2, 3])
    group = rnd.choice([1, 2, 3, 4, 5, 7])
    bias = rnd.random() < 0.3
    config = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
        "num_hidden_layers": rnd.choice([1, 2, 3]), "hidden_size": rnd.choice([40, 72, 104, 136, 200]),
        "num_attention_heads": kv_heads * group, "num_key_value_heads": kv_heads,
        "head_dim": rnd.choice([16, 32, 48, 64, 80, 96, 112, 128]), "intermediate_size": rnd.choice([56, 88, 152, 264]),
        "vocab_size": rnd.choice([97, 263, 1031]), "rope_theta": rnd.choice([10000.0, 500000.0, 1000000.0]),
        "rms_norm_eps": rnd.choice([1e-6, 1e-5, 3e-5]), "tie_word_embeddings": rnd.random() < 0.5,
        "max_position_embeddings": 512, "attention_bias": bias, "hidden_act": "silu",
    }
    page = rnd.choice([4, 8, 16, 24, 64])
    lengths = [rnd.randint(2, 90) for _ in range(5)]
    return config, page, lengths


def _replay(folder, dtype, device, page, lengths, graphs):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 700 + i) for i, n in enumerate(lengths)}
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}
    tol = tolerance_for(dtype, want)
    results = {}
    for mode, steps in [("portions", rc.portions(requests)), ("mixed", rc.mixed(requests)), ("tail", rc.tail_decoded(requests, 6))]:
        pages = rc.peak_tokens(steps, page) // page
        runner = _poisoned(ModelRunner(folder, dtype=dtype, device=device, page_size=page, num_pages=pages, num_state_slots=4,
                                       use_graphs=graphs, max_model_len=128, poison_freed_pages=True))
        results[mode] = rc.run_in_process(runner, steps)
        _check(results[mode], want, tol, f"{dtype} {mode}")
        assert not runner.cache.requests and runner.cache.num_free_pages(0) == pages
    return results


@pytest.mark.parametrize("seed", range(6))
def test_random_configuration_on_emulated_kernels(seed, emulated_kernels, tmp_path):
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    config, page, lengths = random_configuration(seed)
    write_random_model(str(tmp_path), config, seed)
    _replay(str(tmp_path), "float32", "cpu", page, lengths, graphs=False)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(12))
def test_random_configuration_on_gpu(seed, tmp_path):
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    config, page, lengths = random_configuration(seed)
    print(f"seed {seed}: {config}, page {page}, lengths {lengths}", flush=True)
    write_random_model(str(tmp_path), config, seed)
    exact = _replay(str(tmp_path), "float32", "cuda:0", page, lengths, graphs=seed % 2 == 0)
    for mode in ("mixed", "tail"):
        for rid in exact["portions"]:
            assert torch.equal(exact[mode][rid], exact["portions"][rid]), f"float32, {mode} against portions: request {rid}"
    _replay(str(tmp_path), "bfloat16", "cuda:0", page, lengths, graphs=seed % 2 == 1)
