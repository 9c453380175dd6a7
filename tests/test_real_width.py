"""A whole model with the layer sizes of a real member of the family (Qwen3-8B: width 4096, feed-forward 12288, 32
query and 8 key/value heads of 128, vocabulary 151936, pages of 256) and two layers, against the plain
implementation: the kernels that only those widths reach (the few-rows products that keep x in LDS, take it in
pieces or pass over it twice, the library's products, the greedy sampler's pieces, recorded steps at real widths)
run as a model here, not only one by one.

The plain implementation is the same plain torch code as everywhere, evaluated in float32 on the GPU (on the CPU a
vocabulary of 151936 would take minutes). The model folder is written by this file itself, from the tensor names
of a Qwen3 checkpoint, with weights drawn on the GPU.
"""
import json
import os

import pytest
import torch

import plain_qwen3 as plain
import replay_cases as rc
from helpers import first_difference, max_abs_diff, tolerance_for

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2, "hidden_size": 4096,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
    "max_position_embeddings": 4096, "attention_bias": False, "hidden_act": "silu", "eos_token_id": 151645,
    "torch_dtype": "bfloat16",
}


@pytest.fixture(scope="module")
def real_width_folder(tmp_path_factory):
    """config.json and model.safetensors (3.3 GB, bfloat16): matrices N(0, 0.02^2), norm weights 1 + N(0, 0.1^2)."""
    from safetensors.torch import save_file
    c = CONFIG
    H, I, D = c["hidden_size"], c["intermediate_size"], c["head_dim"]
    q, kv = c["num_attention_heads"] * D, c["num_key_value_heads"] * D
    shapes = {"model.embed_tokens.weight": (c["vocab_size"], H), "lm_head.weight": (c["vocab_size"], H),
              "model.norm.weight": (H,)}
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes.update({p + "input_layernorm.weight": (H,), p + "post_attention_layernorm.weight": (H,),
                       p + "self_attn.q_proj.weight": (q, H), p + "self_attn.k_proj.weight": (kv, H),
                       p + "self_attn.v_proj.weight": (kv, H), p + "self_attn.o_proj.weight": (H, q),
                       p + "self_attn.q_norm.weight": (D,), p + "self_attn.k_norm.weight": (D,),
                       p + "mlp.gate_proj.weight": (I, H), p + "mlp.up_proj.weight": (I, H),
                       p + "mlp.down_proj.weight": (H, I)})
    gen = torch.Generator(device="cuda").manual_seed(11)
    tensors = {}
    for name, shape in shapes.items():
        t = torch.randn(shape, generator=gen, device="cuda", dtype=torch.float32)
        t = 1.0 + 0.1 * t if "norm" in name else 0.02 * t
        tensors[name] = t.to(torch.bfloat16).cpu()
    folder = str(tmp_path_factory.mktemp("real_width"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(c, f)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder


@pytest.fixture(scope="module")
def plain_on_gpu(real_width_folder):
    """The requests and the plain implementation's logits for them (float32, on the GPU, moved to the CPU)."""
    cfg, w = plain.read_model_folder(real_width_folder)
    w = {name: t.cuda() for name, t in w.items()}
    lengths = [300, 65, 513, 17, 129, 8]
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 500 + i) for i, n in enumerate(lengths)}
    with torch.no_grad():
        want = {rid: plain.logits(cfg, w, toks).cpu() for rid, toks in requests.items()}
    del w
    torch.cuda.empty_cache()
    return requests, want


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_model_at_real_widths(real_width_folder, plain_on_gpu, dtype, graphs):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    requests, want = plain_on_gpu
    tol = tolerance_for(dtype, want)
    results = {}
    for mode, steps in [("whole", rc.whole(requests)), ("tail", rc.tail_decoded(requests, tail=32)),
                        ("mixed", rc.mixed(requests, sizes=(100, 7, 64, 2, 129, 33)))]:
        pages = rc.peak_tokens(steps, 256) // 256
        runner = ModelRunner(real_width_folder, dtype=dtype, page_size=256, num_pages=pages, num_state_slots=4,
                             use_graphs=graphs, max_model_len=768, poison_freed_pages=True)
        for kv in runner.kv_tensors:
            kv.fill_(float("nan"))                   # a read beyond a request's tokens would show
        results[mode] = rc.run_in_process(runner, steps)
        for rid in requests:
            d = max_abs_diff(results[mode][rid], want[rid])
            assert d <= tol, (f"{dtype} {mode}: request {rid}: max diff {d:.3e} > {tol:.1e}; "
                              + first_difference(results[mode][rid], want[rid], tol))
        assert runner.cache.num_free_pages(0) == pages
        if graphs and mode != "whole":
            stats = runner.get_memory_stats()
            assert stats["graphs_recorded"] and not stats["graphs_refused"], stats
        del runner
        torch.cuda.empty_cache()
    if dtype == "float32":
        for mode in ("tail", "mixed"):
            for rid in requests:
                assert torch.equal(results[mode][rid], results["whole"][rid]), f"float32 {mode} against whole: {rid}"


def test_generation_at_real_widths(real_width_folder):
    """Greedy and seeded sampling through the entry point over the real vocabulary (the sampler's pieces, the head's
    kernels of 1 to 5 rows, recorded steps and steps issued ahead): every greedy token is one the plain implementation
    rates best or nearly so."""
    from nanohybrid_vlm_amd import LLM, SamplingParams
    cfg, w = plain.read_model_folder(real_width_folder)
    w = {name: t.cuda() for name, t in w.items()}
    prompts = [rc.random_tokens(cfg["vocab_size"], n, 600 + n) for n in (40, 3, 260, 17, 90)]
    llm = LLM(real_width_folder, dtype="bfloat16", kvcache_block_size=256, num_kvcache_blocks=12, max_num_batched_tokens=128,
              max_model_len=512)
    params = [SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)] * 4 + [SamplingParams(temperature=0.8, max_tokens=8, seed=3)]
    outs = llm.generate(prompts, params, use_tqdm=False)
    assert llm.num_steps_ahead > 0
    stats = llm.get_memory_stats()
    assert stats["mixed_graphs_recorded"] and not stats["mixed_graphs_refused"], stats      # the prompts' portions ran as graphs
    with torch.no_grad():
        for p, o in list(zip(prompts, outs))[:4]:
            ids = list(p)
            for t in o["token_ids"]:
                row = plain.logits(cfg, w, ids)[-1]
                assert row[t] >= row.max() - 0.1 * row.std(), "a token far from the best was chosen"
                ids.append(t)
    again = LLM(real_width_folder, dtype="bfloat16", kvcache_block_size=256, num_kvcache_blocks=12, max_num_batched_tokens=128,
                max_model_len=512, run_ahead=False).generate(prompts, params, use_tqdm=False)
    assert [o["token_ids"] for o in again] == [o["token_ids"] for o in outs]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_steps_as_graphs_at_real_widths(real_width_folder, plain_on_gpu, dtype):
    """Portions beside decoded tokens, one wanted place a request: the steps of up to 256 tokens replay graphs whose
    buckets are filled by a request of their own; the logits are the plain implementation's, and in float32 the
    eager run's bit for bit."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    requests, full = plain_on_gpu
    steps = rc.mixed(requests, sizes=(100, 7, 64, 2, 129, 33))
    steps = [dict(st, entries=[dict(e, want=[len(e["tokens"]) - 1]) for e in st["entries"]]) for st in steps]
    want, fed = {}, {rid: 0 for rid in requests}
    for st in steps:
        for e in st["entries"]:
            fed[e["id"]] += len(e["tokens"])
            want.setdefault(e["id"], []).append(full[e["id"]][fed[e["id"]] - 1])
    want = {rid: torch.stack(rows) for rid, rows in want.items()}
    tol = tolerance_for(dtype, full)
    results = {}
    for graphs in (True, False):
        pages = rc.peak_tokens(steps, 256) // 256
        runner = ModelRunner(real_width_folder, dtype=dtype, page_size=256, num_pages=pages, num_state_slots=4,
                             use_graphs=graphs, max_model_len=768, poison_freed_pages=True)
        for kv in runner.kv_tensors:
            kv.fill_(float("nan"))
        results[graphs] = rc.run_in_process(runner, steps)
        for rid in requests:
            d = max_abs_diff(results[graphs][rid], want[rid])
            assert d <= tol, f"{dtype}, graphs {graphs}: request {rid}: max diff {d:.3e} > {tol:.1e}"
        stats = runner.get_memory_stats()
        assert bool(stats["mixed_graphs_recorded"]) == graphs and not stats["mixed_graphs_refused"], stats
        del runner
        torch.cuda.empty_cache()
    if dtype == "float32":
        for rid in requests:
            assert torch.equal(results[True][rid], results[False][rid]), rid
