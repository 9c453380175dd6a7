"""Decode and prefill throughput of the Qwen3-8B shape with random bfloat16 weights
on one MI355X, through the engine's own entry point (scheduler, step function,
cache, kernels, sampler).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

A step is one decode step of the whole batch. Each request is a 2,048-token prompt
of random ids followed by generated tokens; W steps run untimed, then exactly K
steps are timed between two synchronisations. One JSON line is printed: ``value``
is decoded tokens a second; ``prefill`` is one 2,048-token prompt; ``roofline``
compares the decode step with the time to read what it must read (all weights it
uses once, and the cache of the live requests) at 8 TB/s; ``points`` holds decoding
at batch 1 and 64.
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0            # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense MFMA, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=192)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", default="8b")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (same layer sizes)")
    ap.add_argument("--prompt-tokens", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--block-size", type=int, default=256)
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 runs")
    ap.add_argument("--eager", action="store_true", help="no HIP graphs")
    ap.add_argument("--max-graph-batch", type=int, default=None, help="largest decode batch that replays a graph")
    return ap.parse_args()


def build_llm(args, max_seqs):
    from nanohybrid_vlm_amd import LLM
    from nanohybrid_vlm_amd.config.registry import named_shapes

    raw = dict(named_shapes()[args.shape])
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    pages_per_seq = -(-args.context // args.block_size)
    llm = LLM(raw, random_weights=0, dtype=args.dtype,
              kvcache_block_size=args.block_size, num_kvcache_blocks=max_seqs * pages_per_seq + 1,
              max_num_seqs=max_seqs, max_num_batched_tokens=max(2048, max_seqs), max_model_len=args.context,
              scheduler_policy="prefill_first",     # while prompts are fed nothing decodes, so all requests decode in step
              enforce_eager=args.eager, **({"max_graph_batch": args.max_graph_batch} if args.max_graph_batch else {}))
    return llm, llm.runner.cfg, full_layers


def model_bytes_and_flops(cfg, itemsize):
    """Bytes of the weights a decode step reads once, cache bytes per token, and flops per token of the layers' matrices."""
    H, I, D = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    Hq, Hkv, L, V = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.num_hidden_layers, cfg.vocab_size
    per_layer = (Hq + 2 * Hkv) * D * H + Hq * D * H + 2 * I * H + I * H + 2 * H + 2 * D
    weight_bytes = (L * per_layer + V * H + H) * itemsize          # layers + head + final norm (embedding rows: negligible)
    kv_bytes_per_token = 2 * L * Hkv * D * itemsize
    matrix_flops_per_token = 2 * L * ((Hq + 2 * Hkv) * D * H + Hq * D * H + 3 * I * H)
    return weight_bytes, kv_bytes_per_token, matrix_flops_per_token


def random_prompts(n, length, vocab, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]


def run_decode(llm, cfg, batch, prompt_tokens, steps, warmup, seed):
    """Prefills ``batch`` prompts, then times ``steps`` decode steps. Returns (seconds, mean context in the timed steps)."""
    import torch
    from nanohybrid_vlm_amd import SamplingParams

    sp = SamplingParams(temperature=0.0, max_tokens=warmup + steps + 1, ignore_eos=True)
    for p in random_prompts(batch, prompt_tokens, cfg.vocab_size, seed):
        llm.add_request(p, sp)
    while llm.scheduler.waiting:                      # all prompts in, nothing timed
        llm.step()
    for _ in range(warmup):
        llm.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        _, stats = llm.step()
        assert stats.num_decode_tokens == batch and stats.num_prefill_tokens == 0
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    while not llm.is_finished():
        llm.step()
    mean_context = prompt_tokens + warmup + (steps + 1) / 2.0
    return seconds, mean_context


def run_prefill(llm, cfg, prompt_tokens, reps=3):
    import torch
    from nanohybrid_vlm_amd import SamplingParams

    sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
    best = None
    warm = 3                                          # untimed runs: a shape of many rows is measured in the third step that meets it
    for i in range(reps + warm):
        llm.add_request(random_prompts(1, prompt_tokens, cfg.vocab_size, 900 + i)[0], sp)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while not llm.is_finished():
            llm.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i >= warm:
            best = dt if best is None else min(best, dt)
    return best


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    import torch

    itemsize = 2 if args.dtype == "bfloat16" else 4
    dname = "bf16" if args.dtype == "bfloat16" else "fp32"
    max_seqs = max(args.batch, 1 if args.no_points else 64)
    llm, cfg, full_layers = build_llm(args, max_seqs)
    weight_bytes, kv_per_token, matrix_flops = model_bytes_and_flops(cfg, itemsize)

    # prefill of one prompt
    T = args.prompt_tokens
    pre_s = run_prefill(llm, cfg, T)
    attn_flops = 2 * 2 * cfg.num_hidden_layers * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2)
    pre_flops = matrix_flops * T + attn_flops + 2 * cfg.vocab_size * cfg.hidden_size
    prefill = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS[dname], 4)}

    def decode_point(batch, steps, warmup, seed):
        s, ctx = run_decode(llm, cfg, batch, T, steps, warmup, seed)
        ms = s / steps * 1e3
        step_bytes = weight_bytes + batch * ctx * kv_per_token
        return batch * steps / s, ms, step_bytes / (ms * 1e-3) / 1e9

    value, ms_per_step, achieved = decode_point(args.batch, args.steps, args.warmup, 1)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            v, _, _ = decode_point(b, min(args.steps, 128), min(args.warmup, 8), 10 + b)
            points[f"decode_b{b}"] = round(v, 1)

    line = {
        "metric": f"decode tok/s, Qwen3-{args.shape} shape, batch {args.batch}, {T}-token prompts",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic: random token ids, random weights N(0, 0.02^2), norms 1 + N(0, 0.1^2)",
        "config": {
            "model": f"Qwen3-{args.shape} shape", "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers,
            "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps, "tied_head": cfg.tie_word_embeddings,
            "global_batch": args.batch, "prompt_len": T, "seq_len": args.context, "kv_block": args.block_size,
            "parallelism": "single GPU", "graphs": not args.eager,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
