"""Decode and prefill throughput of the Qwen3 shapes with random bfloat16 weights on one MI355X, through the
engine's own entry point (scheduler, step function, cache, kernels, sampler).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--shape 8b|14b|32b] [--layers L]

Default (``--shape 8b``): a step is one decode step of the whole batch. Each request is a 2,048-token prompt of
random ids followed by generated tokens; W steps run untimed, then exactly K steps are timed between two
synchronisations. One JSON line is printed: ``value`` is decoded tokens a second; ``prefill`` is one 2,048-token
prompt; ``roofline`` compares the decode step with the time to read what it must read (all weights it uses once, and
the cache of the live requests) at 8 TB/s, and ``measured`` gives the same fractions against what this GPU was
measured to give (a kernel that only reads; the vendor library's large bfloat16 product); ``points`` holds
decoding at batch 1 and 64; ``step_ms`` the timed steps' median and 95th percentile.

``--shape 14b``: 32 requests with prompt lengths uniform in [128, 4096] and 128 generated tokens each, all queued at
once, prompts fed in portions of 2,048 tokens beside the decoding requests (continuous batching).
``--shape 32b``: 16 requests of 8,192 prompt tokens and 256 generated tokens, the cache sized from free memory.
For these two ``value`` is generated tokens a second over the whole run, prompts included; a step is an engine step.

``--workload projections`` is a diagnosis, not the benchmark: a layer's matrix products alone, cold, beside a kernel
that only reads the same bytes (see ``bench_projections``).
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0            # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense MFMA, published


def _int_or_list(text):
    return int(text) if text.isdigit() else text      # (a list of row counts, "1,8,64", for --workload projections)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)     # with the 16 warm-up steps: 256 generated tokens a request
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=_int_or_list, default=None, help="requests decoding side by side (8b: 8, 14b: 32, 32b: 16)")
    ap.add_argument("--shape", default="8b")
    ap.add_argument("--workload", default="auto", choices=("auto", "points", "serving", "projections"),
                    help="points: decode at a fixed batch after equal prompts (8b by default); serving: the 14b / 32b workloads; "
                         "projections: a layer's matrix products alone against a kernel that only reads the same bytes")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (same layer sizes)")
    ap.add_argument("--prompt-tokens", type=int, default=None, help="8b: 2048; 32b: 8192; 14b: the longest prompt, 4096")
    ap.add_argument("--output-tokens", type=int, default=None, help="14b: 128; 32b: 256")
    ap.add_argument("--context", type=int, default=None, help="max_model_len (8b: 4096)")
    ap.add_argument("--token-budget", type=int, default=2048, help="tokens in one step (max_num_batched_tokens): a prompt longer than this is fed in portions")
    ap.add_argument("--block-size", type=int, default=256)
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 runs")
    ap.add_argument("--no-measured-peaks", action="store_true", help="skip the measurement of what this GPU gives")
    ap.add_argument("--eager", action="store_true", help="no HIP graphs")
    ap.add_argument("--max-graph-batch", type=int, default=None, help="largest decode batch that replays a graph")
    ap.add_argument("--residual-dtype", default="float32", choices=("float32", "model"),
                    help="the residual stream between layers: float32, or rounded to the element type as the reference does")
    ap.add_argument("--no-fuse-norms", action="store_true",
                    help="products of few rows leave the residual addition and the norm to kernels of their own")
    ap.add_argument("--gemm-choices", default=None, help="JSON file of matrix-product choices to follow (and to write if absent)")
    return ap.parse_args()


def percentile(values, q):
    values = sorted(values)
    k = (len(values) - 1) * q
    lo, hi = int(k), min(int(k) + 1, len(values) - 1)
    return values[lo] + (values[hi] - values[lo]) * (k - lo)


def build_llm(args, max_seqs, **options):
    from nanohybrid_vlm_amd import LLM
    from nanohybrid_vlm_amd.config.registry import named_shapes

    raw = dict(named_shapes()[args.shape])
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    llm = LLM(raw, random_weights=0, dtype=args.dtype, kvcache_block_size=args.block_size, max_num_seqs=max_seqs,
              enforce_eager=args.eager, gemm_choices=args.gemm_choices, residual_dtype=args.residual_dtype,
              fuse_norms=not args.no_fuse_norms,
              **({"max_graph_batch": args.max_graph_batch} if args.max_graph_batch else {}), **options)
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
    """Prefills ``batch`` prompts, then times ``steps`` decode steps. Returns (seconds, mean context in the timed
    steps, the steps' host times in ms)."""
    import torch
    from nanohybrid_vlm_amd import SamplingParams

    # The engine issues a decode step ahead of its tokens: when the warm-up ends, the first timed step's GPU work is
    # under way already (and done at the synchronisation). So that the timed window still holds exactly ``steps``
    # steps of GPU work, the requests live one token longer than the timed steps: the last timed step issues its
    # successor ahead as every other does, and the closing synchronisation waits for it. Without steps issued
    # ahead the window holds the timed steps' own work. Either way: ``steps`` steps between the two waits.
    sp = SamplingParams(temperature=0.0, max_tokens=warmup + steps + 2, ignore_eos=True)
    for p in random_prompts(batch, prompt_tokens, cfg.vocab_size, seed):
        llm.add_request(p, sp)
    while llm.scheduler.waiting:                      # all prompts in, nothing timed
        llm.step()
    for _ in range(warmup):
        llm.step()
    torch.cuda.synchronize()
    ahead = llm._ahead is not None                    # the timed GPU steps are then the ones after the host's
    step_ms = []
    t0 = time.perf_counter()
    last = t0
    for _ in range(steps):
        _, stats = llm.step()
        assert stats.num_decode_tokens == batch and stats.num_prefill_tokens == 0
        now = time.perf_counter()
        step_ms.append((now - last) * 1e3)
        last = now
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    while not llm.is_finished():
        llm.step()
    mean_context = prompt_tokens + warmup + (steps + 1) / 2.0 + (1 if ahead else 0)
    return seconds, mean_context, step_ms


def run_prefill(llm, cfg, prompt_tokens, reps=5):
    import torch
    from nanohybrid_vlm_amd import SamplingParams

    sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
    times = []
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
            times.append(dt)
    return percentile(times, 0.5)                     # the median of the timed runs


def config_of(args, cfg, full_layers, **more):
    """Every size, flat (at most 20 keys)."""
    out = {
        "model": f"Qwen3-{args.shape} shape", "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers,
        "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
        "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps, "tied_head": cfg.tie_word_embeddings,
        "kv_block": args.block_size, "parallelism": "single GPU", "graphs": not args.eager,
    }
    out.update(more)
    assert len(out) <= 20
    return out


def measured_peaks(args):
    if args.no_measured_peaks:
        return None
    from nanohybrid_vlm_amd.native import ops
    peaks = ops.measured_peaks()
    return {"hbm_read_GBs": round(peaks["hbm_read_GBs"], 1), "gemm_bf16_TFLOPs": round(peaks["gemm_bf16_TFLOPs"], 1)}


def bench_decode_points(args):
    """The headline measurement: decode at a fixed batch after equal prompts, a 2,048-token prefill, batch 1 and 64."""
    import torch

    batch = args.batch or 8
    T = args.prompt_tokens or 2048
    context = args.context or 4096
    itemsize = 2 if args.dtype == "bfloat16" else 4
    dname = "bf16" if args.dtype == "bfloat16" else "fp32"
    max_seqs = max(batch, 1 if args.no_points else 64)
    pages_per_seq = -(-context // args.block_size)
    llm, cfg, full_layers = build_llm(args, max_seqs, num_kvcache_blocks=max_seqs * pages_per_seq + 1,
                                      max_num_batched_tokens=max(args.token_budget, max_seqs), max_model_len=context,
                                      scheduler_policy="prefill_first")   # while prompts are fed nothing decodes, so all requests decode in step
    weight_bytes, kv_per_token, matrix_flops = model_bytes_and_flops(cfg, itemsize)
    peaks = measured_peaks(args)

    pre_s = run_prefill(llm, cfg, T)
    attn_flops = 2 * 2 * cfg.num_hidden_layers * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2)
    pre_flops = matrix_flops * T + attn_flops + 2 * cfg.vocab_size * cfg.hidden_size
    prefill = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS[dname], 4)}

    def decode_point(b, steps, warmup, seed):
        s, ctx, step_ms = run_decode(llm, cfg, b, T, steps, warmup, seed)
        ms = s / steps * 1e3
        step_bytes = weight_bytes + b * ctx * kv_per_token
        return b * steps / s, ms, step_bytes / (ms * 1e-3) / 1e9, step_ms

    value, ms_per_step, achieved, step_ms = decode_point(batch, args.steps, args.warmup, 1)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            if b == batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            v, _, _, _ = decode_point(b, min(args.steps, 128), min(args.warmup, 8), 10 + b)
            points[f"decode_b{b}"] = round(v, 1)

    line = {
        "metric": f"decode tok/s, Qwen3-{args.shape} shape, batch {batch}, {T}-token prompts",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic: random token ids, random weights N(0, 0.02^2), norms 1 + N(0, 0.1^2)",
        "config": config_of(args, cfg, full_layers, global_batch=batch, prompt_len=T, seq_len=context),
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
        "step_ms": {"p50": round(percentile(step_ms, 0.5), 4), "p95": round(percentile(step_ms, 0.95), 4)},
    }
    if peaks:
        line["measured"] = dict(peaks, roofline_frac=round(achieved / peaks["hbm_read_GBs"], 4),
                                prefill_frac=round(pre_flops / pre_s / (peaks["gemm_bf16_TFLOPs"] * 1e12), 4))
    line["gemm_choices"] = llm.gemm_choices()
    if args.gemm_choices:
        import os
        if not os.path.isfile(args.gemm_choices):
            llm.save_gemm_choices(args.gemm_choices)
    print(json.dumps(line), flush=True)
    return 0


def bench_workload(args):
    """The serving workloads: every request queued at once, prompts in portions beside decoding requests."""
    import torch
    from nanohybrid_vlm_amd import SamplingParams

    itemsize = 2 if args.dtype == "bfloat16" else 4
    dname = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.shape != "32b":
        batch, n_out = args.batch or 32, args.output_tokens or 128
        longest = args.prompt_tokens or 4096
        g = torch.Generator().manual_seed(14)
        lengths = torch.randint(128, longest + 1, (batch,), generator=g).tolist()
        context = args.context or (longest + n_out)
        pages = sum(-(-(n + n_out) // args.block_size) for n in lengths) + 1
        cache = {"num_kvcache_blocks": pages}
        workload = f"{batch} requests, prompts uniform in [128, {longest}], {n_out} new tokens each, portions of {args.token_budget}"
    else:
        batch, n_out = args.batch or 16, args.output_tokens or 256
        longest = args.prompt_tokens or 8192
        lengths = [longest] * batch
        context = args.context or (longest + n_out)
        cache = {"num_kvcache_blocks": -1}            # the cache takes what is left of the device's memory
        workload = f"{batch} requests of {longest} prompt tokens, {n_out} new tokens each, cache sized from free memory"
    llm, cfg, full_layers = build_llm(args, batch, max_num_batched_tokens=args.token_budget, max_model_len=context, **cache)
    weight_bytes, kv_per_token, matrix_flops = model_bytes_and_flops(cfg, itemsize)
    peaks = measured_peaks(args)
    sp = SamplingParams(temperature=0.0, max_tokens=n_out, ignore_eos=True)

    def once(seed):
        prompts = [random_prompts(1, n, cfg.vocab_size, seed + i)[0] for i, n in enumerate(lengths)]
        for p in prompts:
            llm.add_request(p, sp)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = []
        while not llm.is_finished():
            _, st = llm.step()
            steps.append(st)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, steps

    once(1000)                                        # untimed: graphs are recorded, products measured
    wall, steps = once(2000)
    decode_only = [s for s in steps if s.num_prefill_tokens == 0]
    with_prompts = [s for s in steps if s.num_prefill_tokens > 0]
    generated = batch * n_out
    decode_s = sum(s.seconds for s in decode_only)
    decode_tokens = sum(s.num_decode_tokens for s in decode_only)
    live_tokens = sum(lengths) + generated / 2.0      # the cache that a decode-only step reads, about
    decode_ms = decode_s / max(len(decode_only), 1) * 1e3
    achieved = (weight_bytes + live_tokens * kv_per_token) / (decode_ms * 1e-3) / 1e9 if decode_only else 0.0
    prompt_s = sum(s.seconds for s in with_prompts)
    prompt_tokens = sum(s.num_prefill_tokens + s.num_decode_tokens for s in with_prompts)
    stats = llm.get_memory_stats()
    line = {
        "metric": f"generated tok/s, Qwen3-{args.shape} shape, {workload}",
        "value": round(generated / wall, 1), "unit": "tok/s", "n_gpus": 1, "steps": len(steps), "warmup": len(steps),
        "ms_per_step": round(wall / len(steps) * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic: random token ids, random weights N(0, 0.02^2), norms 1 + N(0, 0.1^2)",
        "config": config_of(args, cfg, full_layers, global_batch=batch, prompt_len=longest, seq_len=context,
                            token_budget=args.token_budget, cache_pages=stats["groups"][0]["pages"]),
        "prefill": {"value": round(prompt_tokens / prompt_s, 1) if prompt_s else None, "tokens": sum(lengths),
                    "ms": round(prompt_s * 1e3, 3), "frac": round(matrix_flops * prompt_tokens / prompt_s / PEAK_FLOPS[dname], 4) if prompt_s else None},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": {"decode_only_tok_s": round(decode_tokens / decode_s, 1) if decode_s else None,
                   "decode_only_ms_per_step": round(decode_ms, 4), "wall_s": round(wall, 3),
                   "preemptions": llm.scheduler.num_preemptions},
        "step_ms": {"p50": round(percentile([s.seconds * 1e3 for s in steps], 0.5), 4),
                    "p95": round(percentile([s.seconds * 1e3 for s in steps], 0.95), 4)},
    }
    if peaks:
        line["measured"] = dict(peaks, roofline_frac=round(achieved / peaks["hbm_read_GBs"], 4))
    line["gemm_choices"] = llm.gemm_choices()
    print(json.dumps(line), flush=True)
    return 0


def bench_projections(args):
    """How near a decode step's matrix products are to what the memory gives them: for each of a layer's four weight
    matrices and the head, a chain of products with different weights of that size (1 GB or more in all, so that no
    weight is found in a cache), recorded into a graph as in a decode step, done as the engine does them (the own
    kernel or the library algorithm that the engine's measurement picks) and by the own kernels alone, beside a chain
    of a kernel that only reads the same bytes. Rows: 1, 8 and 64 (``--batch`` for another list, e.g. 1,16)."""
    import ctypes
    import torch
    from nanohybrid_vlm_amd.config.registry import named_shapes, resolve_architecture
    from nanohybrid_vlm_amd.native import ops

    raw = dict(named_shapes()[args.shape])
    cfg = resolve_architecture(raw).parse_config(raw)
    H, I, D = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    shapes = [("qkv", (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * D, H, False), ("o", H, cfg.num_attention_heads * D, False),
              ("gate_up", 2 * I, H, True), ("down", H, I, False), ("head", cfg.vocab_size, H, False)]
    rows = [int(m) for m in str(args.batch).split(",")] if args.batch else [1, 8, 64]
    b = ops.backend()
    stream = torch.cuda.Stream()
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    table = {}

    def chain_us(run, count):
        """Microseconds a call, of ``count`` calls recorded into one graph; the shortest of five replays."""
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            run()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                run()
            graph.replay()
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(5):
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                graph.replay()
                end.record()
                end.synchronize()
                best = min(best, start.elapsed_time(end))
        return best * 1e3 / count

    print(f"{'product':8s} {'MB':>7s} {'rows':>4s} {'engine us':>10s} {'TB/s':>5s} {'own us':>8s} {'TB/s':>5s} {'read us':>8s} {'TB/s':>5s}  engine/read",
          flush=True)
    for name, N, K, gated in shapes:
        nbytes = N * K * 2
        count = min(32, max(4, -(-(1 << 30) // nbytes)))
        weights = [torch.randn(N, K, device="cuda", dtype=torch.bfloat16) * 0.02 for _ in range(count)]

        def read():
            for w in weights:
                b._call("nhv_measure_read", ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(sink.data_ptr()),
                        ctypes.c_size_t(nbytes // 1024 * 1024), ops._stream())
        read_us = chain_us(read, count)
        for M in rows:
            x = torch.randn(M, K, device="cuda", dtype=torch.bfloat16)
            float_result = name == "head"

            def products():
                for w in weights:
                    if gated:
                        ops.gated_linear(x, w)
                    else:
                        ops.linear(x, w, out_dtype=torch.float32 if float_result else None)
            b.measure_linears, b.own_kernels_only = True, False
            products()                                 # (the first call of a shape measures it; the answer is kept)
            b.measure_linears = False
            b.end_measurements()
            engine_us = chain_us(products, count)
            b.own_kernels_only = True
            own_us = chain_us(products, count)
            b.own_kernels_only = False
            table[f"{name}_m{M}"] = {"engine_us": round(engine_us, 2), "own_us": round(own_us, 2), "read_us": round(read_us, 2)}
            print(f"{name:8s} {nbytes / 1e6:7.1f} {M:4d} {engine_us:10.1f} {nbytes / engine_us / 1e6:5.2f} {own_us:8.1f} "
                  f"{nbytes / own_us / 1e6:5.2f} {read_us:8.1f} {nbytes / read_us / 1e6:5.2f}  {engine_us / read_us:.2f}", flush=True)
        del weights
    for M in rows:
        layer = [table[f"{n}_m{M}"] for n in ("qkv", "o", "gate_up", "down")]
        print(f"a layer's four products at {M} rows: engine {sum(t['engine_us'] for t in layer):.1f} us, own kernels "
              f"{sum(t['own_us'] for t in layer):.1f} us, reading alone {sum(t['read_us'] for t in layer):.1f} us", flush=True)
    print(json.dumps({"metric": f"a layer's matrix products against reads of the same bytes, Qwen3-{args.shape} shape",
                      "unit": "us", "dtype": "bf16", "table": table, "gemm_choices": b.choices_table()}), flush=True)
    return 0


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    serving = args.workload == "serving" or (args.workload == "auto" and args.shape in ("14b", "32b"))
    if args.workload == "projections":
        return bench_projections(args)
    if isinstance(args.batch, str):
        print(f"bench.py: --batch {args.batch}: a list of row counts goes with --workload projections only", flush=True)
        return 2
    if serving:
        return bench_workload(args)
    return bench_decode_points(args)


if __name__ == "__main__":
    sys.exit(main())
