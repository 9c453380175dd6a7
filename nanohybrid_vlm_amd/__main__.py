"""Command line: ``python -m nanohybrid_vlm_amd <command> ...``.

The reference ships no command of its own; its command lines are argparse scripts
that build an ``LLM``, run cases and write a JSON file
(tests/5090-test-TP2/run_generation.py:37-59, tests/normal_test/benchmark_hybrid.py:16-65).
Option names and meanings are taken from there where they exist: ``--model``,
``--output``, ``--label``, ``--mode {eager,graph}``, ``--cases P:B``,
``--output-tokens``, ``--repeats``, ``--warmup-output-tokens``, ``--token-budget``,
``--gpu-memory-utilization``, ``--prompt-tokens``, ``--concurrency``.

    generate      token ids in, token ids out (text if the folder has a tokenizer.json)
    bench         cases of P prompt tokens x B requests; tok/s, step times, TTFT/TPOT/E2E as JSON
    random-model  writes config.json + model.safetensors with seeded random weights
    replay        the trace-replay program (same as bin/trace_run)
"""
from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path


def _case(text: str) -> tuple[int, int]:
    try:
        p, b = text.split(":")
        p, b = int(p), int(b)
    except ValueError as e:
        raise argparse.ArgumentTypeError("a case is PROMPT_TOKENS:BATCH, e.g. 2048:8") from e
    if p <= 0 or b <= 0:
        raise argparse.ArgumentTypeError("Case values must be positive")
    return p, b


def _engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--random-weights", type=int, metavar="SEED",
                    help="instead of --model: random weights of --shape or --config, drawn on the device")
    ap.add_argument("--shape", default="tinyA",
                    help="with --random-weights: a named configuration of a registered architecture "
                         "(an unknown name lists those there are)")
    ap.add_argument("--config", help="with --random-weights: a config.json to take the sizes from, instead of --shape")
    ap.add_argument("--layers", type=int, help="with --random-weights: override num_hidden_layers")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32", "bf16", "fp32"))
    ap.add_argument("--mode", choices=("eager", "graph"), default="graph", help="graph: decode steps replay HIP graphs")
    ap.add_argument("--token-budget", type=int, default=2048, help="tokens per step (max_num_batched_tokens)")
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    ap.add_argument("--block-size", type=int, default=256, help="tokens per page of the cache")
    ap.add_argument("--num-blocks", type=int, default=-1, help="pages of the cache (-1: from free memory)")
    ap.add_argument("--max-num-seqs", type=int, default=512)
    ap.add_argument("--max-graph-batch", type=int, default=256, help="decode steps of up to this many requests replay a graph")
    ap.add_argument("--max-graph-tokens", type=int, default=256,
                    help="other steps (prompt portions, alone or beside decoded tokens) of up to this many tokens replay a graph; 0: none")
    ap.add_argument("--warm-up", action="store_true",
                    help="measure the matrix products and record the graphs of every step size when the engine starts")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="every step is issued only when the tokens of the step before are known to the host")
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--scheduler-policy", choices=("decode_first", "prefill_first"), default="decode_first")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--enable-prefix-cache", action="store_true",
                    help="requests with a common start share the full pages that hold it")
    ap.add_argument("--plugin", action="append", metavar="MODULE",
                    help="a module to import first: it may register architectures and parts of its own; repeatable")
    ap.add_argument("--gemm-choices", metavar="FILE",
                    help="how each shape of matrix product is done: read from FILE if it exists (nothing is timed then), "
                         "written to it at the end otherwise")
    ap.add_argument("--residual-dtype", choices=("float32", "model"), default="float32",
                    help="the residual stream between layers: kept in float32, or rounded to the model's element type "
                         "after every addition as the reference does")
    ap.add_argument("--no-measure-gemms", action="store_true",
                    help="time no matrix product: shapes follow --gemm-choices, else the fixed rule")


def _import_plugins(names) -> None:
    """Modules that register architectures or parts of their own when imported."""
    from .config.registry import import_plugins
    import_plugins(names)


def _named_config(args) -> dict:
    """config.json contents for --random-weights and random-model: a file, or a registered architecture's named shape."""
    from .config.registry import named_shapes
    if getattr(args, "config", None):
        raw = json.loads(Path(args.config).read_text())
    else:
        shapes = named_shapes()
        if args.shape not in shapes:
            raise SystemExit(f"unknown --shape '{args.shape}'; known: {sorted(shapes)}")
        raw = dict(shapes[args.shape])
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    return raw


def _make_llm(args):
    from . import LLM
    _import_plugins(args.plugin)
    if (args.model is None) == (args.random_weights is None):
        raise SystemExit("give either --model DIR or --random-weights SEED")
    model, random_weights = args.model, None
    if args.random_weights is not None:
        model, random_weights = _named_config(args), args.random_weights
        args.model = f"random {args.config or args.shape}"
    return LLM(model, random_weights=random_weights, dtype=args.dtype, enforce_eager=args.mode == "eager",
               max_num_batched_tokens=args.token_budget, gpu_memory_utilization=args.gpu_memory_utilization,
               kvcache_block_size=args.block_size, num_kvcache_blocks=args.num_blocks, max_num_seqs=args.max_num_seqs,
               max_model_len=args.max_model_len, scheduler_policy=args.scheduler_policy, seed=args.seed,
               enable_prefix_cache=args.enable_prefix_cache, max_graph_batch=args.max_graph_batch, max_graph_tokens=args.max_graph_tokens, warm_up=args.warm_up,
               run_ahead=not args.no_run_ahead, gemm_choices=args.gemm_choices, measure_gemms=not args.no_measure_gemms,
               residual_dtype=args.residual_dtype)


def _save_choices(llm, args) -> None:
    import os
    if args.gemm_choices and not os.path.isfile(args.gemm_choices):
        llm.save_gemm_choices(args.gemm_choices)


def _percentile(values, q):
    if not values:
        return None
    values = sorted(values)
    k = (len(values) - 1) * q
    lo, hi = int(k), min(int(k) + 1, len(values) - 1)
    return values[lo] + (values[hi] - values[lo]) * (k - lo)


def _summary(values) -> dict | None:
    """mean, p50, p95, p99 and max of a request metric (tests/5090-test-TP2/suite_common.py:29-45)."""
    values = [float(v) for v in values if v is not None]
    if not values:
        return None
    return {"mean": statistics.fmean(values), "p50": _percentile(values, 0.5), "p95": _percentile(values, 0.95),
            "p99": _percentile(values, 0.99), "max": max(values)}


def cmd_generate(args) -> int:
    from . import SamplingParams
    llm = _make_llm(args)
    prompts = []
    for text in args.prompt or []:
        prompts.append(text)
    for ids in args.prompt_ids or []:
        prompts.append([int(t) for t in ids.replace(",", " ").split()])
    if not prompts:
        print("give --prompt TEXT or --prompt-ids '1 2 3' (repeatable)", file=sys.stderr)
        return 2
    sp = SamplingParams(temperature=args.temperature, max_tokens=args.output_tokens, ignore_eos=args.ignore_eos)
    outputs = llm.generate(prompts, sp, use_tqdm=not args.quiet)
    _save_choices(llm, args)
    result = [{"prompt": p, **o} for p, o in zip(prompts, outputs)]
    text = json.dumps(result, indent=2)
    if args.output:
        Path(args.output).write_text(text)
    else:
        print(text)
    return 0


def cmd_bench(args) -> int:
    import torch
    from . import SamplingParams
    if args.kernel_times and args.mode != "eager":
        print("--kernel-times needs --mode eager", file=sys.stderr)
        return 2
    llm = _make_llm(args)
    timer = None
    if args.kernel_times:
        from .native import ops
        timer = ops.kernel_times()
        times = timer.__enter__()
    vocab = llm.runner.vocab_size
    gen = torch.Generator().manual_seed(args.seed)
    results = []
    for prompt_tokens, batch in args.cases:
        for rep in range(-1, args.repeats):                        # -1: warm-up with fewer output tokens
            n_out = args.warmup_output_tokens if rep < 0 else args.output_tokens
            sp = SamplingParams(temperature=0.0, max_tokens=n_out, ignore_eos=True)
            prompts = [torch.randint(0, vocab, (prompt_tokens,), generator=gen).tolist() for _ in range(batch)]
            for p in prompts:
                llm.add_request(p, sp)
            step_ms, prefill_tokens, decode_tokens, prefill_s, decode_s = [], 0, 0, 0.0, 0.0
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while not llm.is_finished():
                _, st = llm.step()
                step_ms.append(st.seconds * 1e3)
                if st.num_prefill_tokens:
                    prefill_tokens += st.num_prefill_tokens
                    prefill_s += st.seconds
                else:
                    decode_tokens += st.num_decode_tokens
                    decode_s += st.seconds
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
            metrics = llm.get_completed_request_metrics()
            if rep < 0:
                continue
            results.append({
                "label": args.label, "prompt_tokens": prompt_tokens, "batch": batch, "output_tokens": n_out,
                "repeat": rep, "wall_s": wall,
                "prefill_tok_s": prefill_tokens / prefill_s if prefill_s else None,
                "decode_tok_s": decode_tokens / decode_s if decode_s else None,
                "step_ms_p50": _percentile(step_ms, 0.5), "step_ms_p95": _percentile(step_ms, 0.95),
                "step_ms_p99": _percentile(step_ms, 0.99),
                "ttft_ms_mean": statistics.fmean(m.ttft_ms for m in metrics),
                "tpot_ms_mean": statistics.fmean(m.tpot_ms for m in metrics if m.tpot_ms is not None) if n_out > 1 else None,
                "e2e_ms_mean": statistics.fmean(m.e2e_ms for m in metrics),
                # the requests' distributions (tests/5090-test-TP2/suite_common.py:103-183)
                "ttft_ms": _summary(m.ttft_ms for m in metrics), "tpot_ms": _summary(m.tpot_ms for m in metrics),
                "e2e_ms": _summary(m.e2e_ms for m in metrics), "queue_ms": _summary(m.queue_ms for m in metrics),
                "preemptions": llm.scheduler.num_preemptions,
            })
            print(json.dumps(results[-1]), flush=True)
    if timer is not None:
        timer.__exit__(None, None, None)
        print(times.table())
    print(json.dumps({"memory": llm.get_memory_stats()}), flush=True)
    _save_choices(llm, args)
    if args.output:
        Path(args.output).write_text(json.dumps({"model": args.model, "mode": args.mode, "dtype": args.dtype,
                                                 "token_budget": args.token_budget, "results": results}, indent=2))
    return 0


def cmd_random_model(args) -> int:
    from .weights.random_init import write_random_model
    _import_plugins(args.plugin)
    write_random_model(args.out, _named_config(args), args.seed, args.store_dtype)
    print(args.out)
    return 0


def cmd_replay(argv) -> int:
    import runpy
    script = Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    sys.argv = [str(script), *argv]
    runpy.run_path(str(script), run_name="__main__")
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "replay":
        return cmd_replay(argv[1:])
    ap = argparse.ArgumentParser(prog="python -m nanohybrid_vlm_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate from prompts")
    _engine_options(g)
    g.add_argument("--prompt", action="append", help="a text prompt (needs tokenizer.json); repeatable")
    g.add_argument("--prompt-ids", action="append", help="a prompt as token ids, e.g. '5 17 3'; repeatable")
    g.add_argument("--output-tokens", type=int, default=64)
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--output", help="JSON file for the result (default: standard output)")
    g.add_argument("--quiet", action="store_true")
    g.set_defaults(fn=cmd_generate)

    b = sub.add_parser("bench", help="throughput and latency of cases P:B")
    _engine_options(b)
    b.add_argument("--cases", type=_case, nargs="+", required=True, help="PROMPT_TOKENS:BATCH ...")
    b.add_argument("--output-tokens", type=int, default=64)
    b.add_argument("--repeats", type=int, default=2)
    b.add_argument("--warmup-output-tokens", type=int, default=8)
    b.add_argument("--label", default="run")
    b.add_argument("--kernel-times", action="store_true",
                   help="print the device time per kernel (eager mode only: events around every kernel call)")
    b.add_argument("--output", help="JSON file for all results")
    b.set_defaults(fn=cmd_bench)

    r = sub.add_parser("random-model", help="write a model folder with seeded random weights")
    r.add_argument("--out", required=True)
    r.add_argument("--shape", default="tinyA", help="a named configuration of a registered architecture")
    r.add_argument("--config", help="a config.json to use instead of a named shape")
    r.add_argument("--plugin", action="append", metavar="MODULE",
                   help="a module to import first: it may register architectures and parts of its own; repeatable")
    r.add_argument("--layers", type=int, help="override num_hidden_layers")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--store-dtype", default="bfloat16", choices=("bfloat16", "float32"))
    r.set_defaults(fn=cmd_random_model)

    sub.add_parser("replay", help="trace replay; options as bin/trace_run")
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
