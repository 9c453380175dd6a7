"""The same requests fed whole, with a decoded tail, in portions and mixed with
others on few pages must give the plain implementation's logits at every position.

Without a GPU the engine's logic runs on the CPU stand-in for the kernels
(float32 only); with ``-m gpu`` it runs on the HIP kernels in float32 and bfloat16.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import replay_cases as rc
from helpers import TOLERANCE, first_difference, max_abs_diff, sharpen, tolerance_for

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _requests(vocab):
    # lengths around page edges (pages of 8 and 64) and one long request
    return {f"r{i}": rc.random_tokens(vocab, n, 100 + i) for i, n in enumerate([5, 64, 33, 65, 130, 17, 96, 1, 40])}


def _plain_logits(folder, requests):
    cfg, w = plain.read_model_folder(folder)
    return {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}


def _check(got, want, tol, what):
    for rid in want:
        assert got[rid].shape == want[rid].shape, f"{what}: request {rid}: shape {got[rid].shape}"
        d = max_abs_diff(got[rid], want[rid])
        assert d <= tol, f"{what}: request {rid}: max diff {d:.3e} > {tol:.1e}; {first_difference(got[rid], want[rid], tol)}"


def _rounding_reference(folder, requests):
    """bfloat16 with sharpened attention: rounding q and k to 8 bits moves scores of size 16 by up to 0.06
    and the logits by several 1e-2, which would hide a lost key. There the reference is the CPU stand-in for
    the kernels run in bfloat16 (same places of rounding, whole requests, its float32 run is itself checked
    against the plain implementation), and the tolerance stays that of bfloat16."""
    from emulated_kernels import EmulatedBackend
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    from nanohybrid_vlm_amd.native import ops
    old = ops._backend
    ops.set_backend(EmulatedBackend())
    try:
        runner = ModelRunner(folder, dtype="bfloat16", device="cpu", page_size=16, num_pages=16, num_state_slots=2)
        return rc.run_in_process(runner, rc.whole(requests))
    finally:
        ops.set_backend(old)


def _poisoned(runner):
    """Every slot of the cache that no live request owns holds NaN: at the start all of them, later (the
    runner's ``poison_freed_pages``) every page that is given back. A kernel that reads a slot beyond a
    request's tokens, or a page that the request no longer owns, turns its logits into NaN."""
    for kv in runner.kv_tensors:
        kv.fill_(float("nan"))
    return runner


def _run_all_modes(make_runner, folder, dtype, rounding_reference=False):
    cfg, _ = plain.read_model_folder(folder)
    requests = _requests(cfg["vocab_size"])
    want = _rounding_reference(folder, requests) if rounding_reference else _plain_logits(folder, requests)
    tol = tolerance_for(dtype, want)
    if rounding_reference:
        # both sides round to bfloat16 here, at the same places but with sums in another order, and the
        # sharpened scores amplify each side's rounding: their difference may be twice one side's error.
        # (A lost key or a wrong page moves these logits by about their whole deviation.)
        tol *= 2
    results = {}
    for mode, steps, page, pages in [
        ("whole", rc.whole(requests), 8, 20),
        ("tail", rc.tail_decoded(requests), 8, 20),
        ("portions", rc.portions(requests), 8, 20),
        # so few pages that every page is used again several times
        ("mixed", rc.mixed(requests), 8, None),
    ]:
        if pages is None:
            pages = rc.peak_tokens(steps, page) // page
        runner = make_runner(folder, dtype, page, pages)
        results[mode] = rc.run_in_process(runner, steps)
        _check(results[mode], want, tol, f"{dtype} {mode}")
        assert not runner.cache.requests, "every request was ended"
        assert runner.cache.num_free_pages(0) == pages, "every page came back"
    return results


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_on_emulated_kernels(model_folders, emulated_kernels, name, tmp_path):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner

    def make(folder, dtype, page, pages):
        return _poisoned(ModelRunner(folder, dtype=dtype, device="cpu", page_size=page, num_pages=pages,
                                     num_state_slots=4, poison_freed_pages=True))

    folder = model_folders[name]
    if name != "C":
        folder = sharpen(folder, str(tmp_path / "sharp"))
    _run_all_modes(make, folder, "float32")


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "A_sharp", "B_sharp"])
def test_replay_on_gpu(model_folders, name, dtype, graphs, tmp_path):
    """With ``graphs`` every step of single tokens replays a recorded HIP graph (one per batch size), between
    eager steps of prompt portions: each replay is compared with the plain implementation."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner

    def make(folder, dtype, page, pages):
        return _poisoned(ModelRunner(folder, dtype=dtype, device="cuda:0", page_size=page, num_pages=pages,
                                     num_state_slots=4, use_graphs=graphs, max_model_len=160, poison_freed_pages=True))

    folder = model_folders[name.split("_")[0]]
    if name.endswith("_sharp"):
        folder = sharpen(folder, str(tmp_path / "sharp"))
    results = _run_all_modes(make, folder, dtype, rounding_reference=(dtype == "bfloat16" and name.endswith("_sharp")))
    if dtype == "float32":
        # in 32-bit the ways of cutting agree with each other far more closely than with the plain implementation
        for mode in ("tail", "portions", "mixed"):
            for rid in results["whole"]:
                d = max_abs_diff(results[mode][rid], results["whole"][rid])
                assert d <= 2e-6, f"float32 {mode} against whole: request {rid}: {d:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(model_folders, dtype, graphs):
    """One token a step from the very first token on, 500 steps, two requests side by side that start at
    different times: every page edge, every split edge of the decode kernel and the first positions."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    a = rc.random_tokens(cfg["vocab_size"], 500, 1)
    b = rc.random_tokens(cfg["vocab_size"], 300, 2)
    steps = []
    for i in range(500):
        entries = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        if 100 <= i < 400:
            entries.append({"id": "b", "tokens": [b[i - 100]], "want": [0]})
        steps.append({"step": i, "entries": entries, "end": (["a"] if i == 499 else []) + (["b"] if i == 399 else [])})
    runner = ModelRunner(folder, dtype=dtype, page_size=8, num_pages=101, num_state_slots=2, use_graphs=graphs,
                         max_model_len=512)
    got = rc.run_in_process(runner, steps)
    _check(got, {"a": plain.logits(cfg, w, a), "b": plain.logits(cfg, w, b)}, TOLERANCE[dtype], f"{dtype} long decoding")
    if graphs:
        # a graph's kernels are laid out for the contexts of the step that recorded it: past 384 keys it is recorded again
        assert runner.get_memory_stats()["graphs_rerecorded"] >= 1


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_the_family_head_size(model_folders, dtype, graphs):
    """Head size 128 with 4 query heads per key/value head and pages of 64 and 256: the kernels and tile shapes
    that the real sizes use, in a model small enough for the plain implementation. Requests up to 700 tokens."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["D"]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 200 + i) for i, n in enumerate([700, 65, 300, 129, 16])}
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}
    for page in (64, 256):
        for mode, steps in [("whole", rc.whole(requests)), ("tail", rc.tail_decoded(requests, tail=40)),
                            ("mixed", rc.mixed(requests, sizes=(100, 7, 64, 2, 129, 33)))]:
            pages = rc.peak_tokens(steps, page) // page
            runner = _poisoned(ModelRunner(folder, dtype=dtype, page_size=page, num_pages=pages, num_state_slots=4,
                                           use_graphs=graphs, max_model_len=768, poison_freed_pages=True))
            got = rc.run_in_process(runner, steps)
            _check(got, want, tolerance_for(dtype, want), f"{dtype} head size 128, pages of {page}, {mode}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_steps_of_many_requests_replay_checked_graphs(model_folders, dtype):
    """Steps of 17 to 64 single tokens: in bfloat16 their graphs hold the library's matrix products and are
    checked when recorded (replayed three times between eager work, compared bit by bit). 40 requests decode
    side by side, 15 of them end, the rest goes on: graphs of more than 16 rows, every logit against the plain
    implementation."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["D"]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], 30 + (i * 7) % 23 + (20 if i >= 15 else 0), 400 + i)
                for i in range(40)}
    prompt = 18
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:prompt], "want": [prompt - 1]}
                                     for rid, toks in requests.items()], "end": []}]
    fed = {rid: prompt for rid in requests}
    while any(fed[rid] < len(toks) for rid, toks in requests.items()):
        entries = [{"id": rid, "tokens": [toks[fed[rid]]], "want": [0]} for rid, toks in requests.items() if fed[rid] < len(toks)]
        for e in entries:
            fed[e["id"]] += 1
        steps.append({"step": len(steps), "entries": entries,
                      "end": [e["id"] for e in entries if fed[e["id"]] == len(requests[e["id"]])]})
    sizes = {len(s["entries"]) for s in steps[1:]}
    assert max(sizes) == 40 and any(16 < n <= 32 for n in sizes)
    runner = ModelRunner(folder, dtype=dtype, page_size=64, num_pages=2 * len(requests) + 1, num_state_slots=40,
                         use_graphs=True, max_model_len=128)
    got = rc.run_in_process(runner, steps)
    want = {rid: plain.logits(cfg, w, toks)[prompt - 1:] for rid, toks in requests.items()}
    _check(got, want, tolerance_for(dtype, want), f"{dtype} decoding of 40 requests through graphs")
    stats = runner.get_memory_stats()
    recorded = stats["graphs_recorded"]
    assert max(recorded) >= 40 and any(16 < b <= 32 for b in recorded) and stats["graphs_refused"] == [], stats


@pytest.mark.gpu
def test_a_graph_that_fails_its_check_is_not_used(model_folders, capfd):
    """The check of a graph with library calls in it is made to fail from the host: the step that recorded it
    returns the eager result, later steps of that size run eagerly, and every logit is still right."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["D"]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], 24 + i % 3, 900 + i) for i in range(20)}
    prompt = 18
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:prompt], "want": [prompt - 1]}
                                     for rid, toks in requests.items()], "end": []}]
    for t in range(prompt, 26):
        entries = [{"id": rid, "tokens": [toks[t]], "want": [0]} for rid, toks in requests.items() if t < len(toks)]
        steps.append({"step": len(steps), "entries": entries, "end": [e["id"] for e in entries if t == len(requests[e["id"]]) - 1]})
    runner = ModelRunner(folder, dtype="bfloat16", page_size=64, num_pages=len(requests) + 1, num_state_slots=20,
                         use_graphs=True, max_model_len=64)
    runner.graph_check = lambda replayed, eager: False
    got = rc.run_in_process(runner, steps)
    want = {rid: plain.logits(cfg, w, toks)[prompt - 1:] for rid, toks in requests.items()}
    _check(got, want, tolerance_for("bfloat16", want), "decoding of 20 requests with refused graphs")
    stats = runner.get_memory_stats()
    assert 24 in stats["graphs_refused"] and stats["graphs_recorded"] == [], stats
    assert "run eagerly" in capfd.readouterr().err


def _trace_run(folder, dtype, steps, out_dir, max_tokens, extra=()):
    cmd = [sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *extra]
    proc = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps]
    return proc


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, dtype, tmp_path):
    """The program itself, as a user starts it: mixed trace, pool made for the trace's peak, files compared."""
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 7 + i) for i, n in enumerate([70, 130, 9, 64, 65, 100])}
    steps = rc.mixed(requests)
    out_dir = str(tmp_path / "out")
    _trace_run(folder, dtype, steps, out_dir, rc.peak_tokens(steps, 64))
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}
    fed = {rid: 0 for rid in requests}
    V = cfg["vocab_size"]
    for st in steps:
        data = np.fromfile(os.path.join(out_dir, f"{st['step']}.f32"), dtype="<f4").reshape(-1, V)
        row = 0
        for e in st["entries"]:
            n = len(e["tokens"])
            ref = want[e["id"]][fed[e["id"]]:fed[e["id"]] + n]
            d = max_abs_diff(torch.from_numpy(data[row:row + n].copy()), ref)
            assert d <= TOLERANCE[dtype], f"step {st['step']} request {e['id']}: {d:.3e}"
            fed[e["id"]] += n
            row += n
        assert row == data.shape[0]
