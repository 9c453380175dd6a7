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
    and the logits by several 1e-2, which would hide a lost key. There the reference is the plain implementation
    with every stored result rounded to bfloat16 (``plain.stored_as``: the same formulas, whole requests, no cache),
    and the tolerance stays that of bfloat16."""
    cfg, w = plain.read_model_folder(folder)
    with plain.stored_as(torch.bfloat16):
        return {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}


def _poisoned(runner):
    """Every slot of the cache that no live request owns holds NaN: at the start all of them, later (the
    runner's ``poison_freed_pages``) every page that is given back. A kernel that reads a slot beyond a
    request's tokens, or a page that the request no longer owns, turns its logits into NaN."""
    for kv in runner.kv_tensors:
        kv.fill_(float("nan"))
    return runner


def _run_all_modes(make_runner, folder, dtype, rounding_reference=False, stats=None):
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
        if stats is not None:
            for key in stats:
                stats[key] = sorted(set(stats[key]) | set(runner.get_memory_stats()[key]))
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
    runner_stats = {"graphs_recorded": [], "graphs_refused": []}
    results = _run_all_modes(make, folder, dtype, rounding_reference=(dtype == "bfloat16" and name.endswith("_sharp")),
                             stats=runner_stats)
    if graphs:
        assert runner_stats["graphs_recorded"] and not runner_stats["graphs_refused"], runner_stats
    for mode in ("tail", "portions", "mixed"):
        for rid in results["whole"]:
            if dtype == "float32":
                # in 32-bit every sum has one order, whatever the batch: the ways of cutting agree bit for bit
                assert torch.equal(results[mode][rid], results["whole"][rid]), \
                    f"float32 {mode} against whole: request {rid}: {max_abs_diff(results[mode][rid], results['whole'][rid]):.3e}"
            else:
                # in bfloat16 all ways store the same keys and values (one kernel writes them) and round the same
                # tensors; what differs is the attention kernel (prompt portions or single tokens), which rounds the
                # softmax's weights to bfloat16 against another maximum, and the order of sums: half of what the
                # plain implementation is allowed to be away (measured where the scores are sharpened: 7e-3 for
                # configuration A and 1.9e-2 for B, the same on every run, where the allowance against the reference is
                # 4e-2; a lost key or a wrong page moves these logits by 1e-1 and more)
                d = max_abs_diff(results[mode][rid], results["whole"][rid])
                bound = (1.0 if name.endswith("_sharp") else 0.5) * TOLERANCE["bfloat16"]
                assert d <= bound, f"bfloat16 {mode} against whole: request {rid}: {d:.3e}"


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
        # (and only then: a graph that was recorded again at every step would show here)
        assert 1 <= runner.get_memory_stats()["graphs_rerecorded"] <= 4


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
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_steps_of_up_to_256_requests_replay_graphs(model_folders, dtype):
    """The batch sizes that the default configuration records (``max_graph_batch`` 256): 230 requests decode side by
    side after their prompts; 210 short ones end one after the other, so that the steps go down through the
    buckets 256, 192, 128, 96, 64, ... to the 20 long ones, which decode on from 250 to 465 keys: their bucket's
    graph, laid out for the contexts of the step that recorded it, is recorded again on the way. Every logit is
    compared with the plain implementation; in float32 also bit by bit with the same trace run eagerly."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["D"]
    cfg, w = plain.read_model_folder(folder)
    V = cfg["vocab_size"]
    short_prompt, long_prompt = 18, 250
    requests, prompt_of = {}, {}
    for i in range(210):
        requests[f"s{i}"] = rc.random_tokens(V, short_prompt + 3 + i // 4, 5000 + i)       # 3 to 55 decoded tokens
        prompt_of[f"s{i}"] = short_prompt
    for i in range(20):
        requests[f"l{i}"] = rc.random_tokens(V, long_prompt + 215, 6000 + i)
        prompt_of[f"l{i}"] = long_prompt
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:prompt_of[rid]], "want": [prompt_of[rid] - 1]}
                                     for rid, toks in requests.items()], "end": []}]
    fed = dict(prompt_of)
    while any(fed[rid] < len(toks) for rid, toks in requests.items()):
        entries = [{"id": rid, "tokens": [toks[fed[rid]]], "want": [0]} for rid, toks in requests.items() if fed[rid] < len(toks)]
        for e in entries:
            fed[e["id"]] += 1
        steps.append({"step": len(steps), "entries": entries,
                      "end": [e["id"] for e in entries if fed[e["id"]] == len(requests[e["id"]])]})
    sizes = {len(s["entries"]) for s in steps[1:]}
    assert max(sizes) == 230 and min(sizes) <= 20 and all(any(lo < n <= hi for n in sizes)
                                                         for lo, hi in ((128, 192), (96, 128), (64, 96), (48, 64)))
    pages = sum(-(-len(toks) // 64) for toks in requests.values())

    def run(graphs):
        runner = _poisoned(ModelRunner(folder, dtype=dtype, page_size=64, num_pages=pages, num_state_slots=230,
                                       use_graphs=graphs, max_model_len=512, max_graph_batch=256, poison_freed_pages=True))
        return rc.run_in_process(runner, steps), runner.get_memory_stats()

    got, stats = run(True)
    want = {rid: plain.logits(cfg, w, toks)[prompt_of[rid] - 1:] for rid, toks in requests.items()}
    _check(got, want, tolerance_for(dtype, want), f"{dtype} decoding of 230 requests through graphs")
    assert set(stats["graphs_recorded"]) >= {24, 32, 48, 64, 96, 128, 192, 256} and stats["graphs_refused"] == [], stats
    # the 20 long requests' bucket was recorded at some 305 keys and met 465: recorded again, and compared after that
    assert stats["graphs_rerecorded"] >= 1, stats
    if dtype == "float32":
        eager, _ = run(False)
        for rid in requests:
            assert torch.equal(got[rid], eager[rid]), f"float32 graphs against eager: request {rid}"


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


def _renamed(steps, suffix, first_step):
    """The same trace with other request names and step numbers, so that several traces can follow each other in
    one run of the program."""
    out = []
    for i, st in enumerate(steps):
        out.append({"step": first_step + i, "entries": [dict(e, id=e["id"] + suffix) for e in st["entries"]],
                    "end": [r + suffix for r in st["end"]]})
    return out


def _logits_from_files(out_dir, steps, vocab):
    """Per request the logits of all its tokens, from the program's <step>.f32 files."""
    parts = {}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, f"{st['step']}.f32")
        if not wanted:
            assert not os.path.exists(path)
            continue
        data = np.fromfile(path, dtype="<f4").reshape(-1, vocab)
        assert data.shape[0] == wanted
        row = 0
        for e in st["entries"]:
            n = len(e["want"])
            if n:
                parts.setdefault(e["id"], []).append(torch.from_numpy(data[row:row + n].copy()))
                row += n
    return {rid: torch.cat(p) for rid, p in parts.items()}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_run_program_in_the_four_ways(model_folders, name, dtype, tmp_path):
    """The program itself, as a user starts it, fed the same requests whole, with the last 32 tokens one by one, in
    portions of changing size and mixed on few pages (one run: the four traces follow each other, and the pool is
    made for the largest peak). Every position against the plain implementation; in float32 the four ways agree
    bit for bit."""
    folder = model_folders[name]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 7 + i) for i, n in enumerate([70, 130, 9, 64, 65, 100])}
    ways = {"whole": rc.whole(requests), "tail": rc.tail_decoded(requests), "portions": rc.portions(requests),
            "mixed": rc.mixed(requests)}
    steps, first = [], 0
    for way, trace in ways.items():
        ways[way] = _renamed(trace, "_" + way, first)
        steps += ways[way]
        first += len(trace)
    out_dir = str(tmp_path / "out")
    _trace_run(folder, dtype, steps, out_dir, max(rc.peak_tokens(t, 64) for t in ways.values()))
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}
    got = _logits_from_files(out_dir, steps, cfg["vocab_size"])
    for way in ways:
        for rid in requests:
            d = max_abs_diff(got[f"{rid}_{way}"], want[rid])
            assert d <= TOLERANCE[dtype], f"{way}: request {rid}: {d:.3e}; " + first_difference(got[f"{rid}_{way}"], want[rid], TOLERANCE[dtype])
            if dtype == "float32":
                assert torch.equal(got[f"{rid}_{way}"], got[f"{rid}_whole"]), f"float32: {way} differs from whole for {rid}"


@pytest.mark.gpu
@pytest.mark.parametrize("page", [256, 48])
def test_trace_run_program_with_other_page_sizes(model_folders, page, tmp_path):
    """Pages of 256 tokens (the engine's default) and of 48 (neither a divisor nor a multiple of 64): the pool is made
    from --max-tokens, counted in units of 64 as a caller counts it, and the mixed trace fits and is right."""
    folder = model_folders["D"]
    cfg, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], n, 70 + i) for i, n in enumerate([300, 70, 513, 64, 129, 40])}
    steps = rc.mixed(requests, sizes=(100, 7, 64, 2, 129, 33))
    out_dir = str(tmp_path / "out")
    _trace_run(folder, "bfloat16", steps, out_dir, rc.peak_tokens(steps, 64), extra=("--page-size", str(page)))
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}
    got = _logits_from_files(out_dir, steps, cfg["vocab_size"])
    tol = tolerance_for("bfloat16", want)
    for rid in requests:
        d = max_abs_diff(got[rid], want[rid])
        assert d <= tol, f"pages of {page}: request {rid}: {d:.3e}"


def test_pool_of_a_replay():
    from nanohybrid_vlm_amd.engine.replay import pages_for
    assert pages_for(640, 64) == 10 and pages_for(640, 8) == 80 and pages_for(640, 1) == 640
    # four requests of 65 tokens are counted as 4 x 128 = 512; with pages of 256 each needs one page, of 48 two
    assert pages_for(512, 256) >= 4 and pages_for(512, 48) >= 8
    # the worst case for pages of 256: four requests of 257..320 tokens, counted as 4 x 320
    assert pages_for(4 * 320, 256) >= 8
    for page in (3, 48, 100, 256, 1000):
        for lengths in ([1, 1, 1, 1], [64, 65, 129, 300], [257, 320, 513, 1], [1000, 999, 63, 64]):
            counted = sum(-(-n // 64) * 64 for n in lengths)
            assert pages_for(counted, page) >= sum(-(-n // page) for n in lengths), (page, lengths)




def _replay_with_rounded_residual(folder, device, graphs):
    """The residual stream carried in bfloat16, rounded after every addition as the reference carries it
    (nanovllm/layers/layernorm.py:34-40), instead of in float32: the same four ways against the plain implementation."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    cfg, _ = plain.read_model_folder(folder)
    requests = _requests(cfg["vocab_size"])
    want = _plain_logits(folder, requests)
    tol = tolerance_for("bfloat16", want)
    results = {}
    for mode, steps in [("whole", rc.whole(requests)), ("tail", rc.tail_decoded(requests)),
                        ("portions", rc.portions(requests)), ("mixed", rc.mixed(requests))]:
        pages = rc.peak_tokens(steps, 8) // 8
        runner = _poisoned(ModelRunner(folder, dtype="bfloat16", device=device, page_size=8, num_pages=pages, num_state_slots=4,
                                       use_graphs=graphs, max_model_len=160, poison_freed_pages=True, residual_float32=False))
        assert all(not part.residual_float32 for part in runner.model.walk() if hasattr(part, "residual_float32"))
        results[mode] = rc.run_in_process(runner, steps)
        _check(results[mode], want, tol, f"rounded residual, {mode}")
    return results


@pytest.mark.parametrize("name", ["A", "B"])
def test_rounded_residual_on_emulated_kernels(model_folders, emulated_kernels, name):
    _replay_with_rounded_residual(model_folders[name], "cpu", graphs=False)


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_rounded_residual_on_gpu(model_folders, name, graphs):
    results = _replay_with_rounded_residual(model_folders[name], "cuda:0", graphs)
    for mode in ("tail", "portions", "mixed"):
        for rid in results["whole"]:
            d = max_abs_diff(results[mode][rid], results["whole"][rid])
            assert d <= 0.5 * TOLERANCE["bfloat16"], f"rounded residual, {mode} against whole: request {rid}: {d:.3e}"


# ---------------------------------------------------------------- a whole trace as one object

def _as_whole_trace(requests, steps, **more):
    """The steps of ``replay_cases`` in the other form: the requests' tokens once, and per step how many each feeds."""
    return dict({"requests": requests, "steps": [[{"req": e["id"], "n": len(e["tokens"])} for e in st["entries"]]
                                                 for st in steps]}, **more)


def test_steps_of_a_whole_trace():
    from nanohybrid_vlm_amd.engine.replay import peak_tokens_of, steps_of_trace
    requests = {"a": [5, 17, 3, 9], "b": [1, 2]}
    records = steps_of_trace({"requests": requests, "steps": [[{"req": "a", "n": 3}], [{"req": "a", "n": 1}, {"req": "b", "n": 2}]]})
    assert records == [{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 1, 2]}], "end": []},
                       {"step": 1, "entries": [{"id": "a", "tokens": [9], "want": [0]},
                                               {"id": "b", "tokens": [1, 2], "want": [0, 1]}], "end": ["a", "b"]}]
    assert peak_tokens_of(records) == 128 and peak_tokens_of(records, unit=2) == 6
    mixed = rc.mixed(_requests(50))
    assert steps_of_trace(_as_whole_trace(_requests(50), mixed)) == [
        dict(st, entries=[dict(e, want=list(range(len(e["tokens"])))) for e in st["entries"]]) for st in mixed]
    assert peak_tokens_of(mixed, 8) == rc.peak_tokens(mixed, 8)
    for bad, what in [({"requests": requests, "steps": [[{"req": "c", "n": 1}]]}, "not among"),
                      ({"requests": requests, "steps": [[{"req": "a", "n": 5}]]}, "cannot feed"),
                      ({"requests": requests, "steps": [[{"req": "a", "n": 0}]]}, "cannot feed"),
                      ({"requests": requests, "steps": [[{"req": "a", "n": 4}]]}, "do not feed all tokens of request(s) b"),
                      ({"requests": {}, "steps": []}, "a trace holds")]:
        with pytest.raises(ValueError, match=what.replace("(", r"\(").replace(")", r"\)")):
            steps_of_trace(bad)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_with_a_whole_trace(model_folders, dtype, tmp_path):
    """``bin/trace_run --trace trace.json --out logits.safetensors``: the trace names model, element type, page size
    and pages itself; the file holds every request's logits at all its positions."""
    from safetensors.torch import load_file
    folder = model_folders["B"]
    cfg, _ = plain.read_model_folder(folder)
    requests = _requests(cfg["vocab_size"])
    want = _plain_logits(folder, requests)
    steps = rc.mixed(requests)
    trace = _as_whole_trace(requests, steps, model=folder, dtype=dtype, block_size=16,
                            num_blocks=rc.peak_tokens(steps, 16) // 16)
    path = str(tmp_path / "trace.json")
    with open(path, "w") as f:
        json.dump(trace, f)
    out = str(tmp_path / "logits.safetensors")
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bin", "trace_run"), "--trace", path, "--out", out],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    got = load_file(out)
    assert set(got) == set(requests) and all(got[rid].dtype == torch.float32 for rid in got)
    _check(got, want, tolerance_for(dtype, want), f"whole trace, {dtype}")
    # a random model named by shape and seed, files a step: the same steps as lines give the same files
    trace = _as_whole_trace(requests, steps, shape="tinyB", seed=5, dtype="float32", block_size=16)
    with open(path, "w") as f:
        json.dump(trace, f)
    out_dir = str(tmp_path / "files")
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bin", "trace_run"), "--trace", path, "--out", out_dir],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert sorted(os.listdir(out_dir), key=lambda n: int(n.split(".")[0])) == [f"{i}.f32" for i in range(len(steps))]


# ---------------------------------------------------------------- short steps of any make as graphs

def _last_places_only(steps):
    """The same steps, asking for one place of every entry (its last): what a serving engine asks for."""
    return [dict(st, entries=[dict(e, want=[len(e["tokens"]) - 1]) for e in st["entries"]]) for st in steps]


def _replay_short_steps(folder, dtype, device, graphs, max_graph_tokens=64):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    cfg, _ = plain.read_model_folder(folder)
    requests = _requests(cfg["vocab_size"])
    full = _plain_logits(folder, requests)
    results, stats = {}, {"mixed_graphs_recorded": [], "mixed_graphs_refused": []}
    for mode, steps in [("portions", rc.portions(requests)), ("mixed", rc.mixed(requests))]:
        steps = _last_places_only(steps)
        # the plain logits at the places that the steps ask for, request by request
        want, fed = {}, {rid: 0 for rid in requests}
        for st in steps:
            for e in st["entries"]:
                fed[e["id"]] += len(e["tokens"])
                want.setdefault(e["id"], []).append(full[e["id"]][fed[e["id"]] - 1])
        want = {rid: torch.stack(rows) for rid, rows in want.items()}
        pages = rc.peak_tokens(steps, 8) // 8
        runner = _poisoned(ModelRunner(folder, dtype=dtype, device=device, page_size=8, num_pages=pages, num_state_slots=4,
                                       use_graphs=graphs, max_model_len=160, poison_freed_pages=True,
                                       max_graph_tokens=max_graph_tokens))
        results[mode] = rc.run_in_process(runner, steps)
        _check(results[mode], want, tolerance_for(dtype, want), f"{dtype} {mode}, one place a request")
        for key in stats:
            stats[key] = sorted(set(stats[key]) | set(runner.get_memory_stats()[key]))
    return results, stats


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_short_steps_replay_graphs(model_folders, name, dtype):
    """Portions of prompts, alone and beside decoded tokens, of up to 64 tokens a step: recorded for (tokens,
    requests) rounded up, the bucket filled by a request of its own on the spare page. The same logits as run
    eagerly, bit for bit in float32."""
    folder = model_folders[name]
    with_graphs, stats = _replay_short_steps(folder, dtype, "cuda:0", graphs=True)
    assert stats["mixed_graphs_refused"] == [] and len(stats["mixed_graphs_recorded"]) >= 3, stats
    assert {t for t, _ in stats["mixed_graphs_recorded"]} <= {16, 24, 32, 48, 64}
    eager, none = _replay_short_steps(folder, dtype, "cuda:0", graphs=False)
    assert none["mixed_graphs_recorded"] == []
    for mode in with_graphs:
        for rid in with_graphs[mode]:
            if dtype == "float32":
                assert torch.equal(with_graphs[mode][rid], eager[mode][rid]), f"{mode}: request {rid}"
            else:
                d = max_abs_diff(with_graphs[mode][rid], eager[mode][rid])
                assert d <= 0.5 * TOLERANCE["bfloat16"], f"{mode}: request {rid}: {d:.3e}"


@pytest.mark.gpu
def test_short_step_graphs_stay_within_the_models_positions(model_folders):
    """The tokens that fill a bucket stand at positions below the bucket's size; a model that is allowed fewer
    positions than that runs such steps eagerly."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    folder = model_folders["A"]
    cfg, w = plain.read_model_folder(folder)
    tokens = rc.random_tokens(cfg["vocab_size"], 40, 5)
    runner = ModelRunner(folder, dtype="float32", page_size=64, num_pages=2, num_state_slots=2, use_graphs=True,
                         max_model_len=44, max_graph_tokens=256)
    got = rc.run_in_process(runner, [{"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": [39]}], "end": ["a"]}])
    assert runner.get_memory_stats()["mixed_graphs_recorded"] == []           # 40 tokens round up to 48 > 44 positions
    assert max_abs_diff(got["a"], plain.logits(cfg, w, tokens)[39:]) <= tolerance_for("float32", got)
    runner = ModelRunner(folder, dtype="float32", page_size=64, num_pages=2, num_state_slots=2, use_graphs=True,
                         max_model_len=64, max_graph_tokens=256)
    got = rc.run_in_process(runner, [{"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": [39]}], "end": ["a"]}])
    assert runner.get_memory_stats()["mixed_graphs_recorded"] == [(48, 1)]
    assert max_abs_diff(got["a"], plain.logits(cfg, w, tokens)[39:]) <= tolerance_for("float32", got)


def _decode_logits(folder, device, dtype, fuse, graphs=False):
    """Six requests decoding side by side after their prompts (steps of up to 16 rows), every logit."""
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    cfg, _ = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(cfg["vocab_size"], 20 + 3 * i, 700 + i) for i in range(6)}
    alone = rc.tail_decoded(requests, tail=8)
    steps = alone + _renamed(rc.mixed(requests, max_live=6, sizes=(3, 2, 5)), "'", len(alone))
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=8, num_pages=64, num_state_slots=8, use_graphs=graphs,
                         max_model_len=128, fuse_norms=fuse)
    return requests, rc.run_in_process(runner, steps), runner


@pytest.mark.parametrize("name", ["A", "C"])
def test_products_take_over_norms_on_emulated_kernels(model_folders, emulated_kernels, name):
    """In bfloat16 a product of up to 16 rows may make the residual addition after it and leave only the scaling of
    the rows to the product that reads the norm. With and without, the logits agree within bfloat16's rounding, and
    with it the work really is taken over (the stand-in's fused product is called, the norm's kernel far less)."""
    from nanohybrid_vlm_amd.native import ops
    backend = ops.backend()
    calls = {"fused": 0, "norm": 0}
    fused_linear, rmsnorm = backend.fused_linear, backend.rmsnorm
    backend.fused_linear = lambda *a, **k: (calls.__setitem__("fused", calls["fused"] + 1), fused_linear(*a, **k))[1]
    backend.rmsnorm = lambda *a, **k: (calls.__setitem__("norm", calls["norm"] + 1), rmsnorm(*a, **k))[1]
    try:
        requests, with_fusion, _ = _decode_logits(model_folders[name], "cpu", "bfloat16", True)
        taken_over = dict(calls)
        calls.update(fused=0, norm=0)
        _, without, _ = _decode_logits(model_folders[name], "cpu", "bfloat16", False)
        plain_way = dict(calls)
    finally:
        del backend.fused_linear, backend.rmsnorm
    assert plain_way["fused"] == 0 and taken_over["fused"] > 0
    assert taken_over["norm"] < 0.5 * plain_way["norm"], (taken_over, plain_way)
    want = _plain_logits(model_folders[name], requests)
    tol = tolerance_for("bfloat16", want)
    for rid in with_fusion:
        reference = want[rid.rstrip("'")]
        assert max_abs_diff(with_fusion[rid], without[rid]) <= tol, rid
        assert max_abs_diff(with_fusion[rid], reference) <= tol, rid


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_products_take_over_norms_on_gpu(model_folders, name, graphs):
    """The same on the GPU, for all four small configurations (with and without q/k norms, projection biases, tied
    heads; head sizes 16 to 128): with the norms taken over and without, against the plain implementation."""
    folder = model_folders[name]
    requests, with_fusion, runner = _decode_logits(folder, "cuda:0", "bfloat16", True, graphs)
    _, without, _ = _decode_logits(folder, "cuda:0", "bfloat16", False, graphs)
    want = _plain_logits(folder, requests)
    tol = tolerance_for("bfloat16", want)
    for rid in with_fusion:
        reference = want[rid.rstrip("'")]
        assert max_abs_diff(with_fusion[rid], reference) <= tol, f"taken over, {rid}"
        assert max_abs_diff(without[rid], reference) <= tol, f"plain, {rid}"
    if graphs:
        stats = runner.get_memory_stats()
        assert stats["graphs_recorded"] and not stats["graphs_refused"] and not stats["mixed_graphs_refused"], stats
