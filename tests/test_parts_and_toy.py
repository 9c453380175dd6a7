"""The parts are general: a toy architecture, defined in the tests and nowhere in the package
(``toy_architecture.py``), is registered, built, loaded and stepped through the unchanged
engine (the step function, the scheduler, the entry point, the command line) and compared
with a plain whole-sequence computation.
Also: each built-in part alone against its plain function."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_qwen3 as plain
import replay_cases as rc
import toy_architecture as toy
from helpers import max_abs_diff
from nanohybrid_vlm_amd.cache.manager import NO_PAGE
from nanohybrid_vlm_amd.parts.model import DecoderModel, RunEntry
from nanohybrid_vlm_amd.weights.random_init import write_random_model
from toy_architecture import VOCAB, WINDOW, toy_plain_logits, toy_spec

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture()
def toy_architecture():
    toy.register()
    yield
    toy.unregister()


def _toy_folder(tmp_path, device_state=False, **keys):
    cfg = {"architectures": ["ToyForCausalLM"], "model_type": "toy", "device_state": device_state, **keys}
    return write_random_model(str(tmp_path / f"toy{int(device_state)}{int(bool(keys.get('no_window')))}"), cfg, seed=4)


def _toy_check(device, dtype, tol, tmp_path, device_state=False, graphs=False):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner, StepEntry
    folder = _toy_folder(tmp_path, device_state)
    _, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(VOCAB, n, 30 + i) for i, n in enumerate([9, 40, 23, 17, 31])}
    want = {rid: toy_plain_logits(w, toks) for rid, toks in requests.items()}
    for mode, steps in [("whole", rc.whole(requests)), ("portions", rc.portions(requests)),
                        ("tail", rc.tail_decoded(requests, tail=12)), ("mixed", rc.mixed(requests, max_live=3))]:
        pages = rc.peak_tokens(steps, 4) // 4
        runner = ModelRunner(folder, dtype=dtype, device=device, page_size=4, num_pages=pages, num_state_slots=3,
                             use_graphs=graphs, max_model_len=64)
        assert len(runner.cache.groups) == 2 and runner.cache.groups[1].window == WINDOW
        assert len(runner.kv_tensors) == 3 and len(runner.state_pools) == 1       # entries 0, 2, 3 store keys; entry 1 state
        # a part that walks over the step's requests on the host keeps the whole model out of graphs
        assert runner.use_graphs == (graphs and device_state)
        got = rc.run_in_process(runner, steps)
        for rid in requests:
            d = max_abs_diff(got[rid], want[rid])
            assert d <= tol, f"toy {mode}: request {rid}: {d:.3e}"
        assert all(runner.cache.num_free_pages(g) == pages for g in range(2))
        if runner.use_graphs and mode in ("tail", "mixed"):
            stats = runner.get_memory_stats()
            assert stats["graphs_recorded"] and not stats["graphs_refused"], stats
    # positions of the requests' own on the second axis (the first stays the index): every way of cutting again
    second_axis = {rid: [(5 * i + 3) % 11 + i // 3 for i in range(len(toks))] for rid, toks in requests.items()}
    want = {rid: toy_plain_logits(w, toks, positions=[list(range(len(toks))), second_axis[rid]])
            for rid, toks in requests.items()}
    for mode, steps in [("portions", rc.portions(requests)), ("tail", rc.tail_decoded(requests, tail=12)),
                        ("mixed", rc.mixed(requests, max_live=3))]:
        fed = {rid: 0 for rid in requests}
        for st in steps:
            for e in st["entries"]:
                a, b = fed[e["id"]], fed[e["id"]] + len(e["tokens"])
                e["positions"] = [list(range(a, b)), second_axis[e["id"]][a:b]]
                fed[e["id"]] = b
        pages = rc.peak_tokens(steps, 4) // 4
        runner = ModelRunner(folder, dtype=dtype, device=device, page_size=4, num_pages=pages, num_state_slots=3,
                             use_graphs=graphs, max_model_len=64)
        got = rc.run_in_process(runner, steps)
        for rid in requests:
            d = max_abs_diff(got[rid], want[rid])
            assert d <= tol, f"toy with positions of its own, {mode}: request {rid}: {d:.3e}"
    # the windowed group gives pages back while a request is still alive
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=4, num_pages=16, num_state_slots=3)
    runner.step([StepEntry("x", requests["r1"][:30], [29])])
    assert runner.cache.block_table("x", 0).count(NO_PAGE) == 0
    assert runner.cache.block_table("x", 1).count(NO_PAGE) == (30 - WINDOW + 1) // 4


@pytest.mark.parametrize("device_state", [False, True], ids=["state on the host", "state on the device"])
def test_toy_architecture_on_emulated_kernels(toy_architecture, emulated_kernels, tmp_path, device_state):
    _toy_check("cpu", "float32", 2e-5, tmp_path, device_state)


@pytest.mark.gpu
@pytest.mark.parametrize("device_state,graphs", [(False, False), (False, True), (True, True)],
                         ids=["state on the host", "state on the host, graphs asked for", "state on the device, graphs"])
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_toy_architecture_on_gpu(toy_architecture, dtype, tol, tmp_path, device_state, graphs):
    _toy_check("cuda:0", dtype, tol, tmp_path, device_state, graphs)


def _toy_greedy(w, prompt, n, eos=None, no_window=False):
    ids, out = list(prompt), []
    for _ in range(n):
        t = int(toy_plain_logits(w, ids, no_window)[-1].argmax())
        ids.append(t)
        out.append(t)
        if eos is not None and t == eos:
            break
    return out


def _toy_generate(device, dtype, tmp_path, device_state, no_window=False, **options):
    """The toy through the entry point: scheduler, portions of prompts, so few pages that requests are pushed
    out and computed again (their state starts again from zero), steps issued ahead where the model allows."""
    from nanohybrid_vlm_amd import LLM, SamplingParams
    prompts = [rc.random_tokens(VOCAB, n, 60 + n) for n in (5, 19, 11, 26)]
    results = {}
    for what, pages in (("ample", 64), ("few pages", 13)):
        folder = _toy_folder(tmp_path, device_state, no_window=no_window)
        _, w = plain.read_model_folder(folder)
        # (no prompt is ever overdue: what is pushed out is pushed out for pages, on a fast machine and a slow one)
        llm = LLM(folder, device=device, dtype=dtype, kvcache_block_size=4, num_kvcache_blocks=pages,
                  max_num_batched_tokens=12, max_num_seqs=3, max_model_len=64, max_prefill_wait_ms=1e9, **options)
        assert llm.config.eos == -1 and llm.config.max_model_len == 64      # the toy names no end token
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10), use_tqdm=False)
        results[what] = [o["token_ids"] for o in outs]
        if dtype == "float32":
            assert results[what] == [_toy_greedy(w, p, 10, no_window=no_window) for p in prompts], what
        if what == "few pages":
            assert llm.scheduler.num_preemptions > 0, "the small cache was meant to force a request out"
        stats = llm.get_memory_stats()
        assert stats["live_requests"] == 0 and all(g["free_pages"] == g["pages"] for g in stats["groups"])
        yield llm
    assert results["ample"] == results["few pages"] or dtype != "float32"
    # a configuration that names an end token: the engine takes it from the built model
    folder = write_random_model(str(tmp_path / "toy_eos"), {"architectures": ["ToyForCausalLM"], "model_type": "toy",
                                                            "device_state": device_state, "eos_token_id": 5}, seed=4)
    llm = LLM(folder, device=device, dtype=dtype, kvcache_block_size=4, num_kvcache_blocks=32, max_model_len=64, **options)
    assert llm.config.eos == 5


@pytest.mark.parametrize("device_state", [False, True], ids=["state on the host", "state on the device"])
def test_toy_generates_through_the_entry_point_on_emulated_kernels(toy_architecture, emulated_kernels, tmp_path, device_state):
    for _ in _toy_generate("cpu", "float32", tmp_path, device_state):
        pass


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("device_state,no_window", [(False, False), (True, False), (True, True)],
                         ids=["state on the host", "state on the device", "state on the device, no window"])
def test_toy_generates_through_the_entry_point_on_gpu(toy_architecture, tmp_path, device_state, no_window, dtype):
    for llm in _toy_generate("cuda:0", dtype, tmp_path, device_state, no_window):
        stats = llm.get_memory_stats()
        if device_state:
            # per-request state keeps a model neither out of graphs nor out of steps issued ahead (a step issued
            # ahead may have to be taken back, which a window's pages, given back as it moves, do not allow)
            assert stats["graphs_recorded"] and not stats["graphs_refused"], stats
            assert stats["mixed_graphs_recorded"] and not stats["mixed_graphs_refused"], stats   # prompt portions as graphs too
            assert (llm.num_steps_ahead > 0) == no_window
        else:
            assert not stats["graphs_recorded"] and not stats["mixed_graphs_recorded"] and llm.num_steps_ahead == 0


@pytest.mark.gpu
def test_toy_through_the_command_line(tmp_path):
    """``--plugin`` imports the module that registers the toy; nothing in the package names it."""
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([os.path.join(REPO, "tests"), REPO, os.environ.get("PYTHONPATH", "")]))
    toy.register()
    try:
        folder = _toy_folder(tmp_path, device_state=True)
        _, w = plain.read_model_folder(folder)
    finally:
        toy.unregister()
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", "generate", "--plugin", "toy_architecture",
                           "--model", folder, "--dtype", "float32", "--prompt-ids", "5 17 3 60", "--prompt-ids", "9 8 7",
                           "--output-tokens", "6", "--temperature", "0", "--block-size", "4", "--num-blocks", "32",
                           "--max-model-len", "64", "--quiet"], cwd=REPO, env=env, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = json.loads(proc.stdout)
    assert [o["token_ids"] for o in out] == [_toy_greedy(w, p, 6) for p in ([5, 17, 3, 60], [9, 8, 7])]
    # random weights of a configuration given as a file, for an architecture the package does not know
    cfg_file = tmp_path / "toy_config.json"
    cfg_file.write_text(json.dumps({"architectures": ["ToyForCausalLM"], "model_type": "toy", "device_state": True}))
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", "generate", "--plugin", "toy_architecture",
                           "--random-weights", "3", "--config", str(cfg_file), "--prompt-ids", "1 2 3", "--output-tokens", "4",
                           "--temperature", "0", "--block-size", "4", "--num-blocks", "32", "--max-model-len", "64", "--quiet"],
                          cwd=REPO, env=env, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert len(json.loads(proc.stdout)[0]["token_ids"]) == 4


def test_run_order_is_checked():
    toy.register_parts()
    spec = toy_spec({})
    try:
        spec.run_order = [RunEntry(0), RunEntry(5)]
        with pytest.raises(ValueError, match="names layer 5"):
            DecoderModel(spec)
        spec.run_order = [RunEntry(0), RunEntry(2, cache=0)]                      # a window layer on an all-keys cache
        with pytest.raises(ValueError, match="different caches"):
            DecoderModel(spec)
        spec.run_order = [RunEntry(0, cache=0)]
        with pytest.raises(ValueError, match="earlier entry"):
            DecoderModel(spec)
    finally:
        toy.unregister_parts()
    with pytest.raises(KeyError, match="unknown position encoding"):
        DecoderModel(toy_spec({}))


# ---------------------------------------------------------------- built-in parts alone, on the GPU
def _dev(t, dtype):
    return t.to(dtype).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_builtin_parts_alone(dtype):
    from nanohybrid_vlm_amd.parts.feed_forward import SwiGLU
    from nanohybrid_vlm_amd.parts.norms import RMSNorm
    from nanohybrid_vlm_amd.parts.positions import RotaryEmbedding
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(11, 72, generator=g).to(dtype)
    # norm
    norm = RMSNorm(72, 1e-4)
    wn = (1 + 0.1 * torch.randn(72, generator=g)).to(dtype)
    norm.bind({"weight": wn.cuda()})
    torch.testing.assert_close(norm.forward(x.cuda()).float().cpu(), plain.rms_norm(x, wn.float(), 1e-4), **tol)
    y, res = norm.forward_start(x.cuda())
    y2, res = norm.forward_add(x.cuda(), res)
    ref, s = plain.add_rms_norm(x, x, wn.float(), 1e-4)
    torch.testing.assert_close(y2.float().cpu(), ref, **tol)
    assert torch.equal(res.cpu(), s)
    # feed-forward
    ff = SwiGLU(72, 100)
    gu = (torch.randn(200, 72, generator=g) * 0.1).to(dtype)
    dn = (torch.randn(72, 100, generator=g) * 0.1).to(dtype)
    ff.bind({"gate_up.weight": gu.cuda(), "down.weight": dn.cuda()})
    assert set(ff.param_specs()) == {"gate_up.weight", "down.weight"}
    torch.testing.assert_close(ff.forward(x.cuda(), None).float().cpu(),
                               plain.swiglu(x.float(), gu[:100].float(), gu[100:].float(), dn.float()), **tol)
    # position encoding: its table holds the plain angles
    rope = RotaryEmbedding(rotary_dim=24, max_position=50, base=500.0)
    ang = plain.rope_angles(torch.arange(50), 24, 500.0)
    torch.testing.assert_close(rope.rotation_table(), torch.cat((ang.cos(), ang.sin()), -1))
