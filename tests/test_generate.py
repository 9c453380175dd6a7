"""Generation through the entry point: greedy and seeded temperature sampling against
the plain implementation, with prompts cut to a small token budget, with so few
pages that requests are pushed out and computed again, and with late arrivals."""
import pytest
import torch

import plain_qwen3 as plain
from conftest import TINY
from nanohybrid_vlm_amd import LLM, SamplingParams
from nanohybrid_vlm_amd.sampling.sampler import noise_key
from replay_cases import random_tokens


def _plain_generate(cfg, w, prompt, sp: SamplingParams, request: int, engine_seed: int, eos):
    ids, out = list(prompt), []
    for step in range(sp.max_tokens):
        row = plain.logits(cfg, w, ids)[-1]
        if sp.temperature == 0:
            t = plain.sample_token(row, 0.0, None)
        else:
            seed = engine_seed if sp.seed is None else sp.seed
            t = plain.sample_token(row, sp.temperature, plain.sample_noise(seed, request, step, row.numel()))
        ids.append(t)
        out.append(t)
        if not sp.ignore_eos and t == eos:
            break
    return out


def _workload(name):
    cfg, _ = TINY[name]
    lens = [5, 17, 33] if name == "A" else [1, 13, 40, 64]
    return [random_tokens(cfg["vocab_size"], n, 50 + n) for n in lens]


def _run(folder, device, dtype, name, **options):
    cfg, w = plain.read_model_folder(folder)
    prompts = _workload(name)
    greedy = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    llm = LLM(folder, device=device, dtype=dtype, **options)
    outs = llm.generate(prompts, greedy, use_tqdm=False)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert o["text"] is None
        assert o["token_ids"] == _plain_generate(cfg, w, p, greedy, i, 0, cfg.get("eos_token_id")), f"greedy, prompt {i}"
    # temperature sampling with the engine's counter-based noise, one request with a seed of its own; ends at eos
    params = [SamplingParams(temperature=0.8, max_tokens=12, seed=None if i % 2 else 1000 + i) for i in range(len(prompts))]
    outs = llm.generate(prompts, params, use_tqdm=False)
    for i, (p, sp, o) in enumerate(zip(prompts, params, outs)):
        # request ids go on counting: the second batch has ids len(prompts)..
        want = _plain_generate(cfg, w, p, sp, len(prompts) + i, llm.config.seed, llm.config.eos)
        assert o["token_ids"] == want, f"temperature, prompt {i}"
    metrics = llm.get_completed_request_metrics()
    assert len(metrics) == 2 * len(prompts) and all(m.ttft_ms >= 0 and m.e2e_ms >= m.ttft_ms for m in metrics)
    stats = llm.get_memory_stats()
    assert stats["weight_bytes"] > 0 and stats["kv_cache_bytes"] > 0 and stats["live_requests"] == 0
    assert stats["groups"][0]["free_pages"] == stats["groups"][0]["pages"]
    return llm


@pytest.mark.parametrize("name,options", [
    ("A", dict(kvcache_block_size=4, num_kvcache_blocks=64)),
    ("B", dict(kvcache_block_size=8, num_kvcache_blocks=64, max_num_batched_tokens=7)),        # prompts in portions of 7
    ("B", dict(kvcache_block_size=8, num_kvcache_blocks=13, max_num_batched_tokens=16, max_num_seqs=3)),  # pages run out
])
def test_generate_on_emulated_kernels(model_folders, emulated_kernels, name, options):
    llm = _run(model_folders[name], "cpu", "float32", name, **options)
    if options["num_kvcache_blocks"] == 13:
        assert llm.scheduler.num_preemptions > 0, "the small cache was meant to force a request out"


@pytest.mark.gpu
@pytest.mark.parametrize("name,options", [
    ("A", dict(kvcache_block_size=4, num_kvcache_blocks=64)),
    ("B", dict(kvcache_block_size=8, num_kvcache_blocks=64, max_num_batched_tokens=7)),
    ("B", dict(kvcache_block_size=8, num_kvcache_blocks=13, max_num_batched_tokens=16, max_num_seqs=3)),
])
def test_generate_float32_on_gpu(model_folders, name, options):
    _run(model_folders[name], "cuda:0", "float32", name, **options)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["A", "B"])
def test_generate_bfloat16_on_gpu(model_folders, name):
    """bfloat16 may choose the other of two nearly equal logits. Every chosen token is (nearly) the best of the
    engine's own logits for its place, taken again afterwards with the whole sequence in one step through the same
    runner (what may differ between that step and the step that chose the token is the order of sums: a hundredth of
    the logits' deviation), and one that the plain implementation rates within bfloat16's rounding of its best."""
    import replay_cases as rc
    from helpers import tolerance_for
    folder = model_folders[name]
    cfg, w = plain.read_model_folder(folder)
    prompts = _workload(name)
    llm = LLM(folder, dtype="bfloat16", kvcache_block_size=8, num_kvcache_blocks=64, max_num_batched_tokens=16)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
    sequences = {f"s{i}": list(p) + list(o["token_ids"]) for i, (p, o) in enumerate(zip(prompts, outs))}
    own = rc.run_in_process(llm.runner, rc.whole(sequences))
    worst_own = worst_plain = 0.0
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o["token_ids"]) == 8
        rows = plain.logits(cfg, w, sequences[f"s{i}"])
        tol = tolerance_for("bfloat16", rows)
        for j, t in enumerate(o["token_ids"]):
            at = len(p) - 1 + j
            mine, theirs = own[f"s{i}"][at], rows[at]
            worst_own = max(worst_own, (mine.max() - mine[t]).item())
            worst_plain = max(worst_plain, (theirs.max() - theirs[t]).item())
            assert mine[t] >= mine.max() - 0.1 * tol, f"prompt {i}, token {j}: not the best of the engine's own logits"
            assert theirs[t] >= theirs.max() - tol, f"prompt {i}, token {j}: a token far from the plain implementation's best"
    print(f"furthest from the best: {worst_own:.2e} of the engine's own logits, {worst_plain:.2e} of the plain ones")


def _shared_start_run(folder, device, dtype, name, **options):
    """Prompts with the same first tokens, in a cache so small that requests are pushed out and come back: with
    the prefix cache on, the tokens are those of the plain implementation and fewer of them are computed."""
    cfg, w = plain.read_model_folder(folder)
    start = random_tokens(cfg["vocab_size"], 21, 7)
    prompts = [start + random_tokens(cfg["vocab_size"], n, 70 + n) for n in (1, 6, 12, 3)] + [start[:17]]
    greedy = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    # a budget of 24 tokens a step: the first prompt and the start of the second run before any page is known
    llm = LLM(folder, device=device, dtype=dtype, enable_prefix_cache=True, kvcache_block_size=8,
              max_num_batched_tokens=24, **options)
    outs = llm.generate(prompts, greedy, use_tqdm=False)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert o["token_ids"] == _plain_generate(cfg, w, p, greedy, i, 0, cfg.get("eos_token_id")), f"prompt {i}"
    llm.runner.cache.check()
    assert llm.runner.cache.num_shared_tokens >= 16 * (len(prompts) - 2)
    return llm


@pytest.mark.parametrize("options", [dict(num_kvcache_blocks=64), dict(num_kvcache_blocks=11, max_num_seqs=3)])
def test_prefix_cache_on_emulated_kernels(model_folders, emulated_kernels, options):
    llm = _shared_start_run(model_folders["B"], "cpu", "float32", "B", **options)
    if options["num_kvcache_blocks"] == 11:
        assert llm.scheduler.num_preemptions > 0


@pytest.mark.gpu
@pytest.mark.parametrize("options", [dict(num_kvcache_blocks=64), dict(num_kvcache_blocks=11, max_num_seqs=3),
                                     dict(num_kvcache_blocks=64, enforce_eager=True)])
def test_prefix_cache_on_gpu(model_folders, options):
    _shared_start_run(model_folders["B"], "cuda:0", "float32", "B", **options)


def test_prefix_cache_refusals(model_folders, emulated_kernels):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    with pytest.raises(ValueError, match="poison_freed_pages would destroy"):
        ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=8, num_state_slots=2,
                    share_prefixes=True, poison_freed_pages=True)


def test_late_arrivals_and_step_by_hand(model_folders, emulated_kernels):
    """Requests added while others decode (nanovllm's tests drive llm.step() the same way,
    tests/5090-test-TP2/run_generation.py:62-134)."""
    folder = model_folders["A"]
    cfg, w = plain.read_model_folder(folder)
    llm = LLM(folder, device="cpu", dtype="float32", kvcache_block_size=4, num_kvcache_blocks=64, max_num_batched_tokens=12)
    sp = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
    first = [random_tokens(256, n, n) for n in (6, 9)]
    late = [random_tokens(256, n, n) for n in (30, 21)]
    ids = [llm.add_request(p, sp) for p in first]
    done, mixed_steps = {}, 0
    for _ in range(3):
        out, _ = llm.step()
    ids += [llm.add_request(p, sp) for p in late]
    while not llm.is_finished():
        out, stats = llm.step()
        mixed_steps += bool(stats.num_decode_tokens and stats.num_prefill_tokens)
        done.update(dict(out))
    assert mixed_steps >= 2, "decoded tokens and prompt portions ran in one batch"
    for i, p in zip(ids, first + late):
        assert done[i] == plain.greedy_generate(cfg, w, p, 10)


def test_entry_point_refusals(model_folders, emulated_kernels):
    folder = model_folders["A"]
    with pytest.raises(TypeError, match="unknown engine options"):
        LLM(folder, device="cpu", tensor_parallel_size=2)
    with pytest.raises(FileNotFoundError):
        LLM(folder + "_nowhere", device="cpu")
    llm = LLM(folder, device="cpu", dtype="float32", kvcache_block_size=4, num_kvcache_blocks=8, max_model_len=64)
    assert llm.config.eos == 3 and llm.config.max_model_len == 64
    for bad, err in [([], ValueError), ([1, -2], ValueError), ([1, True], TypeError), ("text", ValueError),
                     ([1, 999], ValueError), ((1, 2), TypeError)]:
        with pytest.raises(err):
            llm.add_request(bad, SamplingParams())
    with pytest.raises(ValueError, match="max_model_len"):
        llm.add_request([1] * 60, SamplingParams(max_tokens=10))
    with pytest.raises(ValueError):
        SamplingParams(temperature=-1)
    with pytest.raises(ValueError):
        SamplingParams(temperature=float("nan"))


@pytest.mark.gpu
def test_steps_issued_ahead_change_no_token(model_folders):
    """A decoding step that is bound to follow is issued before the host knows the tokens it feeds (they go from
    the sampling kernel to the next step on the device). Whatever ends a request meanwhile (an end-of-sequence
    token, its max_tokens), whoever arrives late, and however few pages there are: the tokens are those of the
    plain implementation, with steps issued ahead and without."""
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    V = cfg["vocab_size"]
    prompts = [random_tokens(V, n, 90 + n) for n in (3, 9, 20, 31, 40, 2)]
    greedy = SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True)
    # an end-of-sequence token that greedy decoding of the first prompt meets on its way
    eos = _plain_generate(cfg, w, prompts[0], greedy, 0, 0, None)[6]
    params = [SamplingParams(temperature=0.0, max_tokens=24), SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True),
              SamplingParams(temperature=0.9, max_tokens=20, seed=5), SamplingParams(temperature=0.0, max_tokens=1),
              SamplingParams(temperature=0.0, max_tokens=2), SamplingParams(temperature=0.7, max_tokens=17)]
    want = [_plain_generate(cfg, w, p, sp, i, 0, eos) for i, (p, sp) in enumerate(zip(prompts, params))]
    assert len(want[0]) < 24, "the first request was meant to end at the end-of-sequence token"
    for pages in (64, 14):                                  # ample, and so few that requests are pushed out
        ahead_steps = {}
        for run_ahead in (False, True):
            llm = LLM(folder, dtype="float32", kvcache_block_size=8, num_kvcache_blocks=pages, max_num_batched_tokens=16,
                      eos=eos, run_ahead=run_ahead)
            done = {}
            for p, sp in zip(prompts[:3], params[:3]):
                llm.add_request(p, sp)
            for _ in range(9):                              # the others arrive while the first three decode
                done.update(llm.step()[0])
            for p, sp in zip(prompts[3:], params[3:]):
                llm.add_request(p, sp)
            while not llm.is_finished():
                done.update(llm.step()[0])
            assert [done[i] for i in range(len(prompts))] == want, f"run_ahead={run_ahead}, {pages} pages"
            llm.runner.cache.check()
            assert llm.get_memory_stats()["groups"][0]["free_pages"] == pages
            ahead_steps[run_ahead] = llm.num_steps_ahead
            if pages == 14:
                assert llm.scheduler.num_preemptions > 0, "the small cache was meant to force a request out"
        assert ahead_steps[False] == 0 and ahead_steps[True] >= 10


def _near_best(cfg, w, prompt, tokens, slack=2e-2):
    """Every generated token is one the plain implementation rates within ``slack`` of its best, given the tokens
    before it (bfloat16 may choose the other of two nearly equal logits; from there on the run is its own)."""
    ids = list(prompt)
    for t in tokens:
        row = plain.logits(cfg, w, ids)[-1]
        assert row[t] >= row.max() - slack, "a token far from the best was chosen"
        ids.append(t)


@pytest.mark.gpu
def test_steps_issued_ahead_and_recomputation_in_bfloat16(model_folders):
    """In bfloat16 a recorded step may hold the library's matrix products: the tokens with steps issued ahead are
    bit for bit those without (the same recorded steps run either way), with ample pages and with so few that
    requests are pushed out and computed again; and every token is one the plain implementation rates best or
    nearly so."""
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    V = cfg["vocab_size"]
    prompts = [random_tokens(V, n, 190 + n) for n in (3, 9, 20, 31, 40, 2)]
    params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in (24, 30, 20, 1, 2, 17)]
    for pages in (64, 14):
        runs = {}
        for run_ahead in (False, True):
            llm = LLM(folder, dtype="bfloat16", kvcache_block_size=8, num_kvcache_blocks=pages, max_num_batched_tokens=16,
                      run_ahead=run_ahead)
            done = {}
            for p, sp in zip(prompts[:3], params[:3]):
                llm.add_request(p, sp)
            for _ in range(9):
                done.update(llm.step()[0])
            for p, sp in zip(prompts[3:], params[3:]):
                llm.add_request(p, sp)
            while not llm.is_finished():
                done.update(llm.step()[0])
            runs[run_ahead] = [done[i] for i in range(len(prompts))]
            llm.runner.cache.check()
            assert llm.get_memory_stats()["groups"][0]["free_pages"] == pages
            assert (llm.num_steps_ahead >= 10) == run_ahead
            if pages == 14:
                assert llm.scheduler.num_preemptions > 0, "the small cache was meant to force a request out"
        assert runs[True] == runs[False], f"{pages} pages: steps issued ahead changed a token"
        for p, sp, tokens in zip(prompts, params, runs[True]):
            assert len(tokens) == sp.max_tokens
            _near_best(cfg, w, p, tokens)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cache_sized_from_free_memory(model_folders, dtype):
    """``num_kvcache_blocks=-1`` (the default): the pages are what is left of ``gpu_memory_utilization`` of the
    device's memory after the weights, the state pools, a step's activations and the recorded steps
    (nanovllm/engine/model_runner.py:654-699). The device then holds no more than that share, and generation
    is right."""
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    import gc
    gc.collect()
    torch.cuda.empty_cache()                     # (what earlier tests left in the allocator's reserve goes back: the sizing does the same)
    free_before, total = torch.cuda.mem_get_info()
    share = min(0.9, (total - free_before) / total + 0.04)           # what is in use already and 4 % of the device more
    llm = LLM(folder, dtype=dtype, kvcache_block_size=256, gpu_memory_utilization=share, max_num_batched_tokens=512,
              max_model_len=512)
    stats = llm.get_memory_stats()
    pages = stats["groups"][0]["pages"]
    assert llm.config.num_kvcache_blocks == pages > 0
    item = 4 if dtype == "float32" else 2
    page_bytes = 2 * 256 * cfg["num_key_value_heads"] * cfg["head_dim"] * item * cfg["num_hidden_layers"]
    assert stats["kv_cache_bytes"] == pages * page_bytes
    # most of the 4 % went to pages, and the device's share is kept
    assert 0.5 * 0.04 * total <= stats["kv_cache_bytes"] <= 0.04 * total
    assert total - stats["device_free_bytes"] <= share * total
    prompts = [random_tokens(cfg["vocab_size"], n, 300 + n) for n in (300, 5, 260)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True), use_tqdm=False)
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o["token_ids"] == plain.greedy_generate(cfg, w, p, 6)
        else:
            _near_best(cfg, w, p, o["token_ids"])
    assert total - torch.cuda.mem_get_info()[0] <= share * total + (256 << 20), "generation stayed within the share (and the allocator's slack)"
    # what the sizing set aside was measured: after every size of step has been recorded and a step of the whole
    # token budget (every request wanting logits) has run, the device still holds no more than its share
    probe = stats["cache_sizing_probe"]
    assert probe["tokens"] == 512 and probe["activation_bytes"] > 0 and probe["graph_own_bytes"] > 0, probe
    recorded = llm.warm_up()
    assert 256 in recorded["graphs_recorded"] and len(recorded["mixed_graphs_recorded"]) >= 9, recorded
    from nanohybrid_vlm_amd.engine.runner import StepEntry
    ids = [("full", i) for i in range(min(pages, 300))]
    budget = [1] * (len(ids) - 1) + [512 - (len(ids) - 1)]
    llm.runner.step([StepEntry(r, [1] * n, [n - 1]) for r, n in zip(ids, budget)])
    for r in ids:
        llm.runner.finish(r)
    torch.cuda.synchronize()
    free_now = llm.get_memory_stats()["device_free_bytes"]
    assert free_now >= (1 - share) * total - (256 << 20), (free_now, (1 - share) * total)
    with pytest.raises(RuntimeError, match="no memory left for the cache"):
        LLM(folder, dtype=dtype, kvcache_block_size=256, gpu_memory_utilization=max(0.001, (total - free_before) / total * 0.5))


def test_a_configuration_with_random_weights_in_place_of_a_folder(emulated_kernels):
    """``LLM(config.json contents, random_weights=seed)``: a model of that configuration with weights drawn in
    place; the same seed gives the same model."""
    from conftest import TINY_B
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    options = dict(device="cpu", dtype="float32", kvcache_block_size=4, num_kvcache_blocks=32, max_model_len=64)
    runs = [LLM(dict(TINY_B), random_weights=seed, **options).generate([[5, 17, 3], [9, 200, 31, 7] * 3], sp, use_tqdm=False)
            for seed in (3, 3, 4)]
    assert runs[0] == runs[1] and runs[0] != runs[2]
    assert LLM(dict(TINY_B), random_weights=3, **options).config.eos == TINY_B["eos_token_id"]
    with pytest.raises(TypeError, match="needs random_weights"):
        LLM(dict(TINY_B), **options)
    with pytest.raises(TypeError, match="goes with a configuration"):
        LLM("some folder", random_weights=1, **options)
    with pytest.raises(ValueError, match="dtype"):
        LLM(dict(TINY_B), random_weights=1, device="cpu", dtype="float16")


@pytest.mark.gpu
def test_pinned_gemm_choices_make_bfloat16_runs_repeat_bit_for_bit(model_folders, tmp_path):
    """Which kernel does a bfloat16 matrix product (own, or one of the library's algorithms) is normally decided by
    a timing, once per shape and process. With ``measure_gemms=False`` nothing is timed and every shape follows the
    fixed rule; with ``gemm_choices=FILE`` a run does every product the way an earlier run chose. Either way two
    engines give the same logits bit for bit."""
    import json
    from nanohybrid_vlm_amd.engine.runner import StepEntry
    from nanohybrid_vlm_amd.native import ops
    folder = model_folders["D"]
    cfg, _ = plain.read_model_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 700 + n) for n in (40, 3, 100, 17, 9, 64, 30, 5, 12, 21)]
    options = dict(dtype="bfloat16", kvcache_block_size=64, num_kvcache_blocks=64, max_num_batched_tokens=256, max_model_len=256)

    def logits_of(llm):
        """Prompt portions of many rows, then single tokens of ten requests through a recorded step."""
        runner = llm.runner
        first = runner.step([StepEntry(("probe", i), p, [len(p) - 1]) for i, p in enumerate(prompts)])
        second = runner.step([StepEntry(("probe", i), [7 + i], [0]) for i in range(len(prompts))])
        third = runner.step([StepEntry(("probe", i), [9 + i], [0]) for i in range(len(prompts))])
        for i in range(len(prompts)):
            runner.finish(("probe", i))
        return torch.cat([first, second, third]).cpu()

    backend = ops.backend()
    # nothing measured: the rule, twice
    runs = []
    for _ in range(2):
        backend.chosen.clear()
        llm = LLM(folder, measure_gemms=False, **options)
        runs.append(logits_of(llm))
        assert llm.gemm_choices() == {} and backend.chosen == {}
    assert torch.equal(runs[0], runs[1])
    # measured once, written down, followed by the next engine
    path = str(tmp_path / "choices.json")
    backend.chosen.clear()
    llm = LLM(folder, gemm_choices=path, **options)
    measured = logits_of(llm)
    table = llm.gemm_choices()
    assert table and all(len(k.split(",")) == 5 for k in table), "the recorded step's shapes were measured"
    assert llm.get_memory_stats()["gemm_choices"] == table
    llm.save_gemm_choices()
    assert json.load(open(path)) == table
    backend.chosen.clear()
    llm = LLM(folder, gemm_choices=path, **options)
    assert llm.gemm_choices() == table
    # a second engine of the same process, which measures and keeps the process-wide table, steps in between:
    # neither changes how the other's products are done
    other = LLM(folder, **options)
    assert other.runner.gemm_table is None and other.runner.measure_gemms
    logits_of(other)
    again = logits_of(llm)
    assert backend.measuring_allowed is False and backend.chosen is llm.runner.gemm_table
    assert llm.gemm_choices() == table, "nothing was measured in the second run"
    assert torch.equal(again, measured)
    logits_of(other)
    assert backend.measuring_allowed is True and backend.chosen is backend.shared_chosen
    # a table that names an algorithm the library does not have is refused when the engine starts
    bad = str(tmp_path / "bad.json")
    json.dump({"8,512,512,0,0": 100000}, open(bad, "w"))
    with pytest.raises(Exception, match="algorithms for this shape"):
        LLM(folder, gemm_choices=bad, **options)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_up_records_the_graphs_ahead(model_folders, dtype):
    """With ``warm_up`` every size of step that replays a graph is met once when the engine starts: the graphs are
    there before the first request, nothing stays in the cache, and generation gives the plain tokens."""
    folder = model_folders["B"]
    cfg, w = plain.read_model_folder(folder)
    llm = LLM(folder, dtype=dtype, kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=8, max_graph_tokens=64,
              max_num_batched_tokens=64, warm_up=True)
    stats = llm.get_memory_stats()
    assert stats["graphs_recorded"] == [1, 2, 3, 4, 6, 8] and stats["graphs_refused"] == []
    assert stats["mixed_graphs_recorded"] == [(16, 1), (24, 1), (32, 1), (48, 1), (64, 1)] and stats["mixed_graphs_refused"] == []
    assert stats["live_requests"] == 0 and stats["groups"][0]["free_pages"] == 40
    llm.runner.cache.check()
    if dtype == "float32":
        prompts = [random_tokens(cfg["vocab_size"], n, 300 + n) for n in (5, 30, 47, 12)]
        sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
        out = llm.generate(prompts, sp)
        assert [o["token_ids"] for o in out] == [plain.greedy_generate(cfg, w, p, 6) for p in prompts]
    # asked for again, and with requests under way, it does nothing
    assert llm.warm_up(batch_sizes=[1], token_counts=[16])["graphs_recorded"] == [1, 2, 3, 4, 6, 8]


def _stress(folder, device, seed, options):
    """Requests of random lengths arrive a few at a time while others decode, with so few pages that some are
    pushed out and computed again; every request's tokens must be the plain implementation's."""
    import random
    rnd_ = random.Random(seed)
    cfg, w = plain.read_model_folder(folder)
    V = cfg["vocab_size"]
    requests = [(random_tokens(V, rnd_.randint(1, 70), 1000 * seed + i), rnd_.randint(1, 18)) for i in range(36)]
    llm = LLM(folder, dtype="float32", device=device, kvcache_block_size=8, num_kvcache_blocks=rnd_.choice([28, 40, 90]),
              max_num_batched_tokens=rnd_.choice([16, 48, 96]), max_num_seqs=rnd_.choice([4, 9, 36]),
              max_model_len=96, max_prefill_wait_ms=rnd_.choice([0.0, 1e9]),
              scheduler_policy=rnd_.choice(["decode_first", "prefill_first"]), poison_freed_pages=True, **options)
    # every slot of the cache that no live request owns holds NaN: all of them now, later every page that a finished
    # or pushed-out request gives back (the scheduler's releases go through the runner)
    for kv in llm.runner.kv_tensors:
        kv.fill_(float("nan"))
    ids, done, waiting = {}, {}, list(enumerate(requests))
    while waiting or not llm.is_finished():
        for _ in range(rnd_.randint(0, 3)):
            if waiting:
                i, (prompt, n) = waiting.pop(0)
                ids[llm.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True))] = i
        if not llm.is_finished():
            done.update(llm.step()[0])
    got = {ids[sid]: toks for sid, toks in done.items()}
    for i, (prompt, n) in enumerate(requests):
        assert got[i] == plain.greedy_generate(cfg, w, prompt, n), f"seed {seed}: request {i}"
    stats = llm.get_memory_stats()
    assert stats["live_requests"] == 0 and stats["groups"][0]["free_pages"] == stats["groups"][0]["pages"]
    llm.runner.cache.check()
    return llm, stats


@pytest.mark.parametrize("seed", range(3))
def test_engine_under_random_arrivals_on_emulated_kernels(model_folders, emulated_kernels, seed):
    _stress(model_folders["B"], "cpu", seed, {})


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(6))
def test_engine_under_random_arrivals_on_gpu(model_folders, seed):
    """The same with recorded steps of both kinds (single tokens; short steps of any make) and steps issued ahead."""
    llm, stats = _stress(model_folders["B"], "cuda:0", seed, dict(max_graph_tokens=64))
    assert not stats["graphs_refused"] and not stats["mixed_graphs_refused"]
    assert stats["graphs_recorded"] and stats["mixed_graphs_recorded"], stats


def test_end_token_from_the_tokenizer_and_text_prompts(emulated_kernels, tmp_path):
    """A model folder whose config.json names no end token ends requests where its tokenizer does
    (nanovllm/engine/llm_engine.py:207-223); with a tokenizer.json a prompt may be text and the answer comes as text too."""
    import json
    from conftest import TINY_C
    from tokenizers import Tokenizer, models, pre_tokenizers
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    folder = write_random_model(str(tmp_path / "m"), TINY_C, seed=2)
    assert "eos_token_id" not in TINY_C
    vocab = {f"w{i}": i for i in range(TINY_C["vocab_size"] - 1)}
    vocab["<end>"] = TINY_C["vocab_size"] - 1
    tok = Tokenizer(models.WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(str(tmp_path / "m" / "tokenizer.json"))
    options = dict(dtype="float32", device="cpu", kvcache_block_size=8, num_kvcache_blocks=16, max_model_len=64)
    assert LLM(folder, **options).config.eos == -1                   # a tokenizer alone does not say which token ends
    (tmp_path / "m" / "tokenizer_config.json").write_text(json.dumps({"eos_token": {"content": "<end>"}}))
    llm = LLM(folder, **options)
    assert llm.config.eos == TINY_C["vocab_size"] - 1
    out = llm.generate(["w5 w17 w3"], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True), use_tqdm=False)[0]
    cfg, w = plain.read_model_folder(folder)
    assert out["token_ids"] == plain.greedy_generate(cfg, w, [5, 17, 3], 4)
    assert out["text"] == tok.decode(out["token_ids"])
    (tmp_path / "m" / "tokenizer_config.json").write_text(json.dumps({"eos_token": "w9"}))
    assert LLM(folder, eos=4, **options).config.eos == 4              # an end token that the caller names stands
    assert LLM(folder, **options).config.eos == 9
