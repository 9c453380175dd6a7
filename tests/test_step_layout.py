"""The arrays that a step hands to the kernels: positions, slots, block tables, wanted rows and graph padding.
Checked position by position with plain loops (the reference builds the same arrays in
nanovllm/engine/model_runner.py:1406-1455 for prompts and :1516-1540 for single tokens)."""
import random

import numpy as np
import pytest

from nanohybrid_vlm_amd.cache.manager import OutOfPages
from nanohybrid_vlm_amd.engine.runner import ModelRunner, StepEntry


@pytest.fixture()
def runner(model_folders, emulated_kernels):
    return ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=40, num_state_slots=4)


def _unpack(arrays):
    input_ids, positions, token_req, cu, context_lens, state_slots, slot_mapping, bt = arrays
    return dict(input_ids=input_ids, positions=positions, token_req=token_req, cu=cu, context_lens=context_lens,
                state_slots=state_slots, slot_mapping=slot_mapping, bt=bt)


def test_every_token_lands_on_its_slot(runner):
    rng = random.Random(5)
    lengths = {"a": 0, "b": 0, "c": 0}
    tokens_of = {rid: [] for rid in lengths}
    slot_of_position = {rid: {} for rid in lengths}
    for step in range(12):
        live = rng.sample(sorted(lengths), rng.randint(1, 3))
        entries = []
        for rid in live:
            n = rng.choice([1, 1, 2, 3, 5, 9])
            toks = [rng.randrange(runner.vocab_size) for _ in range(n)]
            entries.append(StepEntry(rid, toks, [n - 1]))
        arrays, meta = runner._layout(entries)
        a = _unpack(arrays)
        row = 0
        for i, e in enumerate(entries):
            table = runner.cache.block_table(e.request_id)
            assert a["cu"][i] == row
            assert a["context_lens"][i] == lengths[e.request_id] + len(e.tokens)
            assert list(a["bt"][i, :len(table)]) == table and (a["bt"][i, len(table):] == -1).all()
            for j, tok in enumerate(e.tokens):
                p = lengths[e.request_id] + j
                assert a["input_ids"][row] == tok
                assert a["positions"][row] == p
                assert a["token_req"][row] == i
                assert a["slot_mapping"][row] == table[p // 4] * 4 + p % 4
                slot_of_position[e.request_id][p] = int(a["slot_mapping"][row])
                row += 1
            assert meta["rows"][i] == row - 1
            lengths[e.request_id] += len(e.tokens)
            tokens_of[e.request_id] += e.tokens
            runner.cache.commit(e.request_id, lengths[e.request_id])
        assert a["cu"][len(entries)] == row == meta["T"]
    # no slot is used by two positions, of one request or of two
    all_slots = [s for m in slot_of_position.values() for s in m.values()]
    assert len(set(all_slots)) == len(all_slots)


def test_padding_rows_store_nothing(runner):
    runner._layout([StepEntry("a", [1, 2, 3, 4, 5], [])])
    runner.cache.commit("a", 5)
    arrays, meta = runner._layout([StepEntry("a", [7], [0])], pad_to=4, table_width=6)
    a = _unpack(arrays)
    assert meta["B"] == 4 and meta["T"] == 4 and meta["rows"] == [0]
    assert a["bt"].shape == (4, 6)
    assert list(a["slot_mapping"][1:]) == [-1, -1, -1]              # nothing is stored for the padding
    # and they read one key on the spare page that no request is ever given, and work on the spare state row
    assert list(a["context_lens"][1:]) == [1, 1, 1] and (a["bt"][1:, 0] == runner.num_pages).all()
    assert runner.num_pages not in [p for r in runner.cache.requests.values() for t in r.tables for p in t]
    assert list(a["state_slots"][1:]) == [runner.num_state_slots] * 3
    assert a["positions"][0] == 5 and a["slot_mapping"][0] == runner.cache.block_table("a")[1] * 4 + 1


def test_bad_entries_are_refused(runner):
    with pytest.raises(ValueError, match="twice"):
        runner._layout([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(ValueError, match="at least one token"):
        runner._layout([StepEntry("a", [], [])])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        runner._layout([StepEntry("a", [runner.vocab_size], [])])
    with pytest.raises(ValueError, match="wanted place"):
        runner._layout([StepEntry("b", [1, 2], [2])])
    with pytest.raises(OutOfPages):
        runner._layout([StepEntry("c", [1] * 161, [])])
    runner.cache.check()
    assert "c" not in runner.cache                                 # all or nothing: not even admitted


def test_a_refused_step_takes_nothing_from_the_cache(runner):
    """Whatever is wrong with a later entry, the earlier ones are not admitted and hold no page."""
    runner._layout([StepEntry("old", [1, 2, 3], [])])
    runner.cache.commit("old", 3)
    free, slots = runner.cache.num_free_pages(), runner.cache.num_free_slots()
    good = StepEntry("new", [1] * 9, [8])
    for bad, error in [(StepEntry("x", [runner.vocab_size + 3], []), ValueError),
                       (StepEntry("x", [1, 2], [5]), ValueError),
                       (StepEntry("x", [1] * (runner.max_position + 1), []), ValueError),
                       (StepEntry("x", [1] * 4 * (free + 1), []), OutOfPages),
                       (StepEntry("new", [4], []), ValueError)]:
        with pytest.raises(error):
            runner._layout([good, StepEntry("old", [7], [0]), bad])
        runner.cache.check()
        assert "new" not in runner.cache and "x" not in runner.cache
        assert runner.cache.num_free_pages() == free and runner.cache.num_free_slots() == slots
        assert runner.cache.num_tokens("old") == 3 and len(runner.cache.block_table("old")) == 1
    with pytest.raises(ValueError, match="max_model_len"):
        runner._layout([good, StepEntry("old", [7], [0])], table_width=2)
    assert "new" not in runner.cache and runner.cache.num_free_pages() == free


def test_graph_buckets_are_powers_of_two_and_the_sizes_half_way_up_to_the_limit(emulated_kernels, model_folders):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    for limit, want in [(64, [1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64]), (16, [1, 2, 3, 4, 6, 8, 12, 16]),
                        (20, [1, 2, 3, 4, 6, 8, 12, 16, 20]), (1, [1])]:
        runner = ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=8, num_state_slots=2,
                             max_graph_batch=limit)
        assert runner.graph_buckets == want


def test_a_recorded_short_step_is_strictly_smaller_than_its_bucket(model_folders, emulated_kernels, tmp_path):
    """A short step of prompt portions is padded to a bucket of tokens by one more request that owns the filling
    tokens. The bucket is strictly larger than the step, so that request has at least one token, and every request
    of the padded batch, also the ones without tokens, has its first row inside the batch: a part that works from the
    step's device tensors may index rows by ``cu_seqlens_q[:-1]`` (the toy's state mixer does)."""
    import torch
    import toy_architecture as toy
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    runner = ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=40, num_state_slots=4)
    runner.use_graphs, runner.max_graph_tokens, runner.mixed_token_buckets = True, 24, [16, 24]
    met = []
    runner._mixed_graph_step = lambda entries, key, keep=True: met.append(key)
    runner.step([StepEntry("a", list(range(15)), [14])])
    runner.step([StepEntry("b", list(range(16)), [15])])                      # fills the bucket of 16: goes to 24
    assert met == [(16, 1), (24, 1)]
    assert runner.step([StepEntry("c", list(range(24)), [23])]).shape == (1, runner.vocab_size)   # no bucket above: eager
    # the layout of such a step, and the toy's state mixer on it
    toy.register()
    try:
        folder = write_random_model(str(tmp_path / "toy"), {"architectures": ["ToyForCausalLM"], "model_type": "toy",
                                                            "device_state": True}, seed=4)
        runner = ModelRunner(folder, dtype="float32", device="cpu", page_size=4, num_pages=40, num_state_slots=4)
        entries = [StepEntry("a", list(range(9)), [8]), StepEntry("b", list(range(6)), [])]
        arrays, meta = runner._layout(entries, pad_to=4, table_width=16, pad_tokens_to=16)
        cu = arrays[3]
        assert meta["T"] == 16 and meta["B"] == 5 and list(cu) == [0, 9, 15, 15, 15, 16]
        assert (cu[:-1] < meta["T"]).all()
        dev = [torch.from_numpy(a) for a in arrays]
        ctx = runner._context(dev, meta, None, 0, max_context_len=64)
        assert ctx.positions.shape == (toy.AXES, 16) and ctx.token_positions.shape == (16,)
        runner.model.forward(ctx)                                              # (no row index runs out of the batch)
    finally:
        toy.unregister()


def test_positions_of_several_axes(model_folders, emulated_kernels, tmp_path):
    """A model of one position axis carries no array of positions unless an entry brings its own; a model of two
    axes always carries [2, T]: the tokens' indices on both axes, or what the entry says."""
    import toy_architecture as toy
    from nanohybrid_vlm_amd.weights.random_init import write_random_model
    runner = ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=40, num_state_slots=4)
    arrays, _ = runner._layout([StepEntry("a", [1, 2, 3], [])])
    assert len(arrays) == 8
    runner.cache.commit("a", 3)
    arrays, _ = runner._layout([StepEntry("a", [4, 5], [], positions=[[9, 11]]), StepEntry("b", [6], [])])
    assert len(arrays) == 9 and arrays[8].tolist() == [[9, 11, 0]] and arrays[1].tolist() == [3, 4, 0]
    with pytest.raises(ValueError, match=r"positions must be \[1\]\[2\]"):
        runner._layout([StepEntry("c", [4, 5], [], positions=[[1, 2], [3, 4]])])
    with pytest.raises(ValueError, match="outside the model's"):
        runner._layout([StepEntry("c", [4, 5], [], positions=[[1, runner.max_position]])])
    toy.register()
    try:
        folder = write_random_model(str(tmp_path / "toy"), {"architectures": ["ToyForCausalLM"], "model_type": "toy"}, seed=4)
        runner = ModelRunner(folder, dtype="float32", device="cpu", page_size=4, num_pages=40, num_state_slots=4)
        arrays, _ = runner._layout([StepEntry("a", [1, 2, 3], [])])
        assert arrays[-1].tolist() == [[0, 1, 2], [0, 1, 2]]
        runner.cache.commit("a", 3)
        arrays, _ = runner._layout([StepEntry("a", [4], [0], positions=[[3], [7]]), StepEntry("b", [5], [0])], pad_to=4, table_width=8)
        assert arrays[-1].tolist() == [[3, 0, 0, 0], [7, 0, 0, 0]]
    finally:
        toy.unregister()
