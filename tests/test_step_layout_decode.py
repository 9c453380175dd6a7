"""The short way of laying out a step of single tokens gives the arrays of the general way."""
import random

import numpy as np

from nanohybrid_vlm_amd.engine.runner import ModelRunner, StepEntry


def test_single_token_layout_equals_the_general_one(model_folders, emulated_kernels):
    rng = random.Random(3)
    for pad_to, width in [(None, None), (8, 40), (16, 64)]:
        runners = [ModelRunner(model_folders["A"], dtype="float32", device="cpu", page_size=4, num_pages=200,
                               num_state_slots=16) for _ in range(2)]
        lengths = [rng.randint(1, 60) for _ in range(6)]
        for r in runners:
            for i, n in enumerate(lengths):
                r._layout([StepEntry(i, [1] * n, [])])
                r.cache.commit(i, n)
        entries = [StepEntry(i, [3 + i], [0] if i % 2 else []) for i in (4, 0, 5, 2)]
        fast_arrays, fast_meta = runners[0]._layout_single_tokens(entries, pad_to, width)
        slow_arrays, slow_meta = runners[1]._layout_general(entries, pad_to, width)
        assert len(fast_arrays) == len(slow_arrays)
        for a, b in zip(fast_arrays, slow_arrays):
            assert a.dtype == b.dtype == np.int32 and a.shape == b.shape and (a == b).all()
        assert fast_meta == slow_meta
        for r in runners:
            r.cache.check()
