"""The scheduler's decisions, driven without a model: a stand-in "model" whose next
token is a function of all tokens so far, so that any schedule must give the same
completions."""
import pytest

from nanohybrid_vlm_amd.cache.manager import CacheManager, PagedGroupSpec
from nanohybrid_vlm_amd.engine.scheduler import Scheduler
from nanohybrid_vlm_amd.engine.sequence import Sequence, SequenceStatus
from nanohybrid_vlm_amd.sampling.params import SamplingParams

VOCAB, EOS = 50, 0


def next_token(tokens):
    return (sum(tokens) * 31 + len(tokens) * 7) % (VOCAB - 1) + 1        # never EOS unless forced


class Clock:
    def __init__(self):
        self.t = 0.0

    def __call__(self):
        return self.t


def make(pages=64, page=4, max_seqs=8, budget=16, policy="decode_first", wait_ms=50.0, slots=None, clock=None,
         max_model_len=4096, share_prefixes=False):
    cache = CacheManager([PagedGroupSpec("all", page, pages)], slots or max_seqs, share_prefixes=share_prefixes)
    return Scheduler(cache, max_seqs, budget, EOS, max_model_len, policy, wait_ms, clock or Clock())


def run(s, prompts, params, next_fn=next_token, max_steps=10000, on_step=None, late=None):
    """Runs to the end; returns completions by request id and the list of plans' summaries."""
    seqs = [Sequence(i, p, sp) for i, (p, sp) in enumerate(zip(prompts, params))]
    for q in seqs:
        s.add(q)
    log, done = [], {}
    late = dict(late or {})
    for step in range(max_steps):
        if step in late:
            q = late.pop(step)
            seqs.append(q)
            s.add(q)
        if s.is_finished():
            break
        plan = s.schedule()
        tokens = []
        for q in plan.seqs:
            n = q.num_scheduled_tokens
            assert n >= 1
            # what the runner does after the pass
            s.cache.commit(q.seq_id, q.num_cached_tokens + n, q.token_ids[q.num_cached_tokens:q.num_cached_tokens + n])
            ends = q.num_cached_tokens + n == q.num_tokens
            tokens.append(next_fn(q.token_ids) if ends else None)
        log.append({"decode": [q.seq_id for q in plan.decode_seqs],
                    "prefill": [(q.seq_id, q.num_scheduled_tokens) for q in plan.prefill_seqs],
                    "preempted": list(plan.preempted_seq_ids)})
        # budgets
        assert sum(q.num_scheduled_tokens for q in plan.seqs) <= s.max_num_batched_tokens
        assert len(plan.seqs) <= s.max_num_seqs
        unfinished = [q for q in plan.prefill_seqs if q.num_cached_tokens + q.num_scheduled_tokens < q.num_tokens]
        assert len(unfinished) <= 1, "at most one unfinished portion in a step"
        for q in s.postprocess(plan.seqs, tokens):
            done[q.seq_id] = q.completion_token_ids
        s.cache.check()
        if on_step:
            on_step(step, s)
    assert s.is_finished(), "did not finish"
    assert not s.cache.requests and s.cache.num_free_pages() == s.cache.groups[0].num_pages
    return done, log


def greedy(n=6):
    return SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)


def expected(prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = next_token(toks)
        toks.append(t)
        out.append(t)
    return out


def test_prompts_are_cut_to_the_budget_in_arrival_order():
    s = make(budget=7)
    prompts = [list(range(1, 21)), [5, 6, 7], [9] * 9]
    done, log = run(s, prompts, [greedy(3)] * 3)
    assert log[0]["prefill"] == [(0, 7)] and log[1]["prefill"] == [(0, 7)]
    assert log[2]["prefill"] == [(0, 6), (1, 1)]              # the rest of the budget goes to the next in line
    assert log[3]["decode"] == [0] and log[3]["prefill"] == [(1, 2), (2, 4)]
    for i, p in enumerate(prompts):
        assert done[i] == expected(p, 3)


def test_decode_first_and_prefill_first():
    prompts = [[1, 2, 3], [4, 5, 6, 7]]
    late = lambda: {2: Sequence(2, [8] * 10, greedy(2))}
    _, log = run(make(budget=8, policy="decode_first"), prompts, [greedy(6)] * 2, late=late())
    assert log[2]["decode"] == [0, 1] and log[2]["prefill"] == [(2, 6)]     # decodes keep going beside the new prompt
    _, log = run(make(budget=8, policy="prefill_first"), prompts, [greedy(6)] * 2, late=late())
    assert log[2]["decode"] == [] and log[2]["prefill"] == [(2, 8)]         # while a prompt waits nothing decodes
    assert log[3]["decode"] == [] and log[3]["prefill"] == [(2, 2)]
    assert log[4]["decode"] == [0, 1, 2]


def test_endings():
    s = make()
    eos_at_third = lambda toks: EOS if len(toks) == 5 else next_token(toks)
    done, _ = run(s, [[1, 2, 3], [1, 2, 3], [1, 2, 3]],
                  [SamplingParams(0.0, 10, False), SamplingParams(0.0, 10, True), SamplingParams(0.0, 2, False)],
                  next_fn=eos_at_third)
    assert done[0][-1] == EOS and len(done[0]) == 3          # the end token is kept and ends the request
    assert len(done[1]) == 10 and done[1][2] == EOS          # ignore_eos runs to max_tokens
    assert len(done[2]) == 2                                 # max_tokens first


def test_when_pages_run_out_the_cheapest_request_is_computed_again():
    # 3 requests of 6 tokens need 2 pages each at first (page 4); decoding to 12 tokens needs 3 each; only 7 pages
    prompts = [[1, 2, 3, 4, 5, 6], [7, 8, 9, 10, 11, 12], [13, 14, 15, 16, 17, 18]]
    s = make(pages=7, page=4, budget=32)
    done, log = run(s, prompts, [greedy(7)] * 3)
    assert s.num_preemptions >= 1 and s.num_recomputed_tokens > 0
    first = next(l for l in log if l["preempted"])
    assert first["preempted"] == [0] or len(first["preempted"]) >= 1
    ample, _ = run(make(pages=64, page=4, budget=32), prompts, [greedy(7)] * 3)
    assert done == ample == {i: expected(p, 7) for i, p in enumerate(prompts)}


def test_victim_is_the_running_request_with_fewest_cached_tokens():
    s = make(pages=5, page=4, budget=32)
    a, b = Sequence(0, list(range(1, 9)), greedy(8)), Sequence(1, [1, 2, 3, 4], greedy(8))
    s.add(a); s.add(b)
    plan = s.schedule()                                    # both prompts: 2 + 1 pages
    for q in plan.seqs:
        s.cache.commit(q.seq_id, q.num_tokens)
    s.postprocess(plan.seqs, [next_token(q.token_ids) for q in plan.seqs])
    plan = s.schedule()                                    # a needs page 3 (9 tokens), b needs page 2 (5 tokens): 5 pages, fine
    assert [q.seq_id for q in plan.decode_seqs] == [0, 1] and not plan.preempted_seq_ids
    for q in plan.seqs:
        s.cache.commit(q.seq_id, q.num_tokens)
    s.postprocess(plan.seqs, [next_token(q.token_ids) for q in plan.seqs])
    for _ in range(3):                                     # a: 10, 11, 12 tokens cached; b: 6, 7, 8
        plan = s.schedule()
        assert not plan.preempted_seq_ids
        for q in plan.seqs:
            s.cache.commit(q.seq_id, q.num_tokens)
        s.postprocess(plan.seqs, [next_token(q.token_ids) for q in plan.seqs])
    plan = s.schedule()                                    # a needs a 4th page: none free -> b (fewer cached tokens) goes
    assert plan.preempted_seq_ids == [1]
    assert b.status == SequenceStatus.WAITING and b.num_cached_tokens == 0 and 1 not in s.cache
    assert [q.seq_id for q in plan.decode_seqs] == [0]
    assert s.waiting[0] is b and b.num_tokens == 4 + 5     # its generated tokens are kept and fed again


def test_a_lone_request_that_cannot_grow_preempts_itself_and_an_impossible_one_is_refused():
    s = make(pages=2, page=4)
    with pytest.raises(ValueError, match="pages"):
        s.add(Sequence(0, [1] * 6, greedy(6)))             # up to 12 tokens = 3 pages > 2
    with pytest.raises(ValueError, match="max_model_len"):
        make(max_model_len=8).add(Sequence(0, [1] * 6, greedy(6)))
    done, _ = run(make(pages=3, page=4), [[1] * 6], [greedy(6)])
    assert done[0] == expected([1] * 6, 6)


def test_a_prompt_that_waited_too_long_gets_room():
    clock = Clock()
    s = make(max_seqs=2, budget=8, wait_ms=50.0, clock=clock)
    a, b, c = (Sequence(i, [i + 1] * 3, greedy(50)) for i in range(3))
    for q in (a, b, c):
        s.add(q)

    def step():
        plan = s.schedule()
        for q in plan.seqs:
            s.cache.commit(q.seq_id, q.num_cached_tokens + q.num_scheduled_tokens)
        toks = [next_token(q.token_ids) if q.num_cached_tokens + q.num_scheduled_tokens == q.num_tokens else None
                for q in plan.seqs]
        s.postprocess(plan.seqs, toks)
        return plan

    plan = step()
    assert [q.seq_id for q in plan.prefill_seqs] == [0, 1]           # two live requests at most: c waits
    plan = step()
    assert [q.seq_id for q in plan.decode_seqs] == [0, 1] and not plan.prefill_seqs
    clock.t += 0.051                                                  # c has now waited more than 50 ms
    plan = step()
    # one place and one token are kept for c: only one request decodes, the other running one makes room
    assert len(plan.decode_seqs) == 1 and [q.seq_id for q in plan.prefill_seqs] == [2]
    assert len(plan.preempted_seq_ids) == 1


def test_stuck_scheduler_says_so():
    s = make(max_seqs=1, slots=1)
    s.cache.admit("someone else")                                      # the only state slot is taken
    s.add(Sequence(0, [1, 2], greedy(2)))
    with pytest.raises(RuntimeError, match="cannot make progress"):
        s.schedule()


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_give_the_same_completions(seed):
    import random
    rng = random.Random(seed)
    prompts = [[rng.randrange(1, VOCAB) for _ in range(rng.randint(1, 30))] for _ in range(12)]
    params = [greedy(rng.randint(1, 12)) for _ in prompts]
    pages = max(-(-(len(p) + sp.max_tokens) // 4) for p, sp in zip(prompts, params)) + rng.randint(0, 6)
    s = make(pages=pages, page=4, max_seqs=rng.randint(1, 5), budget=rng.randint(2, 20),
             policy=rng.choice(["decode_first", "prefill_first"]))
    done, _ = run(s, prompts, params)
    assert done == {i: expected(p, sp.max_tokens) for i, (p, sp) in enumerate(zip(prompts, params))}


@pytest.mark.parametrize("seed", range(6))
def test_shared_prefixes_change_no_completion(seed):
    """Prompts that start alike share pages; requests that are pushed out find their own pages again. The
    completions are those of a run without sharing, and fewer tokens are computed."""
    import random
    rng = random.Random(100 + seed)
    starts = [[rng.randrange(1, VOCAB) for _ in range(rng.randint(4, 20))] for _ in range(3)]
    prompts = [rng.choice(starts) + [rng.randrange(1, VOCAB) for _ in range(rng.randint(0, 9))] for _ in range(12)]
    params = [greedy(rng.randint(1, 12)) for _ in prompts]
    pages = max(-(-(len(p) + sp.max_tokens) // 4) for p, sp in zip(prompts, params)) + rng.randint(0, 6)
    options = dict(pages=pages, page=4, max_seqs=rng.randint(1, 5), budget=rng.randint(2, 20),
                   policy=rng.choice(["decode_first", "prefill_first"]))
    computed = {}
    for share in (False, True):
        s = make(share_prefixes=share, **options)
        done, log = run(s, prompts, params)
        assert done == {i: expected(p, sp.max_tokens) for i, (p, sp) in enumerate(zip(prompts, params))}
        computed[share] = sum(len(e["decode"]) + sum(n for _, n in e["prefill"]) for e in log)
        if share:
            assert s.cache.num_shared_tokens > 0
    assert computed[True] < computed[False]
