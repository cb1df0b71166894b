"""The scheduler's decisions (host code, no GPU): admission, portions under the
token budget, decoding, finishing, freeing, and what happens when pages run out."""
import random

import pytest

from lyapunov_engine_amd.cache import CacheManager, GroupConfig
from lyapunov_engine_amd.engine.scheduler import Scheduler, SchedulerError
from lyapunov_engine_amd.sampling.params import SamplingParams


def make(pages=64, page=4, seqs=8, budget=32, max_len=256, chunk=0, eos=(), slots=None, window=0):
    cache = CacheManager([GroupConfig(pages, page, window)], slots or seqs)
    return cache, Scheduler(cache, max_num_seqs=seqs, max_num_batched_tokens=budget, max_model_len=max_len,
                            max_chunk=chunk, eos_token_ids=eos)


def run_to_end(cache, sched, next_token=lambda seq_id, n: 100 + n, max_steps=10_000, checks=None):
    """Drive the scheduler with a fake model; returns {seq: all tokens}."""
    produced = {}
    for _ in range(max_steps):
        if not sched.has_unfinished():
            break
        plan = sched.schedule()
        if checks:
            checks(plan)
        sampled = []
        for p in plan:
            info = sched.info(p.seq_id)
            assert p.start == info.num_computed and p.count >= 1
            assert p.wants_logits == (p.start + p.count == info.total_len)
            assert cache.capacity(p.seq_id) >= p.start + p.count
            if p.wants_logits:
                sampled.append(next_token(p.seq_id, info.total_len - info.prompt_len))
        sched.post_step(sampled)
        cache.check()
        for p in plan:
            produced[p.seq_id] = sched.tokens(p.seq_id)
    else:
        raise AssertionError("the scheduler did not finish")
    return produced


def test_reference_vector_three_tokens():
    # tests/test_block_manager.py:43-80: prompt [10, 20, 30], max_tokens 3: a prompt step, two decode steps, done
    cache, s = make()
    s.add(0, [10, 20, 30], SamplingParams(max_tokens=3))
    plan = s.schedule()
    assert [(p.start, p.count, p.wants_logits) for p in plan] == [(0, 3, True)]
    s.post_step([7])
    for k in (3, 4):
        plan = s.schedule()
        assert [(p.start, p.count, p.wants_logits) for p in plan] == [(k, 1, True)]
        s.post_step([7])
    info = s.info(0)
    assert info.finished and info.status == "finished_length_capped" and s.tokens(0) == [10, 20, 30, 7, 7, 7]
    assert not s.has_unfinished() and cache.num_free_pages() == 64 and cache.num_requests() == 0
    with pytest.raises(SchedulerError, match="planned 0"):
        s.post_step([1])  # sizes must match (scheduler.cpp:106-109)


def test_prompts_are_cut_into_portions_under_the_budget_beside_decodes():
    cache, s = make(budget=16)
    s.add(0, list(range(5)), SamplingParams(max_tokens=4, ignore_eos=True))
    plan = s.schedule()
    assert [(p.seq_id, p.start, p.count, p.wants_logits) for p in plan] == [(0, 0, 5, True)]
    s.post_step([1])
    s.add(1, list(range(40)), SamplingParams(max_tokens=2, ignore_eos=True))   # longer than the budget: no stall
    seen = []
    for _ in range(3):
        plan = s.schedule()
        seen.append([(p.seq_id, p.start, p.count, p.wants_logits) for p in plan])
        assert sum(p.count for p in plan) <= 16
        s.post_step([1] * sum(p.wants_logits for p in plan))
    assert seen[0] == [(0, 5, 1, True), (1, 0, 15, False)]     # a decoded token first, then what is left of the budget
    assert seen[1] == [(0, 6, 1, True), (1, 15, 15, False)]
    assert seen[2] == [(0, 7, 1, True), (1, 30, 10, True)]     # the portion that ends the prompt asks for logits
    assert s.info(0).finished


def test_max_chunk_and_max_num_seqs():
    cache, s = make(seqs=2, budget=64, chunk=8)
    for i in range(3):
        s.add(i, list(range(20)), SamplingParams(max_tokens=1))
    plan = s.schedule()
    assert [(p.seq_id, p.count) for p in plan] == [(0, 8), (1, 8)] and s.num_waiting() == 1
    s.post_step([])
    done = run_to_end(cache, s)
    assert all(len(done[i]) == 21 for i in range(3))


def test_finishing_on_eos_max_tokens_and_model_length():
    cache, s = make(eos=(2, 9), max_len=12)
    s.add(0, [1, 1, 1], SamplingParams(max_tokens=50))
    s.add(1, [1, 1, 1], SamplingParams(max_tokens=50, ignore_eos=True))
    s.add(2, [1] * 8, SamplingParams(max_tokens=50, ignore_eos=True))
    run_to_end(cache, s, next_token=lambda sid, n: 9 if n == 2 else 5)
    assert s.info(0).status == "finished_stopped" and s.tokens(0) == [1, 1, 1, 5, 5, 9]
    assert s.info(1).status == "finished_length_capped" and len(s.tokens(1)) == 12   # the model's length
    assert len(s.tokens(2)) == 12
    assert cache.num_requests() == 0 and cache.num_free_pages() == 64
    s.forget(0)
    with pytest.raises(SchedulerError):
        s.info(0)


def test_requests_that_can_never_run_are_refused():
    cache, s = make(pages=8, page=4, max_len=64)
    with pytest.raises(SchedulerError, match="empty"):
        s.add(0, [], SamplingParams())
    with pytest.raises(SchedulerError, match="max_model_len"):
        s.add(0, [1] * 64, SamplingParams())
    with pytest.raises(SchedulerError, match="pages"):
        s.add(0, [1] * 30, SamplingParams(max_tokens=10))      # 40 tokens > 8 pages of 4
    s.add(0, [1] * 30, SamplingParams(max_tokens=2))           # 32 tokens fit exactly
    with pytest.raises(SchedulerError, match="in use"):
        s.add(0, [1], SamplingParams())
    assert len(run_to_end(cache, s)[0]) == 32


def test_when_pages_run_out_the_last_admitted_request_is_preempted_and_recomputed():
    cache, s = make(pages=10, page=4, budget=64)
    s.add(0, [1] * 14, SamplingParams(max_tokens=12, ignore_eos=True))
    s.add(1, [2] * 14, SamplingParams(max_tokens=12, ignore_eos=True))
    preempted, order = [], []

    def checks(plan):
        preempted.extend(s.last_preempted())
        order.append([(p.seq_id, p.start, p.count) for p in plan])

    done = run_to_end(cache, s, next_token=lambda sid, n: 1000 * sid + n, checks=checks)
    assert preempted and set(preempted) == {1}                 # the request admitted last gives way
    assert s.info(1).preemptions >= 1 and s.info(0).preemptions == 0
    # both finish with exactly the tokens an undisturbed run gives
    assert done[0] == [1] * 14 + list(range(12)) and done[1] == [2] * 14 + [1000 + n for n in range(12)]
    # after a preemption the request comes back as one prompt: its own prompt and what it had produced
    i = next(k for k, plan in enumerate(order) if any(sid == 1 and start == 0 and k > 0 for sid, start, _ in plan))
    again = [c for sid, st, c in order[i] if sid == 1][0]
    assert again > 14
    assert s.counters()["preemptions"] == len(preempted)


def test_abort_frees_pages_wherever_the_request_is():
    cache, s = make()
    s.add(0, [1] * 10, SamplingParams(max_tokens=5))
    s.add(1, [1] * 10, SamplingParams(max_tokens=5))
    s.schedule()
    s.post_step([3, 3])
    s.add(2, [1] * 10, SamplingParams(max_tokens=5))
    assert s.abort(0) and s.abort(2) and not s.abort(0) and not s.abort(77)
    assert s.info(0).status == "finished_aborted" and s.num_running() == 1 and s.num_waiting() == 0
    run_to_end(cache, s)
    assert cache.num_free_pages() == 64 and cache.num_requests() == 0


def test_window_group_lets_a_long_request_run_in_few_pages():
    cache, s = make(pages=6, page=4, budget=8, window=5, max_len=200)
    s.add(0, [1] * 50, SamplingParams(max_tokens=30, ignore_eos=True))   # 80 tokens through 6 pages
    done = run_to_end(cache, s)
    assert len(done[0]) == 80 and cache.num_free_pages() == 6


@pytest.mark.parametrize("seed", range(5))
def test_random_load_every_request_finishes_with_the_right_tokens(seed):
    rng = random.Random(seed)
    page = rng.choice([2, 4, 16])
    budget, max_seqs = rng.randint(8, 40), rng.randint(2, 6)
    cache, s = make(pages=rng.randint(24, 60), page=page, seqs=max_seqs, budget=budget,
                    chunk=rng.choice([0, 0, 5]), max_len=120)
    want = {}
    pending = list(range(14))

    def checks(plan):
        assert len({p.seq_id for p in plan}) == len(plan)
        assert sum(p.count for p in plan) <= budget and len(plan) <= max_seqs and s.num_running() <= max_seqs
        while pending and rng.random() < 0.4:
            i = pending.pop(0)
            n, m = rng.randint(1, 40), rng.randint(1, 20)
            if (n + m + page - 1) // page > cache.groups[0].num_pages:
                continue
            s.add(i, [i] * n, SamplingParams(max_tokens=m, ignore_eos=True))
            want[i] = [i] * n + [10_000 * i + k for k in range(m)]

    checks([])
    for _ in range(50):
        done = run_to_end(cache, s, next_token=lambda sid, n: 10_000 * sid + n, checks=checks)
        if not pending:
            break
        checks([])
    for i, toks in want.items():
        assert s.tokens(i) == toks and s.info(i).finished
    assert cache.num_requests() == 0 and cache.num_free_pages() == cache.groups[0].num_pages
