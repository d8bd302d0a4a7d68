"""The scheduler's decisions, with execution simulated by calling back (no GPU),
in the manner of the reference's tests/test_zstreamer.py."""
import random

import pytest

from zse_amd.cache import CacheManager, GroupInfo
from zse_amd.engine.request import FinishReason, Request, RequestState
from zse_amd.engine.scheduler import Scheduler, SchedulerConfig
from zse_amd.sampling import SamplingParams


def make(pages=64, page=4, window=8, seqs=8, budget=64, chunk=16, max_len=512):
    m = CacheManager([GroupInfo(window, [0], pages), GroupInfo(None, [1], pages)], page, seqs, max_len)
    return Scheduler(SchedulerConfig(budget, chunk, seqs), m), m


def req(i, n_prompt, max_tokens=4, stop=None):
    return Request(i, list(range(1, n_prompt + 1)), SamplingParams(max_tokens=max_tokens, stop_tokens=stop))


def run_step(s, token=7):
    plan = s.schedule()
    done = s.on_step_done(plan, {it.request.request_id: token for it in plan.items if it.sample})
    return plan, done


def test_prompt_is_cut_into_portions_under_the_chunk_size():
    # a 120-token prompt with chunk 50 starts with 50 (reference tests/test_zstreamer.py:434-442)
    s, m = make(budget=4096, chunk=50, pages=64)
    r = req("a", 120)
    s.add_request(r)
    sizes = []
    while r.state != RequestState.DECODING:
        plan, _ = run_step(s)
        sizes.append(plan.items[0].count)
    assert sizes == [50, 50, 20]
    assert plan.items[0].sample and r.output_tokens == [7]


def test_token_budget_bounds_every_step_and_decodes_come_first():
    s, m = make(budget=20, chunk=16, pages=128)
    a, b, c = req("a", 3, 50), req("b", 40, 50), req("c", 40, 50)
    for r in (a, b, c):
        s.add_request(r)
    for _ in range(12):
        plan, _ = run_step(s)
        assert plan.num_tokens <= 20
        ids = [it.request.request_id for it in plan.items]
        assert ids == sorted(ids)                         # oldest first
        for it in plan.items:
            if it.request.state == RequestState.DECODING and it.request.num_computed > len(it.request.prompt_tokens):
                assert it.count == 1
    assert a.state == RequestState.DECODING and len(a.output_tokens) > 5


def test_every_request_finishes_in_fifo_order_of_admission():
    s, m = make(budget=32, chunk=8, seqs=2, pages=64)
    rs = [req(i, 5 + 3 * i, max_tokens=3) for i in range(6)]
    for r in rs:
        s.add_request(r)
    order = []
    for _ in range(200):
        if not s.has_work():
            break
        _, done = run_step(s)
        order += [r.request_id for r in done]
    assert not s.has_work() and sorted(order) == list(range(6))
    assert all(r.finish_reason == FinishReason.LENGTH and len(r.output_tokens) == 3 for r in rs)
    assert all(p.free_pages == p.num_pages for p in m.pools) and m.slots.free_slots == 2
    m.check()


def test_stop_token_ends_a_request():
    s, m = make()
    r = req("a", 4, max_tokens=10, stop=[7])
    s.add_request(r)
    run_step(s, token=7)
    assert r.finished and r.finish_reason == FinishReason.STOP and r.output_tokens == [7]
    assert not m.has("a")


def test_admission_waits_when_pages_are_short_and_never_preempts():
    s, m = make(pages=6, page=4, budget=64, chunk=16)
    a, b = req("a", 16, 8), req("b", 16, 8)
    s.add_request(a), s.add_request(b)
    plan = s.schedule()
    # a takes 4 of 6 pages; b's first portion needs 4 and must wait
    assert [it.request.request_id for it in plan.items] == ["a"]
    assert b.state == RequestState.WAITING and not plan.preempted
    assert not m.has("b")                                 # its slot went back


def test_pages_run_out_mid_decode_preempts_the_newest_and_it_recomputes():
    s, m = make(pages=12, page=4, window=64, budget=64, chunk=16, seqs=4)
    a, b = req("a", 7, 30), req("b", 7, 30)
    s.add_request(a), s.add_request(b)
    preempted_seen = False
    for step in range(200):
        if not s.has_work():
            break
        plan, _ = run_step(s, token=step % 50 + 1)
        if plan.preempted:
            preempted_seen = True
            assert plan.preempted == [b]                  # the most recently admitted
            assert b.state == RequestState.PREEMPTED and b.num_computed == 0
            assert s.waiting[0] is b                      # front of the queue
            assert not m.has("b")
            assert len(b.output_tokens) > 0               # keeps what it has produced
        m.check()
    assert preempted_seen and a.finished and b.finished
    assert len(a.output_tokens) == 30 and len(b.output_tokens) == 30
    assert b.num_preemptions >= 1 and a.num_preemptions == 0


def test_recompute_feeds_prompt_plus_generated_tokens():
    s, m = make(pages=12, page=4, window=64, budget=64, chunk=16, seqs=4)
    a, b = req("a", 7, 30), req("b", 7, 30)
    s.add_request(a), s.add_request(b)
    while not b.num_preemptions:
        run_step(s)
    n_out = len(b.output_tokens)
    while b.state != RequestState.PREFILLING:
        plan, _ = run_step(s)
    it = [x for x in plan.items if x.request is b][0]
    assert it.start == 0 and it.count == min(16, 7 + n_out)


def test_a_request_that_cannot_fit_alone_fails_with_an_error():
    s, m = make(pages=2, page=4, budget=64, chunk=16)
    r = req("big", 30, 4)
    s.add_request(r)
    plan = s.schedule()
    assert plan.failed == [r] and r.finish_reason == FinishReason.ERROR and "cache" in r.error
    assert not s.has_work()
    # a decoding request that outgrows the pool alone fails too
    s2, m2 = make(pages=2, page=4, window=64, budget=64, chunk=16)
    r2 = req("grow", 7, 40)
    s2.add_request(r2)
    for _ in range(10):
        run_step(s2)
    assert r2.finish_reason == FinishReason.ERROR and all(p.free_pages == 2 for p in m2.pools)


def test_empty_and_overlong_prompts_are_refused():
    s, m = make(max_len=32)
    with pytest.raises(ValueError):
        s.add_request(Request("e", []))
    with pytest.raises(ValueError):
        s.add_request(req("l", 33))


def test_longest_context_ends_generation():
    s, m = make(max_len=12, pages=16)
    r = req("a", 10, 100)
    s.add_request(r)
    for _ in range(10):
        run_step(s)
    assert r.finish_reason == FinishReason.LENGTH and r.num_tokens == 12


@pytest.mark.parametrize("seed", range(4))
def test_no_starvation_under_random_load(seed):
    rng = random.Random(seed)
    s, m = make(pages=rng.randint(12, 30), page=4, window=8, budget=rng.choice([8, 24, 64]),
                chunk=rng.choice([2, 5, 16]), seqs=rng.randint(2, 5))
    rs = []
    for step in range(400):
        if step < 40 and rng.random() < 0.4:
            r = req(len(rs), rng.randint(1, 20), rng.randint(1, 12))
            rs.append(r)
            s.add_request(r)
        if s.has_work():
            plan, _ = run_step(s, token=rng.randint(1, 99))
            assert plan.num_tokens <= s.config.max_batch_tokens
            assert len(s.running) <= s.config.max_batch_seqs
            m.check()
    assert not s.has_work()
    assert all(r.finished and r.finish_reason == FinishReason.LENGTH for r in rs)
    assert all(len(r.output_tokens) == r.params.max_tokens for r in rs)
    assert all(p.free_pages == p.num_pages for p in m.pools)


def test_a_stop_token_found_after_preemption_ends_the_request_for_good():
    # A run of steps leaves tokens on the device; the newest request is preempted while one of
    # its tokens is still unknown, and that token turns out to be a stop token.  The request
    # must leave the queue: it is never planned, computed or extended again.
    s, m = make(pages=12, page=4, window=64, budget=64, chunk=16, seqs=4)
    a, b = req("a", 7, 30), req("b", 7, 30, stop=[99])
    s.add_request(a), s.add_request(b)
    while not b.num_preemptions:
        plan = s.schedule()
        # ids still on the device: None stands for them, the output gets a placeholder
        s.on_step_done(plan, {it.request.request_id: None for it in plan.items if it.sample})
    assert b in s.waiting and b.state == RequestState.PREEMPTED
    n = len(b.output_tokens)
    assert n >= 2
    b.output_tokens[n - 2] = 99                      # the ids arrive: the one before last ends b
    assert s.finish_at(b, n - 1, FinishReason.STOP) is True
    assert b.finished and b.finish_reason == FinishReason.STOP and len(b.output_tokens) == n - 1
    assert b not in s.waiting and b not in s.running and s.finished["b"] is b
    for _ in range(100):
        if not s.has_work():
            break
        plan = s.schedule()
        assert all(it.request is not b for it in plan.items)
        s.on_step_done(plan, {it.request.request_id: 7 for it in plan.items if it.sample})
        m.check()
    assert not s.has_work() and a.finished and len(b.output_tokens) == n - 1
    assert all(p.free_pages == p.num_pages for p in m.pools)
    # a request that had already ended for another reason is not reported twice
    assert s.finish_at(a, len(a.output_tokens), FinishReason.STOP) is False


def test_every_admission_clears_the_state_slot():
    # whoever makes a request live (first admission, or admission again after preemption),
    # the owner of the slots' memory hears of it, with the slot the request got
    s, m = make(pages=12, page=4, window=64, budget=64, chunk=16, seqs=2)
    cleared = []
    m.on_admit = lambda r, slot: cleared.append((r, slot))
    rs = [req(i, 7, 20) for i in range(4)]
    for r in rs:
        s.add_request(r)
    for _ in range(300):
        if not s.has_work():
            break
        before = set(m.live())
        run_step(s)
        for r in set(m.live()) - before:
            assert (r, m.slot(r)) in cleared
    assert not s.has_work()
    admissions = sum(1 + r.num_preemptions for r in rs)
    assert sum(r.num_preemptions for r in rs) > 0 and len(cleared) >= admissions
    assert {slot for _, slot in cleared} == {0, 1}          # two slots served four requests


def test_penalty_counts_follow_the_continuous_batching_engine():
    r = Request("p", [5, 5, 9], SamplingParams(max_tokens=8, repetition_penalty=1.3))
    assert r.penalty_counts() == {5: 1, 9: 1}                # prompt tokens count once each
    r.output_tokens += [9, 4, 4, 4]
    assert r.penalty_counts() == {5: 1, 9: 2, 4: 3}          # produced tokens add up


def test_a_small_windowed_pool_is_what_runs_out():
    # the windowed group has a pool of its own, sized for its window and a step's tokens: when
    # it is the one that cannot give a page, the newest request gives way as with any pool
    m = CacheManager([GroupInfo(8, [0], 7), GroupInfo(None, [1], 64)], 4, 4, 512)
    s = Scheduler(SchedulerConfig(64, 8, 4), m)
    rs = [req(i, 14, 12) for i in range(3)]          # each holds up to ceil((8 + 8) / 4) + 1 = 5 windowed pages
    for r in rs:
        s.add_request(r)
    seen = False
    for _ in range(300):
        if not s.has_work():
            break
        plan, _ = run_step(s)
        seen = seen or bool(plan.preempted)
        assert m.pools[0].used_pages <= 7
        m.check()
    assert seen and not s.has_work() and all(len(r.output_tokens) == 12 for r in rs)
    assert all(p.free_pages == p.num_pages for p in m.pools)


def test_tokens_at_is_a_slice_of_all_tokens():
    r = Request("t", [1, 2, 3, 4], SamplingParams(max_tokens=8))
    r.output_tokens = [10, 11, 12]
    for start in range(7):
        for count in range(0, 8 - start):
            assert r.tokens_at(start, count) == r.all_tokens[start:start + count]
