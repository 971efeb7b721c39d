"""Scheduler decisions, driven by hand as the engine would (no torch, no model).
Scenarios of reference tests/unit/test_scheduler.py:33-174 (minus static mode),
plus token budget, prompt portions and what happens when pages run out."""

import random

import pytest

from tokamak_amd.cache import CacheGroupSpec, CacheManager, OutOfPagesError
from tokamak_amd.engine.request import FinishReason, Request
from tokamak_amd.engine.scheduler import Scheduler
from tokamak_amd.sampling.params import SamplingParams


def make_seq(rid, prompt_len=4, max_new=8):
    return Request.from_prompt(rid, [1] * prompt_len, SamplingParams(max_new_tokens=max_new))


def make(num_pages=16, page_size=4, max_batch=4, budget=64, chunk=None):
    manager = CacheManager([CacheGroupSpec("full", (0,))], num_pages, page_size, max_batch)
    return Scheduler(manager, max_batch, budget, chunk), manager


def run_step(step, token=0):
    """What the engine does after a step: advance caches, append sampled tokens."""
    for span in step.spans:
        assert span.start == span.request.cached
        span.request.advance(span.length)
    for span in step.spans:
        if span.samples:
            span.request.tokens.append(token)


def finish(seq, manager):
    seq.finish_reason = FinishReason.STOP
    manager.free(seq.rid)


def test_admits_in_fcfs_order_and_batches_prompts_under_the_budget():
    sched, _ = make(budget=10)
    seqs = [make_seq(i) for i in range(3)]
    for s in seqs:
        sched.submit(s)
    step = sched.plan()
    # budget 10: two whole prompts of 4 and the first 2 tokens of the third
    assert [(s.request.rid, s.start, s.length, s.samples) for s in step.spans] == [
        (0, 0, 4, True), (1, 0, 4, True), (2, 0, 2, False)]
    assert sched.running == seqs and not sched.waiting
    run_step(step)
    step = sched.plan()
    # decodes of the first two come first, then the rest of the third prompt
    assert [(s.request.rid, s.start, s.length, s.samples) for s in step.spans] == [
        (0, 4, 1, True), (1, 4, 1, True), (2, 2, 2, True)]
    run_step(step)
    step = sched.plan()
    assert [(s.request.rid, s.length) for s in step.spans] == [(0, 1), (1, 1), (2, 1)]


def test_prompt_is_cut_into_portions_of_prefill_chunk():
    sched, manager = make(num_pages=32, budget=64, chunk=5)
    seq = make_seq(0, prompt_len=12)
    sched.submit(seq)
    cuts = []
    while seq.num_generated == 0:
        step = sched.plan()
        cuts.append((step.spans[0].start, step.spans[0].length, step.spans[0].samples))
        run_step(step)
    assert cuts == [(0, 5, False), (5, 5, False), (10, 2, True)]
    # pages were reserved portion by portion
    assert len(manager.block_table(0)) == 3


def test_admission_respects_max_batch_size():
    sched, manager = make(max_batch=2)
    seqs = [make_seq(i) for i in range(3)]
    for s in seqs:
        sched.submit(s)
    step = sched.plan()
    assert [s.request.rid for s in step.spans] == [0, 1]
    run_step(step)
    step = sched.plan()
    assert [s.request.rid for s in step.spans] == [0, 1]      # batch full: third waits
    run_step(step)
    finish(seqs[0], manager)
    step = sched.plan()
    assert [(s.request.rid, s.length) for s in step.spans] == [(1, 1), (2, 4)]


def test_no_bypass_of_the_head_of_the_queue():
    # 4 pages of 4; first takes 3; second needs 2 and must wait; a third that would fit waits too
    sched, manager = make(num_pages=4)
    first, second, third = make_seq(0, 12), make_seq(1, 8), make_seq(2, 3)
    for s in (first, second, third):
        sched.submit(s)
    step = sched.plan()
    assert [s.request.rid for s in step.spans] == [0]
    run_step(step)
    step = sched.plan()
    assert [s.request.rid for s in step.spans] == [0]
    run_step(step)
    finish(first, manager)
    step = sched.plan()
    assert [s.request.rid for s in step.spans] == [1, 2]


def test_decode_reserves_the_next_tokens_page():
    sched, manager = make(num_pages=8)
    seq = make_seq(0, 4)
    sched.submit(seq)
    run_step(sched.plan())
    assert manager.reserved_tokens(0) == 4
    sched.plan()                       # token 5 needs a second page
    assert manager.reserved_tokens(0) == 8


def test_pages_run_out_newest_is_preempted_and_requeued_at_the_front():
    sched, manager = make(num_pages=4, max_batch=4)
    old, new = make_seq(0, 8, 16), make_seq(1, 8, 16)
    late = make_seq(2, 4, 4)
    sched.submit(old)
    sched.submit(new)
    run_step(sched.plan())             # both prompts, pool now full
    sched.submit(late)
    step = sched.plan()                # both need a third page: none free
    assert [s.request.rid for s in step.spans] == [0]
    assert step.evicted == [new]
    assert new not in sched.running and new.cached == 0 and new.evictions == 1
    assert sched.waiting[0] is new and sched.waiting[1] is late   # front, ahead of later arrivals
    assert manager.block_table(1) == []
    run_step(step)
    finish(old, manager)
    step = sched.plan()
    # the victim resumes over prompt + its generated token, and samples at its end
    assert (step.spans[0].request, step.spans[0].start, step.spans[0].length, step.spans[0].samples) == (new, 0, 9, True)
    assert len(new.tokens) == 9


def test_a_sequence_that_starves_alone_preempts_itself_and_resumes():
    # one page short for the newest: it is its own victim and comes back once there is room
    sched, manager = make(num_pages=3, max_batch=2)
    a, b = make_seq(0, 4, 16), make_seq(1, 8, 16)
    sched.submit(a)
    sched.submit(b)
    run_step(sched.plan())              # a: 1 page, b: 2 pages
    step = sched.plan()                 # a needs a 2nd page -> b (newest) is evicted
    assert step.evicted == [b] and [s.request.rid for s in step.spans] == [0]
    manager.check()


def test_impossible_prompt_raises():
    sched, _ = make(num_pages=2)
    sched.submit(make_seq(0, 12))
    with pytest.raises(OutOfPagesError, match="pool can ever provide"):
        sched.plan()


def test_all_finished_returns_none():
    sched, manager = make()
    seq = make_seq(0)
    sched.submit(seq)
    run_step(sched.plan())
    finish(seq, manager)
    assert not sched.busy
    assert sched.plan() is None


def test_budget_must_cover_the_batch():
    with pytest.raises(ValueError, match="max_num_batched_tokens"):
        make(max_batch=8, budget=4)


def test_one_token_prompt_is_a_portion_then_decodes():
    sched, _ = make()
    seq = make_seq(0, 1)
    sched.submit(seq)
    step = sched.plan()
    assert (step.spans[0].start, step.spans[0].length, step.spans[0].samples) == (0, 1, True)
    run_step(step)
    step = sched.plan()
    assert (step.spans[0].start, step.spans[0].length) == (1, 1)


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_finish_with_every_page_back(seed):
    rng = random.Random(seed)
    sched, manager = make(num_pages=12, page_size=4, max_batch=3, budget=16, chunk=7)
    seqs = [make_seq(i, rng.randint(1, 30), rng.randint(1, 12)) for i in range(12)]
    for s in seqs:
        sched.submit(s)
    steps = 0
    while sched.busy:
        step = sched.plan()
        assert step is not None and step.spans
        assert step.num_tokens <= 16 and len(step.spans) <= 3
        ids = [s.request.rid for s in step.spans]
        assert len(set(ids)) == len(ids)
        for span in step.spans:
            # the pages for the span are there before it runs
            assert len(manager.block_table(span.request.rid)) * 4 >= span.start + span.length
        run_step(step)
        for span in step.spans:
            seq = span.request
            if span.samples and (seq.num_generated >= seq.params.max_new_tokens
                                 or len(seq.tokens) >= 48):
                finish(seq, manager)
        manager.check()
        steps += 1
        assert steps < 2000
    assert all(s.finished for s in seqs)
    assert manager.num_free_pages() == 12 and manager.slots.num_free == 3


# ---------------------------------------------------------------------------
# one step ahead: plans made before the tokens of the step before are read
# ---------------------------------------------------------------------------
def launch(step):
    """What the step loop does when it launches a step: caches advance, sampled tokens
    are on their way (rows in the order of the sampling spans)."""
    row = 0
    for span in step.spans:
        assert span.start == span.request.cached
        span.request.advance(span.length)
    for span in step.spans:
        if span.samples:
            span.request.unknown += 1
            span.request.feed_row = row
            row += 1


def read(step, token=0, eos=()):
    """... and when it reads them."""
    for span in step.spans:
        if span.samples and not span.request.finished:
            span.request.accept(token, eos_token_ids=tuple(eos), context_limit=10 ** 6)


def test_a_decode_span_may_be_a_token_that_is_still_on_the_gpu():
    sched, _ = make(budget=16)
    a, b = make_seq(0, prompt_len=4, max_new=3), make_seq(1, prompt_len=6, max_new=8)
    sched.submit(a)
    sched.submit(b)
    first = sched.plan()
    launch(first)
    assert a.unknown == b.unknown == 1 and a.length == 5 and a.decoding and not a.closing
    second = sched.plan()                       # planned before the first step's tokens are read
    assert [(s.request.rid, s.start, s.length, s.samples, s.feed) for s in second.spans] == [
        (0, 4, 1, True, 0), (1, 6, 1, True, 1)]
    assert a.span(1) == [0]                     # a placeholder: the step takes the token from the sampler's output
    launch(second)
    read(first, token=7)
    assert a.tokens[-1] == 7 and a.unknown == 1 and a.num_drawn == 2
    third = sched.plan()
    launch(third)
    read(second, token=8)
    # a has drawn three tokens of three: it is certain to end, and is planned no further
    assert a.unknown == 1 and a.closing and not a.decoding
    fourth = sched.plan()
    assert [s.request.rid for s in fourth.spans] == [1]
    launch(fourth)
    read(third, token=9)
    assert a.finished and a.finish_reason == FinishReason.LENGTH and a.generated == [7, 8, 9]


def test_a_plan_may_be_empty_while_the_last_tokens_are_on_their_way():
    sched, manager = make()
    a = make_seq(0, prompt_len=3, max_new=1)
    sched.submit(a)
    first = sched.plan()
    launch(first)
    assert a.closing and sched.busy
    waiting = sched.plan()
    assert waiting is not None and waiting.spans == []      # not "nothing left", and nobody is evicted for it
    read(first, token=5)
    assert a.finished
    manager.free(a.rid)
    assert sched.plan() is None


def test_an_end_that_is_read_late_costs_one_token_and_nothing_else():
    sched, manager = make()
    a, b = make_seq(0, prompt_len=3, max_new=8), make_seq(1, prompt_len=3, max_new=8)
    sched.submit(a)
    sched.submit(b)
    first = sched.plan()
    launch(first)
    second = sched.plan()
    launch(second)
    read(first, token=2, eos=(2,))              # both stop on the token of the first step ...
    assert a.finished and b.finished and a.finish_reason == FinishReason.STOP
    read(second, token=3)                       # ... and the second step's tokens are dropped
    assert a.generated == [2] and b.generated == [2]
    for r in (a, b):
        manager.free(r.rid)
    assert sched.plan() is None
    manager.check()
    assert manager.num_free_pages() == manager.num_pages()


def test_a_request_evicted_with_a_token_on_its_way_waits_until_it_is_read():
    sched, manager = make(num_pages=4, page_size=4, max_batch=2, budget=16)
    a, b = make_seq(0, prompt_len=8, max_new=8), make_seq(1, prompt_len=8, max_new=8)
    sched.submit(a)
    sched.submit(b)
    first = sched.plan()
    launch(first)                               # 2 pages each: the pool is full, both tokens on their way
    second = sched.plan()                       # a's next token needs a third page: b, the newest, goes
    assert [r.rid for r in second.evicted] == [1] and [s.request.rid for s in second.spans] == [0]
    assert b.cached == 0 and b.unknown == 1 and sched.waiting[0] is b
    launch(second)
    read(first, token=4)
    assert b.tokens[-1] == 4 and b.unknown == 0 and len(b.tokens) == 9
    third = sched.plan()
    assert all(s.request is not b or s.feed is None for s in third.spans)


# ---------------------------------------------------------------------------
# the whole step loop one step ahead, as LLM.generate runs it, without a GPU
# ---------------------------------------------------------------------------
def ahead_loop(sched, manager, token_of, eos=(), context_limit=10 ** 6, in_turn=False):
    """The step loop of the entry point: plan and launch step i+1, then read step i.
    ``token_of(request, draw)`` is the sampler.  Returns the plans, in order."""
    plans = []
    in_flight = None

    def read_back(step, tokens):
        for span, token in zip([s for s in step.spans if s.samples], tokens):
            request = span.request
            if request.finished:
                continue
            if request.accept(token, eos_token_ids=tuple(eos), context_limit=context_limit):
                manager.free(request.rid)

    guard = 0
    while sched.busy or in_flight is not None:
        guard += 1
        assert guard < 5000
        plan = sched.plan() if sched.busy else None
        launched = None
        if plan is not None:
            plans.append(plan)
            for span in plan.spans:
                request = span.request
                assert not request.finished, f"a span was planned for finished request {request.rid}"
                assert span.start == request.cached
                assert len(manager.block_table(request.rid)) * manager.page_size >= span.start + span.length
            ids = [s.request.rid for s in plan.spans]
            assert len(set(ids)) == len(ids)
            if plan.spans:
                tokens = [token_of(s.request, s.request.num_drawn) for s in plan.spans if s.samples]
                launch(plan)
                launched = (plan, tokens) if tokens else None
        if in_flight is not None:
            read_back(*in_flight)
        else:
            assert plan is not None and plan.spans, "unfinished requests, but no step"
        in_flight = launched
        if in_flight is not None and in_turn:
            read_back(*in_flight)
            in_flight = None
        manager.check()
    return plans


def test_a_request_that_ends_while_it_waits_is_never_planned_again():
    # ten pages of eight tokens, three prompts of twenty; request 2 draws its EOS as its fifth
    # token and is evicted while that token is on its way
    EOS = 99
    manager = CacheManager([CacheGroupSpec("full", (0,))], 10, 8, 3)
    sched = Scheduler(manager, 3, 64)
    requests = [Request.from_prompt(i, [1] * 20, SamplingParams(max_new_tokens=30)) for i in range(3)]
    for r in requests:
        sched.submit(r)

    def token_of(request, draw):
        return EOS if request.rid == 2 and draw == 4 else 7

    plans = ahead_loop(sched, manager, token_of, eos=(EOS,))
    assert any(requests[2] in p.evicted for p in plans)            # the case is the one meant
    assert requests[2].finish_reason == FinishReason.STOP and requests[2].generated[-1] == EOS
    assert len(requests[2].generated) == 5
    assert all(r.finished for r in requests)
    assert requests[0].num_generated == 30 and requests[1].num_generated == 30
    assert manager.num_free_pages() == 10 and manager.slots.num_free == 3
    assert not sched.waiting or all(r.finished for r in sched.waiting)


def test_a_victim_that_ends_with_the_token_on_its_way_is_released_not_queued():
    sched, manager = make(num_pages=4, page_size=4, max_batch=2, budget=16)
    a, b = make_seq(0, prompt_len=8, max_new=8), make_seq(1, prompt_len=8, max_new=1)
    sched.submit(a)
    sched.submit(b)
    first = sched.plan()
    launch(first)                               # the pool is full; b's only token is on its way
    assert b.closing
    second = sched.plan()                       # a needs a third page: b gives its pages back ...
    assert second.released == [b] and second.evicted == []
    assert [s.request.rid for s in second.spans] == [0]
    assert b not in sched.running and b not in sched.waiting and b.evictions == 0   # ... and is not queued
    assert manager.block_table(1) == []
    launch(second)
    read(first, token=4)
    assert b.finished and b.generated == [4]
    manager.free(b.rid)                         # what the reader does; nothing is left to give back
    manager.check()


@pytest.mark.parametrize("seed", range(40))
def test_random_workloads_one_step_ahead_with_stops(seed):
    rng = random.Random(1000 + seed)
    EOS = 5
    pages = rng.randint(6, 14)
    sched, manager = make(num_pages=pages, page_size=4, max_batch=rng.randint(1, 4), budget=16,
                          chunk=rng.choice([None, 3, 7]))
    limit = pages * 4
    seqs = [make_seq(i, rng.randint(1, min(20, limit - 2)), rng.randint(1, 14)) for i in range(rng.randint(3, 12))]
    for s in seqs:
        sched.submit(s)
        s.context_limit = min(limit, s.prompt_len + s.params.max_new_tokens)
    draws = {}

    def token_of(request, draw):
        # a fixed token per (request, draw): the same under any schedule
        return draws.setdefault((request.rid, draw), EOS if rng.random() < 0.12 else rng.randint(6, 50))

    ahead_loop(sched, manager, token_of, eos=(EOS,), context_limit=limit)
    assert all(s.finished for s in seqs)
    assert manager.num_free_pages() == pages and manager.slots.num_free == manager.slots.num_slots
    ahead = [list(s.generated) for s in seqs]

    # the same requests read in turn give the same tokens
    sched2, manager2 = make(num_pages=pages, page_size=4, max_batch=sched.max_batch_size, budget=16,
                            chunk=None if sched.chunk == 16 else sched.chunk)
    again = [make_seq(s.rid, s.prompt_len, s.params.max_new_tokens) for s in seqs]
    for s in again:
        sched2.submit(s)
        s.context_limit = min(limit, s.prompt_len + s.params.max_new_tokens)
    ahead_loop(sched2, manager2, token_of, eos=(EOS,), context_limit=limit, in_turn=True)
    assert [list(s.generated) for s in again] == ahead
