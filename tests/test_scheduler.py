"""The scheduler's decisions (no GPU): a fake "model" answers with a token that depends on
the request's tokens so far, so preemption and recomputation must reproduce it."""

import pytest

from flyweight_amd.cache import CacheManager, FixedState, PagedKV
from flyweight_amd.engine.scheduler import (EVENT_ERROR, EVENT_FINISHED, EVENT_PREFILL, EVENT_TOKEN, Scheduler,
                                            SchedulerError)
from flyweight_amd.sampling import GREEDY

NEEDS = {0: PagedKV(2, 16), 1: FixedState((4, 2))}


def oracle(tokens):
    return (sum(tokens) * 31 + len(tokens)) % 97


def make(num_pages=8, max_requests=4, **kw):
    cache = CacheManager(NEEDS, num_pages=num_pages, max_requests=max_requests)
    return cache, Scheduler(cache, max_positions=kw.pop("max_positions", 4096), **kw)


def drive(scheduler, cache, max_steps=10000, log=None):
    """Runs to completion; returns request id -> (tokens, finished-event count)."""
    seen = {}
    steps = 0
    while scheduler.has_work():
        plan = scheduler.schedule()
        # what the step function would check
        ids = [s.request.id for s in plan.segments]
        assert len(ids) == len(set(ids)), "a request appears twice in a step"
        assert plan.num_tokens <= scheduler.max_batch_tokens
        for segment in plan.segments:
            r = segment.request
            assert r.live and list(segment.tokens) == r.tokens[r.computed:r.computed + len(segment.tokens)]
            assert cache.pages_missing(r.id, r.computed + len(segment.tokens)) == {0: 0}, "pages were not reserved"
            assert segment.wants_logits == (r.computed + len(segment.tokens) == len(r.tokens))
        sampled = {s.request.id: oracle(s.request.tokens) for s in plan.segments if s.wants_logits}
        if log is not None:
            log.append(plan)
        for event in scheduler.complete(plan, sampled):
            seen.setdefault(event[0], []).append(event)
        cache.check_invariants()
        steps += 1
        assert steps < max_steps, "the scheduler does not make progress"
    return seen


def expected_tokens(prompt, count, stop=()):
    tokens, out = list(prompt), []
    for _ in range(count):
        t = oracle(tokens)
        out.append(t)
        tokens.append(t)
        if t in stop:
            break
    return out


def test_submit_validation():
    cache, scheduler = make(max_positions=100)
    with pytest.raises(SchedulerError, match="empty"):
        scheduler.submit([], 4)
    with pytest.raises(SchedulerError, match="exceeds the context"):
        scheduler.submit([1] * 90, 11)
    with pytest.raises(SchedulerError, match="at least 1"):
        scheduler.submit([1], 0)
    scheduler.submit([1] * 90, 10)
    for _ in range(255):
        scheduler.submit([1], 1)
    with pytest.raises(SchedulerError, match="queue"):
        scheduler.submit([1], 1)


def test_token_ids_are_checked_against_the_vocabulary_at_submit():
    cache = CacheManager(NEEDS, num_pages=8, max_requests=4)
    scheduler = Scheduler(cache, max_positions=4096, vocab_size=97)
    with pytest.raises(SchedulerError, match=r"token id 97 at place 2 of the prompt is outside the vocabulary \(0\.\.96\)"):
        scheduler.submit([1, 96, 97], 4)
    with pytest.raises(SchedulerError, match="token id -1 at place 0"):
        scheduler.submit([-1], 4)
    with pytest.raises(SchedulerError, match="stop token 500"):
        scheduler.submit([1], 4, stop_tokens=[500])
    assert not scheduler.has_work() and not scheduler.requests
    scheduler.submit([0, 96], 4, stop_tokens=[96])
    assert scheduler.has_work()


def test_prompt_is_cut_into_portions_under_the_budget_and_decodes_come_first():
    cache, scheduler = make(num_pages=16, max_batch_tokens=24, chunk_size=16)
    a = scheduler.submit(list(range(40)), 5)
    log = []
    plan = scheduler.schedule()
    assert [(s.request.id, len(s.tokens), s.wants_logits) for s in plan.segments] == [(a.id, 16, False)]
    scheduler.complete(plan, {})
    b = scheduler.submit(list(range(10)), 3)
    plan = scheduler.schedule()          # a's next portion, and b's prompt in what is left of the budget
    assert [(s.request.id, len(s.tokens), s.wants_logits) for s in plan.segments] == [(a.id, 16, False), (b.id, 8, False)]
    scheduler.complete(plan, {})
    plan = scheduler.schedule()
    assert [(s.request.id, len(s.tokens), s.wants_logits) for s in plan.segments] == [(a.id, 8, True), (b.id, 2, True)]
    scheduler.complete(plan, {a.id: oracle(a.tokens), b.id: oracle(b.tokens)})
    c = scheduler.submit(list(range(30)), 2)
    plan = scheduler.schedule()          # both decode rows first, then the newcomer's portion
    assert [(s.request.id, len(s.tokens)) for s in plan.segments] == [(a.id, 1), (b.id, 1), (c.id, 16)]
    assert all(s.wants_logits for s in plan.segments[:2]) and not plan.segments[2].wants_logits


def test_runs_to_the_same_tokens_as_one_request_alone():
    cache, scheduler = make(num_pages=32, max_batch_tokens=32, chunk_size=16)
    prompts = [list(range(5)), list(range(3, 20)), list(range(7, 38)), [9]]
    requests = [scheduler.submit(p, 8) for p in prompts]
    seen = drive(scheduler, cache)
    for request, prompt in zip(requests, prompts):
        assert request.generated == expected_tokens(prompt, 8)
        kinds = [e[2] for e in seen[request.id]]
        assert kinds.count(EVENT_FINISHED) == 1 and kinds[-1] == EVENT_FINISHED and kinds.count(EVENT_TOKEN) == 8
    assert cache.stats()["pages_free"] == 32 and cache.slots.free_count == 4 and not cache.requests


def test_stop_token_and_position_limit_end_a_request():
    cache, scheduler = make(max_positions=12)
    prompt = [1, 2, 3]
    stop = expected_tokens(prompt, 4)[2]
    a = scheduler.submit(prompt, 9, stop_tokens=[stop])
    b = scheduler.submit([5] * 8, 4)
    drive(scheduler, cache)
    assert a.generated == expected_tokens(prompt, 9, stop=(stop,)) and a.generated[-1] == stop
    assert len(b.generated) == 4 and len(b.prompt) + len(b.generated) == 12


def test_out_of_pages_preempts_the_newest_and_never_the_oldest():
    # 4 pages of 64: two requests of 100 + 120 tokens cannot both finish
    cache, scheduler = make(num_pages=4, max_batch_tokens=256, chunk_size=128)
    old = scheduler.submit([3] * 100, 120)
    new = scheduler.submit([4] * 100, 120)
    log = []
    seen = drive(scheduler, cache, log=log)
    assert scheduler.preemptions >= 1 and old.preemptions == 0 and new.preemptions >= 1
    assert old.generated == expected_tokens([3] * 100, 120)
    assert new.generated == expected_tokens([4] * 100, 120)     # recomputed, nothing lost or doubled
    preempting = [p for p in log if p.preempted]
    assert all(p.preempted[0] is new for p in preempting)
    assert all(not p.admitted for p in preempting), "nobody is admitted in a step in which somebody gave way"
    assert [e[2] for e in seen[new.id]].count(EVENT_FINISHED) == 1
    # a preempted request recomputes prompt + generated as portions and asks for logits only at the end
    after = log[log.index(preempting[0]) + 1:]
    recompute = [s for p in after for s in p.segments if s.request is new and len(s.tokens) > 1]
    assert recompute and list(recompute[0].tokens[:100]) == [4] * 100
    assert cache.stats()["pages_free"] == 4


def test_a_request_that_cannot_fit_alone_fails_and_the_rest_goes_on():
    cache, scheduler = make(num_pages=2, max_batch_tokens=256, chunk_size=256)
    big = scheduler.submit([1] * 100, 100)       # 200 tokens need 4 pages, the pool has 2
    small = scheduler.submit([2] * 10, 5)
    seen = drive(scheduler, cache)
    assert big.finished and big.error and "pages" in big.error and [e[2] for e in seen[big.id]] == [EVENT_ERROR]
    assert small.generated == expected_tokens([2] * 10, 5)
    assert cache.stats()["pages_free"] == 2


def test_prefills_that_block_each_other_are_untangled():
    # two prompts of 150 tokens need 3 pages each, the pool has 4: the second must give way
    cache, scheduler = make(num_pages=4, max_batch_tokens=128, chunk_size=64)
    a = scheduler.submit([1] * 150, 4)
    b = scheduler.submit([2] * 150, 4)
    drive(scheduler, cache)
    assert a.generated == expected_tokens([1] * 150, 4) and b.generated == expected_tokens([2] * 150, 4)
    assert a.preemptions == 0


def test_live_limit_and_slots_bound_admission():
    cache, scheduler = make(num_pages=64, max_requests=2, max_batch_tokens=64, chunk_size=8)
    requests = [scheduler.submit([i + 1] * 4, 3) for i in range(5)]
    log = []
    drive(scheduler, cache, log=log)
    assert max(len({s.request.id for s in p.segments}) for p in log) <= 2
    assert all(r.generated == expected_tokens(r.prompt, 3) for r in requests)
    order = [r.id for p in log for r in p.admitted]
    assert order == sorted(order)                # first come, first admitted


def test_cancel_frees_everything():
    cache, scheduler = make()
    a = scheduler.submit([1] * 70, 50)
    b = scheduler.submit([2] * 5, 50)
    for _ in range(3):
        plan = scheduler.schedule()
        scheduler.complete(plan, {s.request.id: oracle(s.request.tokens) for s in plan.segments if s.wants_logits})
    assert scheduler.cancel(a.id) and scheduler.cancel(b.id) and not scheduler.cancel(12345)
    plan = scheduler.schedule()
    events = scheduler.complete(plan, {})
    assert sorted(e[0] for e in events if e[2] == EVENT_FINISHED) == [a.id, b.id]
    assert not scheduler.has_work() and cache.stats()["pages_free"] == 8 and cache.slots.free_count == 4


def test_a_plain_decode_step_goes_through_arrays_and_decides_the_same():
    """plan_next / fill_decode / complete_ordered against schedule / complete: the same requests
    driven both ways produce the same tokens, events and block tables at every step; a step that
    is not one token per request (a prompt portion, an admission) is refused and read as objects."""
    import numpy as np
    prompts = [[3, 1, 4, 1, 5], [9, 2, 6], [5, 3, 5, 8, 9, 7, 9, 3, 2, 3, 8]]
    results = []
    for arrays in (False, True):
        cache, scheduler = make(num_pages=8, max_requests=4, max_batch_tokens=64, chunk_size=8)
        for prompt in prompts:
            scheduler.submit(prompt, 20, GREEDY)
        log = []
        stride = 3
        while scheduler.has_work():
            counts = scheduler.plan_next()
            rows = counts[0]
            tokens, positions, slots = (np.full(rows, -7, dtype=np.int32) for _ in range(3))
            tables = np.full((1, rows, stride), -7, dtype=np.int32)
            filled = scheduler.fill_decode(rows, tokens, positions, slots, stride, tables, rows * stride) if arrays else -1
            plain = rows and counts[0] == counts[1] and not any(counts[2:6])
            if arrays:
                assert (filled == rows) == bool(plain)
            plan = scheduler.read_plan(counts)
            if filled == rows:
                # what the arrays hold is what the objects say
                assert tokens.tolist() == [s.tokens[0] for s in plan.segments]
                assert positions.tolist() == [s.request.computed for s in plan.segments]
                assert slots.tolist() == [cache.slot_of(s.request.id) for s in plan.segments]
                expected = cache.block_table_rows(0, [s.request.id for s in plan.segments], stride=stride)
                assert tables[0].tolist() == expected.tolist()
                drawn = np.asarray([oracle(s.request.tokens) for s in plan.segments], dtype=np.int32)
                events = scheduler.complete_ordered(drawn)
            else:
                assert (tokens == -7).all() and (tables == -7).all(), "a refused plan writes nothing"
                sampled = {s.request.id: oracle(s.request.tokens) for s in plan.segments if s.wants_logits}
                events = scheduler.complete(plan, sampled)
            log.append(events)
            cache.check_invariants()
        results.append((log, {r.id: r.generated for r in scheduler.requests.values()}))
    assert results[0] == results[1]
    assert any(len(events) >= 3 and all(kind == EVENT_TOKEN for _, _, kind in events) for events in results[1][0])


def drive_with_failures(scheduler, cache, refuses, max_steps=1000):
    """``drive`` with a step function that fails: ``refuses(segment)`` true means the step would
    refuse that segment before anything ran, as a check of the entries does. The request at fault
    is failed, the rest of the plan runs."""
    seen = {}
    steps = 0
    while scheduler.has_work():
        plan = scheduler.schedule()
        for segment in list(plan.segments):
            if refuses(segment):
                assert scheduler.fail(segment.request.id, f"refused at {segment.request.computed}")
                plan.segments.remove(segment)
                plan.failed.append(segment.request)
        for segment in plan.segments:       # the others' reservations stand
            r = segment.request
            assert r.live and cache.pages_missing(r.id, r.computed + len(segment.tokens)) == {0: 0}
        sampled = {s.request.id: oracle(s.request.tokens) for s in plan.segments if s.wants_logits}
        for event in scheduler.complete(plan, sampled):
            seen.setdefault(event[0], []).append(event)
        cache.check_invariants()
        steps += 1
        assert steps < max_steps
    return seen


@pytest.mark.parametrize("fails_at", [0, 16, 37])
def test_one_request_that_fails_leaves_the_others_running(fails_at):
    """Three requests, the middle one fails in its first portion, in its second, or while it decodes:
    it ends with one error event and gives everything back, the other two produce what they
    produce alone."""
    cache, scheduler = make(num_pages=8, max_requests=4, max_batch_tokens=48, chunk_size=16)
    first = scheduler.submit(list(range(30)), 6)
    bad = scheduler.submit(list(range(5, 40)), 6)
    last = scheduler.submit(list(range(7, 20)), 6)
    seen = drive_with_failures(scheduler, cache, lambda s: s.request is bad and s.request.computed + len(s.tokens) > fails_at)
    assert [kind for _, _, kind in seen[bad.id] if kind != EVENT_PREFILL] == [EVENT_TOKEN] * (3 if fails_at == 37 else 0) + [EVENT_ERROR]
    assert bad.finished and not bad.live and "refused at" in bad.error
    assert not scheduler.fail(bad.id, "again")          # it has ended already
    assert first.generated == expected_tokens(list(range(30)), 6)
    assert last.generated == expected_tokens(list(range(7, 20)), 6)
    assert [kind for _, _, kind in seen[first.id]][-1] == EVENT_FINISHED
    assert cache.stats()["pages_free"] == 8 and cache.stats()["slots_free"] == 4 and not cache.requests


def test_a_whole_step_that_fails_ends_its_requests_and_the_queue_goes_on():
    cache, scheduler = make(num_pages=8, max_requests=2, max_batch_tokens=64, chunk_size=32)
    a, b = scheduler.submit([1] * 20, 3), scheduler.submit([2] * 20, 3)
    waiting = scheduler.submit([3] * 20, 3)             # no slot for it yet
    plan = scheduler.schedule()
    assert [s.request for s in plan.segments] == [a, b]
    for segment in plan.segments:                       # the step failed while it ran
        scheduler.fail(segment.request.id, "the step failed")
    plan.failed.extend(s.request for s in plan.segments)
    plan.segments = []
    events = scheduler.complete(plan, {})
    assert sorted(events) == [(a.id, 0, EVENT_ERROR), (b.id, 0, EVENT_ERROR)]
    cache.check_invariants()
    seen = drive(scheduler, cache)
    assert waiting.generated == expected_tokens([3] * 20, 3) and cache.stats()["pages_free"] == 8


def test_a_failure_between_two_plans_is_not_lost():
    cache, scheduler = make(num_pages=8, max_requests=2)
    a, b = scheduler.submit([1] * 5, 3), scheduler.submit([2] * 5, 3)
    plan = scheduler.schedule()
    scheduler.complete(plan, {a.id: oracle(a.tokens), b.id: oracle(b.tokens)})
    assert scheduler.fail(b.id, "gone")                 # no plan is outstanding
    seen = drive(scheduler, cache)
    assert [e for e in seen[b.id]] == [(b.id, 0, EVENT_ERROR)]
    assert a.generated == expected_tokens([1] * 5, 3)
    assert scheduler.forget(b.id) and b.id not in scheduler.requests and not scheduler.forget(b.id)


def test_steps_ahead_of_the_host_and_requests_that_end_in_the_middle_of_them():
    """What a turn of several decode steps relies on: how many steps may follow a plain decode plan
    (room in the context, tokens to go for at least one request, no place for anybody who waits),
    that a request which ends on the way (a stop token, its last token) is missing from the plans
    after it while the others keep their rows' order, and that held plans admit nobody."""
    import numpy as np
    cache, scheduler = make(num_pages=16, max_requests=3)
    prompts = [[3, 4, 5], [9, 8], [20, 21, 22, 23]]
    # the second request will stop at the third token it draws, the third has seven tokens to draw
    stop = expected_tokens(prompts[1], 3)[2]
    assert stop not in expected_tokens(prompts[1], 2)
    budgets = [30, 30, 7]
    requests = [scheduler.submit(p, n, stop_tokens=[stop] if i == 1 else []) for i, (p, n) in enumerate(zip(prompts, budgets))]
    plan = scheduler.schedule()                         # the prompts
    scheduler.complete(plan, {s.request.id: oracle(s.request.tokens) for s in plan.segments})
    late = scheduler.submit([1, 2], 4)                  # every slot is taken: it waits
    counts = scheduler.plan_next()                      # a plain decode plan of three rows
    assert counts[0] == counts[1] == 3 and not any(counts[2:6])
    ahead, rows = scheduler.steps_ahead(7, 3)
    assert ahead == 7 and list(rows[:3]) == [r.id for r in requests]
    assert scheduler.steps_ahead(100, 3)[0] == 30 - 1 - 1   # the longest budget: one token drawn, one by this plan
    # the device runs the turn on whoever ends on the way; the host then hands the steps over in order
    sequences = [list(p) + expected_tokens(p, 1) for p in prompts]
    live = [True, True, True]
    scheduler.hold_admissions(7)
    for step in range(1 + 7):
        if step:
            counts = scheduler.plan_next()
            assert counts[0] == counts[1] == sum(live) and not any(counts[2:6]), "nobody is admitted while the turn is handed over"
        drawn = [oracle(sequence) for sequence in sequences]
        for sequence, token in zip(sequences, drawn):
            sequence.append(token)                      # every row goes on, whether its request still lives or not
        events = scheduler.complete_ordered(np.array([t for t, alive in zip(drawn, live) if alive], dtype=np.int32))
        owners = [e[0] for e in events if e[2] == EVENT_TOKEN]
        assert owners == [r.id for r, alive in zip(requests, live) if alive], "the rows keep their order"
        for e in events:
            if e[2] == EVENT_FINISHED:
                live[[r.id for r in requests].index(e[0])] = False
        cache.check_invariants()
    scheduler.hold_admissions(0)
    assert live == [True, False, False] and not late.live
    assert requests[1].generated == expected_tokens(prompts[1], 30, stop=(stop,)) and len(requests[1].generated) == 3
    assert requests[2].generated == expected_tokens(prompts[2], 7)
    assert requests[0].generated == expected_tokens(prompts[0], 9)
    # the hold is over: who waited comes in, and while there is a place for somebody no steps run ahead
    another = scheduler.submit([5, 6], 4)
    counts = scheduler.plan_next()
    assert counts[4] == 2 and late.live and another.live and scheduler.steps_ahead(4, 3)[0] == 0


def test_a_turn_whose_later_plan_differs_ends_its_requests_and_nobody_else():
    """``complete_turn`` hands a turn of decode steps that ran ahead over to the scheduler. If
    the plan the scheduler makes for a later step is not the step that ran (here: a request is
    cancelled between the turn's run and its handing over), the requests still live in the
    turn end with an error (their state on the device is ahead of the scheduler's lengths),
    everything they held comes back, the tokens handed over before are kept, and whoever
    waited goes on afterwards. A turn whose plans agree gives the events of its single steps,
    and the budgets that bound a turn's reservations are the tokens each request has to go."""
    import numpy as np
    cache, scheduler = make(num_pages=16, max_requests=3)
    prompts = [[3, 4, 5], [9, 8], [20, 21, 22, 23]]
    requests = [scheduler.submit(p, n) for p, n in zip(prompts, (30, 3, 30))]
    plan = scheduler.schedule()
    scheduler.complete(plan, {s.request.id: oracle(s.request.tokens) for s in plan.segments})
    late = scheduler.submit([1, 2], 4)                  # every slot is taken: it waits
    sequences = [list(p) + expected_tokens(p, 1) for p in prompts]

    def turn(steps):
        """What the device would draw in ``steps`` steps of all three rows."""
        drawn = np.zeros((steps, 3), dtype=np.int32)
        for step in range(steps):
            for row, sequence in enumerate(sequences):
                drawn[step, row] = oracle(sequence)
                sequence.append(int(drawn[step, row]))
        return drawn

    # a turn that goes through: the second request ends on its third token, in the turn's second step
    counts = scheduler.plan_next()
    assert counts[0] == counts[1] == 3 and not any(counts[2:6])
    assert scheduler.plan_budgets(3).tolist() == [30 - 2, 3 - 2, 30 - 2]
    ahead, rows = scheduler.steps_ahead(3, 3)
    assert ahead == 3
    events, differing = scheduler.complete_turn(turn(4), list(rows[:3]))
    assert differing is None
    assert [e[0] for e in events if e[2] == EVENT_TOKEN] == [1, 2, 3, 1, 2, 3, 1, 3, 1, 3]
    assert (requests[1].id, 3, EVENT_FINISHED) in events and not late.live
    cache.check_invariants()
    # the next turn: one slot is free now, so the scheduler would admit; a turn only starts when it says so
    counts = scheduler.plan_next()
    assert counts[4] == 1 and late.live
    plan = scheduler.read_plan(counts)
    scheduler.complete(plan, {s.request.id: oracle(s.request.tokens) for s in plan.segments if s.wants_logits})
    for sequence, request in zip(sequences, requests):
        if not request.finished:
            sequence[:] = request.tokens
    # a turn of the three running requests, one of which is cancelled while the device runs ahead
    counts = scheduler.plan_next()
    assert counts[0] == counts[1] == 3 and not any(counts[2:6])
    ahead, rows = scheduler.steps_ahead(3, 3)
    assert ahead == 3 and list(rows[:3]) == [requests[0].id, requests[2].id, late.id]
    sequences = [requests[0].tokens, requests[2].tokens, late.tokens]
    drawn = turn(4)
    before = {r.id: len(r.generated) for r in (requests[0], requests[2], late)}
    assert scheduler.cancel(requests[2].id)
    events, differing = scheduler.complete_turn(drawn, list(rows[:3]))
    assert differing is not None and not differing.segments
    # the first step's tokens were handed over as drawn; then the plans parted
    assert [e for e in events if e[2] == EVENT_TOKEN] == [(requests[0].id, int(drawn[0, 0]), EVENT_TOKEN),
                                                            (requests[2].id, int(drawn[0, 1]), EVENT_TOKEN),
                                                            (late.id, int(drawn[0, 2]), EVENT_TOKEN)]
    events = scheduler.complete(differing, {})
    kinds = {e[0]: e[2] for e in events}
    assert kinds == {requests[0].id: EVENT_ERROR, late.id: EVENT_ERROR, requests[2].id: EVENT_FINISHED}
    assert "ran ahead" in requests[0].error and "ran ahead" in late.error and requests[2].error is None
    assert all(len(r.generated) == before[r.id] + 1 for r in (requests[0], requests[2], late))
    assert not scheduler.has_work() and len(cache.requests) == 0
    assert cache.groups[0].pool.in_use == 0 and cache.slots.free_count == 3
    cache.check_invariants()
    # the scheduler is as good as new
    fresh = scheduler.submit([7, 7, 7], 5)
    seen = drive(scheduler, cache)
    assert [e[1] for e in seen[fresh.id] if e[2] == EVENT_TOKEN] == expected_tokens([7, 7, 7], 5)
