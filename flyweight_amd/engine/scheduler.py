"""The scheduler: which tokens of which requests run in the next step.

Continuous batching with prompts cut into portions. Each step, under a token budget:
every running request that has one token left to feed (a decode) contributes that row;
the rest of the budget goes to prompt portions, oldest request first, then to admitting
waiting requests while a slot, the live limit and the pages for a first portion allow. A
request's tokens are ``prompt + generated``; ``computed`` of them are in the cache, and the
logits of the last one are asked for exactly when a portion reaches the end, so a prompt's
last portion and a decode row are the same case.

When pages run out for a decode row, the most recently admitted request is preempted: its
pages and slot are freed and it goes back to the front of the waiting queue keeping its
generated tokens, to be recomputed later (logits do not depend on how tokens are cut into
steps, so it continues as if nothing had happened). The oldest request is never preempted; a
request that cannot fit alone ends with an error. The reference has no pages to run out of
(a slot reserves the whole context, native/src/v2_runtime.cpp:33578-33609) and visits tasks
round-robin, one prompt chunk or one token per visit (:33730-33787).

The decisions are made by the host library (C++, ``csrc/host/scheduler.hpp``) on the cache's
own bookkeeping; this file is its Python face: it keeps what only Python needs of a request
(sampling configuration, random stream) and turns plans and events into objects. It decides;
it runs nothing.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .. import host
from ..cache import CacheManager
from ..sampling import GREEDY, SamplingConfig, make_rng

# event kinds, as the reference numbers them (native/include/flyweight_v2.h:413-417)
EVENT_TOKEN, EVENT_FINISHED, EVENT_ERROR, EVENT_PREFILL = 0, 1, 2, 3
MAX_QUEUED = 256        # native/src/v2_runtime.cpp:32588-32591


class SchedulerError(ValueError):
    pass


class Request:
    """A request as Python sees it: what was submitted, and a view of its progress, which the
    host library keeps."""

    def __init__(self, scheduler: "Scheduler", request_id: int, prompt: List[int], max_new_tokens: int,
                 sampling: SamplingConfig, stop_tokens: Tuple[int, ...]):
        self._scheduler = scheduler
        self.id = request_id
        self.prompt = prompt
        self.max_new_tokens = max_new_tokens
        self.sampling = sampling
        self.stop_tokens = stop_tokens
        self.rng = make_rng(sampling.seed, request_id)

    def _info(self) -> List[int]:
        out = host.ints(9)
        scheduler = self._scheduler
        if scheduler._lib.fwh_request_info(scheduler._native, self.id, out) < 0:
            raise SchedulerError(host.last_error())
        return list(out)

    computed = property(lambda self: self._info()[0])       # tokens whose keys/values/state are in the cache
    live = property(lambda self: bool(self._info()[1]))
    finished = property(lambda self: bool(self._info()[2]))
    cancelled = property(lambda self: bool(self._info()[3]))
    admitted_at = property(lambda self: self._info()[4])    # admission counter: larger = more recent
    preemptions = property(lambda self: self._info()[5])

    @property
    def generated(self) -> List[int]:
        scheduler = self._scheduler
        count = self._info()[7]
        out = host.ints(count)
        scheduler._lib.fwh_request_generated(scheduler._native, self.id, out, count)
        return list(out[:count])

    @property
    def error(self) -> Optional[str]:
        scheduler = self._scheduler
        text = scheduler._lib.fwh_request_error(scheduler._native, self.id).decode("utf-8", "replace")
        return text or None

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.generated

    @property
    def remaining(self) -> int:
        info = self._info()
        return info[6] + info[7] - info[0]

    def __repr__(self) -> str:
        return f"Request({self.id}, prompt of {len(self.prompt)}, max_new_tokens={self.max_new_tokens})"


@dataclass
class PlannedSegment:
    request: Request
    tokens: Sequence[int]       # a piece of the plan's int32 array
    wants_logits: bool


@dataclass
class StepPlan:
    segments: List[PlannedSegment] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)
    admitted: List[Request] = field(default_factory=list)
    cancelled: List[Request] = field(default_factory=list)
    num_tokens: int = 0
    serial: int = 0         # plans are completed in the order they were made, each once


class Scheduler:
    def __init__(self, cache: CacheManager, max_positions: int, max_batch_tokens: int = 2048,
                 chunk_size: int = 512, max_live: Optional[int] = None, vocab_size: Optional[int] = None):
        """``vocab_size``: token ids of prompts and stop tokens are checked against it when a
        request is submitted (None: the vocabulary is not known here and nothing is checked)."""
        if max_batch_tokens < 1 or chunk_size < 1:
            raise SchedulerError("max_batch_tokens and chunk_size must be positive")
        self.cache = cache
        self.max_positions = max_positions
        self.max_batch_tokens = max_batch_tokens
        self.chunk_size = chunk_size
        self.max_live = min(max_live or cache.max_requests, cache.max_requests)
        self.requests: Dict[int, Request] = {}
        self._lib = host.library()
        self._native = self._lib.fwh_scheduler_create(cache.native_handle, max_positions, max_batch_tokens, chunk_size,
                                                      self.max_live, MAX_QUEUED, int(vocab_size or 0))
        if not self._native:
            raise SchedulerError(host.last_error())
        self._serial = 0
        self._drawing = set()       # unfinished requests whose tokens are drawn, not taken as the most likely

    def __del__(self):
        if getattr(self, "_native", None):
            self._lib.fwh_scheduler_destroy(self._native)
            self._native = None

    # ----- submitting -------------------------------------------------------------------
    def submit(self, prompt: Sequence[int], max_new_tokens: int, sampling: SamplingConfig = GREEDY,
               stop_tokens: Sequence[int] = ()) -> Request:
        """Validation as the reference's task submit (native/src/v2_runtime.cpp:32502-32520):
        a prompt, room for prompt + output in the context, a bounded queue."""
        prompt = [int(t) for t in prompt]
        stop = tuple(int(t) for t in stop_tokens)
        request_id = self._lib.fwh_scheduler_submit(self._native, (ctypes.c_int * max(len(prompt), 1))(*prompt), len(prompt),
                                                    int(max_new_tokens), (ctypes.c_int * max(len(stop), 1))(*stop), len(stop))
        if request_id < 0:
            raise SchedulerError(host.last_error())
        request = Request(self, request_id, prompt, int(max_new_tokens), sampling, stop)
        self.requests[request_id] = request
        if not sampling.greedy:
            self._drawing.add(request_id)
        return request

    def cancel(self, request_id: int) -> bool:
        if request_id not in self.requests:
            return False
        return bool(self._lib.fwh_scheduler_cancel(self._native, int(request_id)))

    def fail(self, request_id: int, message: str) -> bool:
        """Ends one request with an error: it gives back what it holds and leaves the plan made
        last (whose other segments stand); its error event comes out of that plan's completion.
        False if it has ended already."""
        if request_id not in self.requests:
            return False
        status = self._lib.fwh_scheduler_fail(self._native, int(request_id), str(message).encode("utf-8", "replace"))
        if status < 0:
            raise SchedulerError(host.last_error())
        return bool(status)

    def forget(self, request_id: int) -> bool:
        """Drops the record of a request that has ended (its prompt, its output, its error text)."""
        request = self.requests.get(request_id)
        if request is None or not self._lib.fwh_scheduler_forget(self._native, int(request_id)):
            return False
        del self.requests[request_id]
        self._drawing.discard(request_id)
        return True

    def has_work(self) -> bool:
        return bool(self._lib.fwh_scheduler_has_work(self._native))

    @property
    def preemptions(self) -> int:
        return self._lib.fwh_scheduler_preemptions(self._native)

    def _queue(self, which: int) -> List[Request]:
        count = self._lib.fwh_scheduler_queue(self._native, which, host.ids(0), 0)
        out = host.ids(count)
        self._lib.fwh_scheduler_queue(self._native, which, out, count)
        return [self.requests[out[i]] for i in range(count)]

    waiting = property(lambda self: self._queue(0))
    running = property(lambda self: self._queue(1))         # in admission order, oldest first

    # ----- planning ---------------------------------------------------------------------
    def schedule(self) -> StepPlan:
        """Plans the next step and reserves its pages. The slots of the requests admitted in it
        start at zero."""
        return self.read_plan(self.plan_next())

    # The two halves of ``schedule``, for a caller that can serve a plain decode step without
    # an object per request: ``plan_next`` makes the plan in the host library and says how large
    # it is; ``fill_decode`` writes such a step's batch straight into a captured step's upload
    # buffer and ``complete_ordered`` finishes it; ``read_plan`` gives any plan as objects.
    def plan_next(self):
        """Plans the next step (pages reserved); returns its counts: segments, tokens,
        preempted, failed, admitted, cancelled, and the most tokens its block tables cover."""
        counts = host.ints(7)
        if self._lib.fwh_scheduler_schedule(self._native, counts) < 0:
            raise SchedulerError(host.last_error())
        self._serial += 1
        return counts

    @property
    def all_greedy(self) -> bool:
        return not self._drawing

    def fill_decode(self, capacity: int, tokens, positions, slots, table_stride: int, tables, group_stride: int) -> int:
        """If the plan made last is one token for each of its requests and nothing else, writes
        the step's tokens, positions, slots and block-table rows to these int32 arrays (numpy
        views of a pinned buffer) and returns the number of rows; -1 otherwise."""
        rows = self._lib.fwh_plan_fill_decode(self._native, int(capacity), tokens.ctypes.data, positions.ctypes.data,
                                              slots.ctypes.data, int(table_stride),
                                              tables.ctypes.data if tables is not None else None, int(group_stride))
        if rows == host.NOT_DECODE_ONLY:
            return -1
        if rows < 0:
            raise SchedulerError(host.last_error())
        return rows

    def hold_admissions(self, plans: int) -> None:
        """The next ``plans`` plans admit nobody (the steps they stand for have already run, with
        the requests that were running); 0 ends the hold."""
        self._lib.fwh_scheduler_hold_admissions(self._native, int(plans))

    def plan_requests(self, rows: int, tokens: Optional[int] = None):
        """The requests (ids) of the plan made last, in the order of its ``rows`` segments, which
        hold ``tokens`` tokens together (default: one each)."""
        owners, lengths, wants, flat = host.ids(rows), host.ints(rows), host.ints(rows), host.ints(tokens or rows)
        self._lib.fwh_plan_segments(self._native, owners, lengths, wants, flat)
        return owners

    def steps_ahead(self, limit: int, rows: int):
        """For a plain decode plan: how many further steps of this batch may run before the host
        looks again (no place for a waiting request right now, room in the context for every
        request, tokens to go for at least one), at most ``limit``. Requests that end on the way
        (a stop token, their last token) are missing from the plans after it. And the plan's
        requests (their ids) in row order."""
        requests = host.ids(rows)
        ahead = self._lib.fwh_plan_steps_ahead(self._native, int(limit), requests, rows)
        if ahead < 0:
            raise SchedulerError(host.last_error())
        return ahead, requests

    def plan_budgets(self, rows: int) -> np.ndarray:
        """For each of the ``rows`` segments of the plan made last: how many tokens its request may
        still generate after the one this plan gives it (int32)."""
        out = host.ints(rows)
        made = self._lib.fwh_plan_budgets(self._native, out, rows)
        if made != rows:
            raise SchedulerError(host.last_error() if made < 0 else f"the plan has {made} segments, not {rows}")
        return np.frombuffer(out, dtype=np.int32, count=rows)

    def complete_ordered(self, tokens) -> List[Tuple[int, int, int]]:
        """``complete`` for the plan made last, the tokens (int32 numpy array) in the order of
        its segments that wanted logits."""
        self._serial += 1
        count = int(tokens.shape[0])
        capacity = 2 * count + 1
        event_owner, event_value, event_kind = host.ids(capacity), host.ints(capacity), host.ints(capacity)
        made = self._lib.fwh_scheduler_complete_ordered(self._native, tokens.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), count,
                                                        event_owner, event_value, event_kind, capacity)
        if made < 0:
            raise SchedulerError(host.last_error())
        return self._events(event_owner, event_value, event_kind, made)

    TURN_DIFFERS = "the scheduler's plan differs from the decode steps that ran ahead of it"

    def complete_turn(self, tokens, row_requests: Sequence[int]):
        """Finishes a turn of decode steps that ran back to back on the device: ``tokens`` int32
        [steps, at least the plan's rows], ``row_requests`` the ids of the plan made last in row
        order. The first step's tokens complete that plan; for every further step the scheduler
        makes the plan it ran by (admitting nobody: whoever waits comes in with the next turn) and
        takes its tokens. A request that ended on the way (a stop token, its last token) is
        missing from the later plans, the others keep their order; what its row went on to draw is
        dropped. Returns (events, None).

        If a later plan is not the step that ran (somebody was cancelled or gave way meanwhile),
        the requests still live in the turn end with an error: their fixed-size state on the
        device is several tokens ahead of the scheduler's lengths and cannot be wound back. The
        rest of that plan stands; it is returned for the caller to run: (events, plan)."""
        rows = len(row_requests)
        events = self.complete_ordered(np.ascontiguousarray(tokens[0][:rows]))
        live = np.ones(rows, dtype=bool)
        checked = 0
        self.hold_admissions(len(tokens) - 1)
        try:
            for later in tokens[1:]:
                ended = {task for task, _, kind in events[checked:] if kind in (EVENT_FINISHED, EVENT_ERROR)}
                checked = len(events)
                if ended:
                    live &= np.array([request not in ended for request in row_requests], dtype=bool)
                going = int(live.sum())
                if going == 0:
                    break
                again = self.plan_next()
                if again[0] != going or again[1] != going or any(again[2:6]):
                    plan = self.read_plan(again)
                    ahead = [request for request, alive in zip(row_requests, live) if alive]
                    for request in ahead:
                        if self.fail(request, self.TURN_DIFFERS):
                            plan.failed.append(self.requests[request])
                    plan.segments = [s for s in plan.segments if s.request.id not in set(ahead)]
                    plan.preempted = [r for r in plan.preempted if r.id not in set(ahead)]
                    return events, plan
                events.extend(self.complete_ordered(np.ascontiguousarray(later[:rows][live])))
        finally:
            self.hold_admissions(0)
        return events, None

    def _events(self, owners, values, kinds, count: int) -> List[Tuple[int, int, int]]:
        events = list(zip(owners[:count], values[:count], kinds[:count]))
        if self._drawing:
            for owner, _, kind in events:
                if kind in (1, 2):
                    self._drawing.discard(owner)
        return events

    def read_plan(self, counts) -> StepPlan:
        """The plan made last (by ``plan_next``) as objects."""
        segments, tokens = counts[0], counts[1]
        plan = StepPlan(num_tokens=tokens, serial=self._serial)
        if segments:
            owners, lengths, wants = host.ids(segments), host.ints(segments), host.ints(segments)
            # a segment's tokens are a piece of one int32 array: a prompt portion has thousands, and a
            # Python object for each would cost the step more than its smaller kernels
            flat, at = np.empty(max(tokens, 1), dtype=np.int32), 0
            self._lib.fwh_plan_segments(self._native, owners, lengths, wants, flat.ctypes.data_as(ctypes.POINTER(ctypes.c_int)))
            for i in range(segments):
                plan.segments.append(PlannedSegment(self.requests[owners[i]], flat[at:at + lengths[i]], bool(wants[i])))
                at += lengths[i]
        for which, target in enumerate((plan.preempted, plan.failed, plan.admitted, plan.cancelled)):
            if counts[2 + which]:
                out = host.ids(counts[2 + which])
                self._lib.fwh_plan_list(self._native, which, out)
                target.extend(self.requests[out[i]] for i in range(counts[2 + which]))
        cache = self.cache
        for request in plan.admitted:
            if request.id in cache.requests:
                cache.start_slot(cache.slot_of(request.id))
        return plan

    # ----- after the step ---------------------------------------------------------------
    def complete(self, plan: StepPlan, sampled: Dict[int, int]) -> List[Tuple[int, int, int]]:
        """``sampled``: request id -> token drawn from the logits of its last row. Returns
        events (request id, token or progress, kind)."""
        if plan.serial != self._serial:
            raise SchedulerError("only the plan made last can be completed, and only once")
        self._serial += 1
        wanting = [s.request.id for s in plan.segments if s.wants_logits]
        missing = [r for r in wanting if r not in sampled]
        if missing:
            raise KeyError(missing[0])
        owners = (ctypes.c_int64 * max(len(wanting), 1))(*wanting)
        drawn = (ctypes.c_int * max(len(wanting), 1))(*[int(sampled[r]) for r in wanting])
        capacity = 2 * len(plan.segments) + len(plan.failed) + len(plan.cancelled) + 1
        event_owner, event_value, event_kind = host.ids(capacity), host.ints(capacity), host.ints(capacity)
        count = self._lib.fwh_scheduler_complete(self._native, owners, drawn, len(wanting), event_owner, event_value,
                                                 event_kind, capacity)
        if count < 0:
            raise SchedulerError(host.last_error())
        return self._events(event_owner, event_value, event_kind, count)
