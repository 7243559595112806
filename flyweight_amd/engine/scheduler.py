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

This file decides; it runs nothing. It needs only the cache manager's bookkeeping.
"""

from __future__ import annotations

import collections
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache import CacheManager
from ..sampling import GREEDY, SamplingConfig, make_rng

# event kinds, as the reference numbers them (native/include/flyweight_v2.h:413-417)
EVENT_TOKEN, EVENT_FINISHED, EVENT_ERROR, EVENT_PREFILL = 0, 1, 2, 3
MAX_QUEUED = 256        # native/src/v2_runtime.cpp:32588-32591


class SchedulerError(ValueError):
    pass


@dataclass
class Request:
    id: int
    prompt: List[int]
    max_new_tokens: int
    sampling: SamplingConfig = GREEDY
    stop_tokens: Tuple[int, ...] = ()
    generated: List[int] = field(default_factory=list)
    computed: int = 0               # tokens whose keys/values/state are in the cache
    live: bool = False
    finished: bool = False
    cancelled: bool = False
    error: Optional[str] = None
    admitted_at: int = -1           # admission counter: larger = more recent
    preemptions: int = 0
    rng: object = None

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.generated

    def tokens_from(self, first: int, count: int) -> List[int]:
        """tokens[first:first + count] without joining the two lists."""
        end, split = first + count, len(self.prompt)
        if end <= split:
            return self.prompt[first:end]
        if first >= split:
            return self.generated[first - split:end - split]
        return self.prompt[first:] + self.generated[:end - split]

    @property
    def remaining(self) -> int:
        return len(self.prompt) + len(self.generated) - self.computed


@dataclass
class PlannedSegment:
    request: Request
    tokens: List[int]
    wants_logits: bool


@dataclass
class StepPlan:
    segments: List[PlannedSegment] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)
    admitted: List[Request] = field(default_factory=list)
    cancelled: List[Request] = field(default_factory=list)
    num_tokens: int = 0
    _planned: set = field(default_factory=set)      # ids of the requests that have a segment

    def add(self, segment: PlannedSegment) -> None:
        self.segments.append(segment)
        self.num_tokens += len(segment.tokens)
        self._planned.add(segment.request.id)

    def drop(self, request: Request) -> None:
        if request.id not in self._planned:
            return
        self.num_tokens -= sum(len(s.tokens) for s in self.segments if s.request is request)
        self.segments = [s for s in self.segments if s.request is not request]
        self._planned.discard(request.id)

    def has(self, request: Request) -> bool:
        return request.id in self._planned


class Scheduler:
    def __init__(self, cache: CacheManager, max_positions: int, max_batch_tokens: int = 2048,
                 chunk_size: int = 512, max_live: Optional[int] = None):
        if max_batch_tokens < 1 or chunk_size < 1:
            raise SchedulerError("max_batch_tokens and chunk_size must be positive")
        self.cache = cache
        self.max_positions = max_positions
        self.max_batch_tokens = max_batch_tokens
        self.chunk_size = chunk_size
        self.max_live = min(max_live or cache.max_requests, cache.max_requests)
        self.waiting: Deque[Request] = collections.deque()
        self.running: List[Request] = []        # in admission order, oldest first
        self.requests: Dict[int, Request] = {}
        self._next_id = 1
        self._admissions = 0
        self.preemptions = 0

    # ----- submitting -------------------------------------------------------------------
    def submit(self, prompt: Sequence[int], max_new_tokens: int, sampling: SamplingConfig = GREEDY,
               stop_tokens: Sequence[int] = ()) -> Request:
        """Validation as the reference's task submit (native/src/v2_runtime.cpp:32502-32520):
        a prompt, room for prompt + output in the context, a bounded queue."""
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise SchedulerError("the prompt is empty")
        if max_new_tokens < 1:
            raise SchedulerError("max_tokens must be at least 1")
        if len(prompt) + max_new_tokens > self.max_positions:
            raise SchedulerError(f"prompt ({len(prompt)}) + max_tokens ({max_new_tokens}) exceeds the context "
                                 f"of {self.max_positions}")
        if len(self.waiting) >= MAX_QUEUED:
            raise SchedulerError(f"the queue holds {MAX_QUEUED} requests already")
        request = Request(id=self._next_id, prompt=prompt, max_new_tokens=int(max_new_tokens), sampling=sampling,
                          stop_tokens=tuple(int(t) for t in stop_tokens))
        request.rng = make_rng(sampling.seed, request.id)
        self._next_id += 1
        self.requests[request.id] = request
        self.waiting.append(request)
        return request

    def cancel(self, request_id: int) -> bool:
        request = self.requests.get(request_id)
        if request is None or request.finished:
            return False
        request.cancelled = True
        return True

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ----- planning ---------------------------------------------------------------------
    def _evict(self, request: Request) -> None:
        self.cache.release(request.id)
        request.live = False
        request.computed = 0
        self.running.remove(request)

    def _fail(self, request: Request, message: str, plan: StepPlan) -> None:
        if request.live:
            self._evict(request)
        request.error = message
        request.finished = True
        plan.failed.append(request)

    def _preempt(self, victim: Request, plan: StepPlan) -> None:
        plan.drop(victim)
        self._evict(victim)
        victim.preemptions += 1
        self.preemptions += 1
        self.waiting.appendleft(victim)
        plan.preempted.append(victim)

    def _fits(self, request: Request, new_length: int) -> bool:
        cache = self.cache
        if cache.pages_for(new_length) > cache.max_pages_per_request:
            return False
        return all(cache.groups[g].pool.free_count >= n for g, n in cache.pages_missing(request.id, new_length).items())

    def schedule(self) -> StepPlan:
        plan = StepPlan()
        # cancelled requests leave first
        for request in [r for r in self.running if r.cancelled]:
            self._evict(request)
            request.finished = True
            plan.cancelled.append(request)
        for request in [r for r in self.waiting if r.cancelled]:
            self.waiting.remove(request)
            request.finished = True
            plan.cancelled.append(request)
        while True:
            self._plan_once(plan)
            if plan.segments or not self.running:
                return plan
            # every running request waits for pages and none can move
            if len(self.running) == 1:
                self._fail(self.running[0], "out of cache pages: the request does not fit even alone", plan)
            else:
                self._preempt(self.running[-1], plan)

    def _plan_once(self, plan: StepPlan) -> None:
        cache = self.cache
        planned = plan.has

        # 1. decode rows, oldest first; make room by preempting the newest
        for request in list(self.running):
            if not request.live or request.remaining != 1 or planned(request):
                continue
            if plan.num_tokens >= self.max_batch_tokens:
                break
            while request.live and not self._fits(request, request.computed + 1):
                if len(self.running) == 1:
                    self._fail(request, "out of cache pages: the request does not fit even alone", plan)
                else:
                    self._preempt(self.running[-1], plan)       # may be the request itself, if it is the newest
            if not request.live:
                continue
            cache.reserve(request.id, request.computed + 1)
            plan.add(PlannedSegment(request, request.tokens_from(request.computed, 1), True))

        # 2. portions of prompts of running requests, oldest first
        for request in list(self.running):
            if request.remaining < 1 or planned(request):
                continue
            if plan.num_tokens >= self.max_batch_tokens:
                break
            self._plan_portion(request, plan)

        # 3. admissions, in queue order, while everything a first portion needs is there;
        #    none in a step in which somebody had to give way
        while (self.waiting and not plan.preempted and plan.num_tokens < self.max_batch_tokens
               and len(self.running) < self.max_live and cache.slots.free_count > 0):
            request = self.waiting[0]
            total = len(request.prompt) + request.max_new_tokens
            limit = min(cache.max_pages_per_request, cache.num_pages)
            if cache.groups and cache.pages_for(total) > limit:
                self.waiting.popleft()
                self._fail(request, f"the request needs {cache.pages_for(total)} cache pages for {total} tokens; "
                                    f"the pool holds {limit}", plan)
                continue
            portion = min(request.remaining, self.chunk_size, self.max_batch_tokens - plan.num_tokens)
            if any(group.pool.free_count < cache.pages_for(portion) for group in cache.groups):
                break
            self.waiting.popleft()
            cache.admit(request.id)
            request.live = True
            request.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(request)
            plan.admitted.append(request)
            self._plan_portion(request, plan)

    def _plan_portion(self, request: Request, plan: StepPlan) -> None:
        portion = min(request.remaining, self.chunk_size, self.max_batch_tokens - plan.num_tokens)
        # shrink to what the pool can hold right now; a portion may be cut anywhere
        while portion >= 1 and not self._fits(request, request.computed + portion):
            portion -= (request.computed + portion) % self.cache.page_size or self.cache.page_size
        if portion < 1:
            return
        self.cache.reserve(request.id, request.computed + portion)
        plan.add(PlannedSegment(request, request.tokens_from(request.computed, portion), portion == request.remaining))

    # ----- after the step ---------------------------------------------------------------
    def complete(self, plan: StepPlan, sampled: Dict[int, int]) -> List[Tuple[int, int, int]]:
        """``sampled``: request id -> token drawn from the logits of its last row. Returns
        events (request id, token or progress, kind)."""
        events: List[Tuple[int, int, int]] = []
        for request in plan.failed:
            events.append((request.id, 0, EVENT_ERROR))
        for request in plan.cancelled:
            events.append((request.id, len(request.generated), EVENT_FINISHED))
        for segment in plan.segments:
            request = segment.request
            request.computed += len(segment.tokens)
            self.cache.commit(request.id, request.computed)
            if not segment.wants_logits:
                events.append((request.id, request.computed, EVENT_PREFILL))
                continue
            token = int(sampled[request.id])
            request.generated.append(token)
            events.append((request.id, token, EVENT_TOKEN))
            done = (token in request.stop_tokens or len(request.generated) >= request.max_new_tokens
                    or len(request.prompt) + len(request.generated) >= self.max_positions)
            if done:
                self._evict(request)
                request.finished = True
                events.append((request.id, len(request.generated), EVENT_FINISHED))
        return events
