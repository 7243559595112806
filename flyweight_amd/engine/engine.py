"""The Python entry point, in the manner of the reference's binding: a ``Model`` opened
from a folder and a ``Runtime`` over it (``V2Model`` / ``V2QwenRuntime``,
src/flyweight/v2.py:2188-2440,3297-4029). Method names and meanings follow the reference
where it has them: ``prepare``, ``decode``, ``generate(prompt, max_tokens, callback)``,
``task_submit``, ``engine_step`` -> [(task id, token, kind)], ``task_cancel``,
``task_error``, ``reset``, ``info``, ``close``. ``step`` (logits of a mixed batch) has no
counterpart there: the reference returns tokens, never logits.
"""

from __future__ import annotations

import time
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import OutOfPages
from ..sampling import GREEDY, SamplingConfig, pack_settings, sample_rows
from .model import CausalLM, load_model, parse_dtype
from .scheduler import (EVENT_ERROR, EVENT_FINISHED, EVENT_PREFILL, EVENT_TOKEN, Request, Scheduler,
                        SchedulerError)
from .step import StepEntry, StepError, Stepper

PAGE_SIZE = 64
MAX_KEPT_ERRORS = 1024


class EngineError(RuntimeError):
    pass


class Model:
    """A model folder (config.json + safetensors) loaded onto the GPU."""

    def __init__(self, path: str, dtype="bfloat16", device: str = "cuda:0"):
        self.path = path
        self.dtype = parse_dtype(dtype)
        self.config, self.model = load_model(path, dtype=self.dtype, device=device)

    @classmethod
    def random(cls, config, seed: int = 0, dtype="bfloat16", device: str = "cuda:0", scale: str = "small") -> "Model":
        """A model of ``config`` (a registered architecture's configuration) with random
        weights drawn on the device; nothing is written to disk."""
        from ..kernels import ops
        from ..weights import random_tensors_on_device
        from .model import CausalLM
        self = cls.__new__(cls)
        self.path, self.dtype, self.config = None, parse_dtype(dtype), config
        target = torch.device(device)
        if target.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError("flyweight_amd runs on a GPU only (no CPU path); no HIP device is available")
        ops.library()
        self.model = CausalLM(config.model_spec())
        self.model.bind(random_tensors_on_device(self.model.tensors(), seed, target, self.dtype, scale), self.dtype, target)
        return self

    @property
    def spec(self):
        return self.model.spec

    def tensors(self) -> Dict[str, Tuple[Tuple[int, ...], str]]:
        return {name: (decl.shape, decl.role) for name, decl in self.model.tensors().items()}

    def native_runtime(self, **options) -> "Runtime":
        return Runtime(self, **options)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


class Runtime:
    def __init__(self, model: Model, context_limit: Optional[int] = None, parallel_sequences: int = 16,
                 num_pages: Optional[int] = None, max_batch_tokens: int = 2048, prefill_rows: int = 512,
                 decode_steps_per_turn: int = 1):
        """``context_limit``: most tokens (prompt + output) of one request, at most the
        model's ``max_position_embeddings``. ``parallel_sequences``: most requests live at
        once. ``num_pages``: cache pages (of 64 tokens) per page group; by default enough
        for every live request at the full context. ``prefill_rows``: most tokens of one
        prompt portion; ``max_batch_tokens``: most tokens of one step. ``decode_steps_per_turn``:
        when every running request decodes, takes the most likely token and can neither stop nor
        be joined by another (no stop tokens, budget left, nobody waiting), up to this many decode
        steps run back to back on the device before the host is asked again; ``engine_step`` then
        returns the events of all of them. More throughput, tokens in bursts."""
        self.model = model
        spec = model.spec
        self.context_limit = min(context_limit or spec.max_positions, spec.max_positions)
        self.parallel_sequences = max(1, int(parallel_sequences))
        per_request = (self.context_limit + PAGE_SIZE - 1) // PAGE_SIZE
        self.num_pages = int(num_pages) if num_pages else per_request * self.parallel_sequences
        self.max_batch_tokens = int(max_batch_tokens)
        self.prefill_rows = int(prefill_rows)
        self.decode_steps_per_turn = max(1, int(decode_steps_per_turn))
        self.stepper: Optional[Stepper] = None
        self.scheduler: Optional[Scheduler] = None
        self._errors: Dict[int, str] = {}           # task -> text, the last MAX_KEPT_ERRORS of them
        self._outputs: Dict[int, List[int]] = {}    # live task -> tokens so far
        self._collecting: Optional[Dict[int, List[int]]] = None
        self._held_events: List[Tuple[int, int, int]] = []
        self._decode_request: Optional[Hashable] = None
        self._counters = {"decode_calls": 0, "decode_ns": 0, "prefill_calls": 0, "prefill_tokens": 0, "prefill_ns": 0,
                          "steps": 0}

    # ----- lifetime ---------------------------------------------------------------------
    def prepare(self) -> "Runtime":
        if self.stepper is None:
            self.stepper = Stepper(self.model.model, num_pages=self.num_pages, max_requests=self.parallel_sequences,
                                   page_size=PAGE_SIZE, context_limit=self.context_limit)
            self.scheduler = Scheduler(self.stepper.cache, max_positions=self.context_limit,
                                       max_batch_tokens=self.max_batch_tokens, chunk_size=self.prefill_rows,
                                       max_live=self.parallel_sequences, vocab_size=self.model.spec.vocab_size)
        return self

    def reset(self) -> None:
        """Forget every request and give all cache memory back (state slots are zeroed
        again when next handed out)."""
        self.prepare()
        for request in list(self.stepper.cache.requests):
            self.stepper.cache.release(request)
        self.scheduler = Scheduler(self.stepper.cache, max_positions=self.context_limit,
                                   max_batch_tokens=self.max_batch_tokens, chunk_size=self.prefill_rows,
                                   max_live=self.parallel_sequences, vocab_size=self.model.spec.vocab_size)
        self._decode_request = None
        self._errors.clear()
        self._outputs.clear()
        self._held_events = []

    def close(self) -> None:
        self.stepper = None
        self.scheduler = None

    def __enter__(self):
        return self.prepare()

    def __exit__(self, *exc):
        self.close()
        return False

    # ----- logits -----------------------------------------------------------------------
    def admit(self, request: Hashable) -> None:
        self.prepare().stepper.admit(request)

    def release(self, request: Hashable) -> None:
        self.stepper.release(request)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """One mixed batch -> float32 logits [wanted, vocab] on the device."""
        return self.prepare().stepper.step(entries)

    # ----- single sequence, as the reference's decode(token) -> token ---------------------
    def decode(self, token: int) -> int:
        """Feeds one token to the runtime's own sequence and returns the greedy next token."""
        self.prepare()
        if self._decode_request is None:
            self._decode_request = ("decode", id(self))
            self.stepper.admit(self._decode_request)
        began = time.perf_counter_ns()
        logits = self.stepper.step([StepEntry(self._decode_request, [int(token)], [0])])
        token = sample_rows(logits, [GREEDY], [None])[0]
        self._counters["decode_calls"] += 1
        self._counters["decode_ns"] += time.perf_counter_ns() - began
        return token

    # ----- tasks ------------------------------------------------------------------------
    def task_submit(self, prompt: Sequence[int], max_tokens: int, stop_tokens: Sequence[int] = (),
                    temperature: float = 0.0, top_k: int = 20, top_p: float = 0.95, min_p: float = 0.0,
                    seed: Optional[int] = None) -> int:
        """Queues a request and returns its task id. Refused here, before it takes a place: an
        empty prompt, ``max_tokens`` < 1, prompt + ``max_tokens`` beyond the context, a token id
        or stop token outside the vocabulary, sampling settings out of range, a full queue."""
        self.prepare()
        sampling = SamplingConfig(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p, seed=seed)
        try:
            return self.scheduler.submit(prompt, max_tokens, sampling, stop_tokens).id
        except SchedulerError as error:
            raise EngineError(str(error)) from None

    def task_cancel(self, task_id: int) -> bool:
        return self.scheduler.cancel(task_id)

    def task_error(self, task_id: int) -> Optional[str]:
        return self._errors.get(task_id)

    def engine_step(self) -> List[Tuple[int, int, int]]:
        """One step of everything that can move: returns (task id, token or progress, kind)
        with kind 0 token, 1 finished, 2 error, 3 prefill progress. A request that the step
        refuses, or that took part in a step that failed while it ran, ends with an error event
        (its text in ``task_error``) and gives back what it held; the others go on, as the
        reference isolates a task's failure (native/src/v2_runtime.cpp:33788-33797)."""
        self.prepare()
        held, self._held_events = self._held_events, []
        if not self.scheduler.has_work():
            return held
        events = self._advance()
        self._note(events)
        return held + events if held else events

    def _advance(self) -> List[Tuple[int, int, int]]:
        scheduler = self.scheduler
        counts = scheduler.plan_next()
        # A plain decode step (one token for every request of the plan, every token the most likely
        # one, nothing else happened) that a captured step serves goes from the scheduler's plan to
        # the upload buffer and back without an object per request.
        if counts[0] and counts[0] == counts[1] and not any(counts[2:6]):
            captured = self.stepper.planned_decode(counts[0], counts[6] + self.decode_steps_per_turn - 1)
            if captured is not None:
                began = time.perf_counter_ns()
                settings_of = None if scheduler.all_greedy else self._sampling_of
                try:
                    ran = self.stepper.replay_planned(captured, scheduler, self.decode_steps_per_turn, settings_of)
                except Exception as error:
                    return self._fail_step(scheduler.read_plan(counts), error)
                if ran is not None:
                    tokens, row_requests, moved_on = ran
                    if moved_on is not None:
                        # the generators have drawn on the device: the requests' own copies follow
                        for request, state in zip(row_requests, moved_on.tolist()):
                            drawing = scheduler.requests[request]
                            if not drawing.sampling.greedy:
                                drawing.rng.state = state
                    self._counters["steps"] += len(tokens)
                    self._counters["decode_calls"] += counts[0] * len(tokens)
                    self._counters["decode_ns"] += time.perf_counter_ns() - began
                    events, differing = scheduler.complete_turn(tokens, row_requests)
                    if differing is None:
                        return events
                    # a later plan was not the step that ran: the turn's requests have ended with an
                    # error; what else that plan holds runs now
                    self._counters["failed_steps"] = self._counters.get("failed_steps", 0) + 1
                    return events + self._run_plan(differing)
        return self._run_plan(scheduler.read_plan(counts))

    def _run_plan(self, plan) -> List[Tuple[int, int, int]]:
        """Runs a plan's segments as one step through the step function and completes it."""
        scheduler = self.scheduler
        sampled: Dict[int, int] = {}
        while plan.segments:
            entries = [StepEntry(s.request.id, s.tokens, [len(s.tokens) - 1] if s.wants_logits else [])
                       for s in plan.segments]
            began = time.perf_counter_ns()
            try:
                logits = self.stepper.step(entries)
                wanting = [s.request for s in plan.segments if s.wants_logits]
                if wanting:
                    tokens = sample_rows(logits, [r.sampling for r in wanting], [r.rng for r in wanting])
                    sampled = {r.id: t for r, t in zip(wanting, tokens)}
            except StepError as error:
                # Found before anything ran or changed: the request at fault leaves, the rest of the
                # plan stands (its pages stay reserved) and runs without it.
                at_fault = [s for s in plan.segments if s.request.id == error.request]
                if not at_fault:
                    return self._fail_step(plan, error)
                scheduler.fail(error.request, str(error))
                plan.failed.append(at_fault[0].request)
                plan.segments = [s for s in plan.segments if s.request.id != error.request]
                continue
            except Exception as error:
                return self._fail_step(plan, error)
            elapsed = time.perf_counter_ns() - began
            self._counters["steps"] += 1
            prompt_tokens = sum(len(s.tokens) for s in plan.segments if len(s.tokens) > 1)
            if prompt_tokens:
                self._counters["prefill_calls"] += 1
                self._counters["prefill_tokens"] += prompt_tokens
                self._counters["prefill_ns"] += elapsed
            else:
                self._counters["decode_calls"] += len(plan.segments)
                self._counters["decode_ns"] += elapsed
            break
        return scheduler.complete(plan, sampled)

    def _sampling_of(self, row_requests, settings, states) -> None:
        """Fills what the device sampler reads for the rows of a decode plan."""
        requests = [self.scheduler.requests[request] for request in row_requests]
        pack_settings([r.sampling for r in requests], [r.rng for r in requests], self.model.spec.vocab_size, settings, states)

    def _fail_step(self, plan, error: Exception) -> List[Tuple[int, int, int]]:
        """A step failed while it ran (or for a reason that names no request): what the cache
        holds of the requests that took part cannot be trusted any more (fixed-size state is
        updated in place), so each of them ends with an error and gives back its pages and slot.
        Requests that were not in the step are untouched and go on with the next one."""
        text = f"the step failed: {type(error).__name__}: {error}"
        for segment in plan.segments:
            self.scheduler.fail(segment.request.id, text)
            plan.failed.append(segment.request)
        plan.segments = []
        self._counters["failed_steps"] = self._counters.get("failed_steps", 0) + 1
        return self.scheduler.complete(plan, {})

    def _note(self, events: List[Tuple[int, int, int]]) -> None:
        """Keeps what the runtime itself needs of new events: the output so far of live tasks
        (for ``run``), the error text of tasks that failed; and lets the scheduler forget a task
        once its last event is on its way to the caller, so that a long-lived runtime does not
        grow with every task it has served."""
        scheduler = self.scheduler
        for task, value, kind in events:
            if kind == EVENT_TOKEN:
                self._outputs.setdefault(task, []).append(value)
            elif kind in (EVENT_FINISHED, EVENT_ERROR):
                tokens = self._outputs.pop(task, [])
                if self._collecting is not None:
                    self._collecting[task] = tokens
                if kind == EVENT_ERROR:
                    request = scheduler.requests.get(task)
                    self._errors[task] = (request.error if request is not None else None) or "failed"
                    while len(self._errors) > MAX_KEPT_ERRORS:
                        self._errors.pop(next(iter(self._errors)))
                scheduler.forget(task)

    # ----- blocking generation ------------------------------------------------------------
    def generate(self, prompt: Sequence[int], max_tokens: int,
                 callback: Optional[Callable[[int], Optional[bool]]] = None, **sampling) -> List[int]:
        """Generates up to ``max_tokens`` tokens after ``prompt``; ``callback(token)`` is
        called for each and stops the generation by returning False (as the reference's
        generate, src/flyweight/v2.py:3837-3876). Greedy unless sampling settings are given.
        Events of other tasks that move meanwhile are kept for the next ``engine_step``."""
        task = self.task_submit(prompt, max_tokens, **sampling)
        produced: List[int] = []
        while True:
            events = self.engine_step()
            self._held_events.extend(event for event in events if event[0] != task)
            for task_id, value, kind in events:
                if task_id != task:
                    continue
                if kind == EVENT_TOKEN:
                    produced.append(value)
                    if callback is not None and callback(value) is False:
                        # Tokens of the same turn that lie behind this one are dropped.
                        self.task_cancel(task)
                        return produced
                elif kind == EVENT_ERROR:
                    raise EngineError(self.task_error(task) or "generation failed")
                elif kind == EVENT_FINISHED:
                    return produced
            if not self.scheduler.has_work():
                return produced

    def run(self) -> Dict[int, List[int]]:
        """Steps until every submitted task has ended; returns task id -> generated tokens for
        the tasks that ended meanwhile (a failed task: what it had generated; its text is in
        ``task_error``). Events are not handed out."""
        self.prepare()
        self._collecting = {}
        try:
            while self.scheduler.has_work():
                self.engine_step()
            return self._collecting
        finally:
            self._collecting = None
            self._held_events = []

    # ----- counters ---------------------------------------------------------------------
    @property
    def info(self) -> Dict[str, int]:
        data = dict(self._counters)
        if self.stepper is not None:
            data.update(self.stepper.cache.stats())
            data["preemptions"] = self.scheduler.preemptions
        from ..kernels import ops
        if ops.kernel_profile_active():
            # per kernel entry point: calls, GPU and host-launch milliseconds (FLYWEIGHT_KERNEL_PROFILE=1)
            data["kernels"] = ops.kernel_profile_report()
        return data
