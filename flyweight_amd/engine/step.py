"""The step function: one batch of (request, its next tokens) through the model.

A step holds *segments*: a request's next ``n >= 1`` tokens, whether a portion of its
prompt or one decoded token. Any mix, cut anywhere. The step runs only the tokens it is
given, against the cache earlier steps left, appends to that cache, and returns float32
logits at the wanted places. The reference has three disjoint entry points instead (one
token -> argmax, native/src/v2_runtime.cpp:27525; R rows of one sequence without logits,
native/src/v2_mtp_verifier.inc:4086-4121) and never a mixed batch.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager, OutOfPages
from ..kernels import ops
from .model import CacheView, CausalLM


class StepError(ValueError):
    """What a step refuses, found before anything ran or changed. ``request`` names the entry
    at fault where there is one, so that a caller can leave that request out and run the rest."""

    def __init__(self, message: str, request: Hashable = None):
        super().__init__(message)
        self.request = request


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()       # places among ``tokens`` whose logits are asked for
    # What the position encodings see for these tokens, if not their places in the sequence
    # (the default): one non-negative number per token. Where a key lies in the cache and which
    # keys a row may see follow the order of the tokens whatever is given here.
    positions: Optional[Sequence[int]] = None


def check_entries(entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int, max_positions: int):
    """What a step may not bring: no entries, an unknown or repeated request, no tokens, a token
    outside the vocabulary, a place outside the entry, a sequence past the model's limit.
    Returns the requests' current lengths and slots (one call into the host library), the
    host library's ids of the requests, for the step's further calls, and the entries' tokens
    as int32 arrays (None for a step of single tokens)."""
    if not entries:
        raise StepError("a step needs at least one entry")
    requests = [entry.request for entry in entries]
    if len(set(requests)) != len(requests):
        seen = set()
        for request in requests:
            if request in seen:
                raise StepError(f"request {request!r} appears twice in one step", request)
            seen.add(request)
    natives = cache.natives_of(requests)
    try:
        lengths, slots = cache.describe(requests, natives)
    except KeyError as error:
        raise StepError(f"request {error.args[0]!r} was not admitted", error.args[0]) from None
    if all(len(entry.tokens) == 1 and entry.positions is None for entry in entries):
        # a decode step: the same checks without a loop over the entries' fields
        tokens = [entry.tokens[0] for entry in entries]
        if max(lengths) + 1 > max_positions:
            entry, start = next((e, s) for e, s in zip(entries, lengths) if s + 1 > max_positions)
            raise StepError(f"request {entry.request!r} would reach {start + 1} tokens; the context limit is {max_positions}", entry.request)
        if not (0 <= int(min(tokens)) and int(max(tokens)) < vocab_size):
            entry = next(e for e in entries if not 0 <= int(e.tokens[0]) < vocab_size)
            raise StepError(f"token id {entry.tokens[0]} of request {entry.request!r} is outside the vocabulary (0..{vocab_size - 1})", entry.request)
        for entry in entries:
            for place in entry.want:
                if int(place) != 0:
                    raise StepError(f"request {entry.request!r} wants logits at place {place} of 1 tokens", entry.request)
        return lengths, slots, natives, None
    arrays = []         # each entry's tokens as one int32 array: made once, the step's upload takes them as they are
    for entry, start in zip(entries, lengths):
        n = len(entry.tokens)
        if n < 1:
            raise StepError(f"request {entry.request!r} brings no tokens", entry.request)
        if start + n > max_positions:
            raise StepError(f"request {entry.request!r} would reach {start + n} tokens; the context limit is {max_positions}", entry.request)
        try:
            tokens = np.asarray(entry.tokens, dtype=np.int32)
            if n == 1:          # the decoded tokens beside a prompt's portion: no reduction for one number
                inside = tokens.ndim == 1 and 0 <= int(tokens[0]) < vocab_size
            else:
                inside = tokens.ndim == 1 and 0 <= int(tokens.min()) and int(tokens.max()) < vocab_size
        except (OverflowError, TypeError, ValueError):
            inside = False
        if not inside:
            bad = next((t for t in entry.tokens if not (isinstance(t, (int, np.integer)) and 0 <= int(t) < vocab_size)), entry.tokens[0])
            raise StepError(f"token id {bad} of request {entry.request!r} is outside the vocabulary (0..{vocab_size - 1})", entry.request)
        arrays.append(tokens)
        for place in entry.want:
            if not 0 <= int(place) < n:
                raise StepError(f"request {entry.request!r} wants logits at place {place} of {n} tokens", entry.request)
        if entry.positions is not None and (len(entry.positions) != n or min(entry.positions) < 0):
            raise StepError(f"request {entry.request!r} gives {len(entry.positions)} positions for {n} tokens, or a negative one",
                            entry.request)
    return lengths, slots, natives, arrays


class _Staging:
    """Pinned host memory that an eager step's index arrays pass through on their way to the
    device: the copy is queued and the host goes on to the step's launches (from pageable
    memory it would stand until the copy has run). One buffer serves every step: before it is
    written again the copy of the step before must have left it."""

    def __init__(self, device: torch.device):
        self.device = device
        self._host: Optional[torch.Tensor] = None
        self._numpy: Optional[np.ndarray] = None
        self._left = torch.cuda.Event()

    def upload(self, pieces: Sequence[np.ndarray]) -> torch.Tensor:
        total = sum(piece.size for piece in pieces)
        if self._host is None or self._host.numel() < total:
            if self._host is not None:
                self._left.synchronize()
            self._host = torch.empty(max(2 * total, 1 << 14), dtype=torch.int32, pin_memory=True)
            self._numpy = self._host.numpy()
        else:
            self._left.synchronize()
        np.concatenate(pieces, out=self._numpy[:total])
        packed = torch.empty(total, dtype=torch.int32, device=self.device)
        packed.copy_(self._host[:total], non_blocking=True)
        self._left.record()
        return packed


class StepContext:
    """The batch as the kernels see it: per-row and per-segment index arrays on the
    device (one upload), block tables per page group, per-step tables of the position
    encodings, and whatever index arrays the model's parts ask for (``Part.step_arrays``: built
    on the host from the batch, they travel in the same upload; a recorded step lets the parts
    bring theirs up to date before every replay, ``Part.refresh_step_arrays``)."""

    FIXED = 6       # tokens, positions, segment of each row, first row of each segment, slots, wanted rows

    def __init__(self, entries: Sequence[StepEntry], cache: CacheManager, device: torch.device, vocab_size: int,
                 max_positions: int, described=None, providers: Sequence = (), staging: Optional[_Staging] = None):
        """``described``: what ``check_entries`` returned if the caller has checked the entries
        already. ``providers``: the parts whose ``step_arrays`` this
        step's upload carries. ``staging``: the pinned memory the upload passes through, if the
        caller keeps some."""
        starts, slots, natives, arrays = described if described is not None else check_entries(entries, cache, vocab_size, max_positions)
        # per-row arrays are made by whole-array operations: a prompt portion has thousands of rows and
        # a step dozens of entries, and a Python loop over either would take longer than some kernels
        if arrays is None:
            arrays = [np.asarray(entry.tokens, dtype=np.int32) for entry in entries]
        counts = np.fromiter((array.size for array in arrays), dtype=np.int64, count=len(arrays))
        first_rows = np.zeros(len(arrays) + 1, dtype=np.int64)
        np.cumsum(counts, out=first_rows[1:])
        starts_array = np.asarray(starts, dtype=np.int64)
        tokens = np.concatenate(arrays)
        row_seg = np.repeat(np.arange(len(arrays), dtype=np.int32), counts)
        row_pos = (np.arange(len(tokens), dtype=np.int64) - np.repeat(first_rows[:-1] - starts_array, counts)).astype(np.int32)
        seg_row0: List[int] = first_rows.tolist()
        seg_slot: List[int] = list(slots)
        want_rows: List[int] = []
        for entry, row0 in zip(entries, seg_row0):
            if len(entry.want):
                want_rows.extend(row0 + int(place) for place in entry.want)
        self.requests: List[Hashable] = [entry.request for entry in entries]
        self.new_lengths: List[int] = (starts_array + counts).tolist()
        given_positions = any(entry.positions is not None for entry in entries)
        encoding_parts = []
        if given_positions:
            for entry, row0, count in zip(entries, seg_row0, counts.tolist()):
                encoding_parts.append(row_pos[row0:row0 + count] if entry.positions is None
                                      else np.asarray(entry.positions, dtype=np.int32))
        self.num_rows = len(tokens)
        self.num_segments = len(entries)
        self.num_wanted = len(want_rows)
        self.wants_every_row = want_rows == list(range(self.num_rows))      # in order: the logits' rows are the step's rows
        self.all_decode = self.num_rows == self.num_segments
        self.max_context = max(self.new_lengths)
        # segments of one token that a mixed step begins with (a scheduler puts the decoded tokens
        # first): mixers may give them to their decode kernels. Their rows are 0 .. n - 1.
        self.decode_prefix = 0 if self.all_decode else int(np.argmax(counts != 1))
        self.device = device
        # the same on the host, for parts that plan their work there
        self.host_row_pos = row_pos
        self.host_seg_row0 = seg_row0
        self.host_seg_slot = seg_slot

        tables = [cache.block_table_rows(g, self.requests, natives=natives) for g in range(len(cache.groups))]
        pieces = [np.asarray(a, dtype=np.int32) for a in (tokens, row_pos, row_seg, seg_row0, seg_slot, want_rows)]
        pieces += [t.reshape(-1) for t in tables]
        if given_positions:
            pieces.append(np.concatenate(encoding_parts))
        extra = self._ask(providers)
        pieces += [array for _, _, array in extra]
        packed = staging.upload(pieces) if staging is not None else torch.from_numpy(np.concatenate(pieces)).to(device)
        views = []
        offset = 0
        for piece in pieces:
            views.append(packed[offset:offset + piece.size])
            offset += piece.size
        self.token_ids, self.row_pos, self.row_seg, self.seg_row0, self.seg_slot, self.want_rows = views[:self.FIXED]
        self.block_tables = [v.view(t.shape) for v, t in zip(views[self.FIXED:], tables)]
        at = self.FIXED + len(tables)
        # what the position encodings see: the places in the sequences, unless the entries say otherwise
        self.encoding_pos = self.row_pos
        if given_positions:
            self.encoding_pos = views[at]
            at += 1
        self._arrays: Dict = {}
        for (key, name, _), view in zip(extra, views[at:]):
            self._arrays.setdefault(key, {})[name] = view
        self._position_tables: Dict = {}

    def _ask(self, providers: Sequence):
        """[(provider key, array name, int32 numpy array)] of every provider, in a fixed order."""
        asked = []
        for part in providers:
            key = part.step_arrays_key()
            for name, array in sorted(part.step_arrays(self).items()):
                asked.append((key, name, np.ascontiguousarray(array, dtype=np.int32).reshape(-1)))
        return asked

    def _refresh_parts(self) -> None:
        """A recorded step: the parts bring their own arrays up to date with this replay's
        positions and slots, in the pinned buffer that the upload takes."""
        for part, arrays in self._provider_arrays:
            part.refresh_step_arrays(self, arrays)

    def step_arrays(self, part) -> Dict[str, torch.Tensor]:
        """The device copies of what ``part.step_arrays`` built for this step. A part that was
        not among the step's providers gets them made now, with an upload of their own."""
        key = part.step_arrays_key()
        if key not in self._arrays:
            if getattr(self, "_provider_arrays", None) is not None:
                raise StepError("a recorded step holds only the arrays of the parts it was built with")
            self._arrays[key] = {name: torch.from_numpy(np.ascontiguousarray(array, dtype=np.int32)).to(self.device)
                                 for name, array in part.step_arrays(self).items()}
        return self._arrays[key]

    @classmethod
    def for_decode_graph(cls, batch: int, cache: CacheManager, device: torch.device, max_context: int,
                         table_stride: int, providers: Sequence = ()) -> "StepContext":
        """A context of ``batch`` single-token segments whose index arrays live in ONE
        persistent device buffer, refreshed before every replay of the captured step. The parts'
        own arrays are built once, for ``batch`` segments of one row each at position 0 (that fixes
        their sizes), and brought up to date by the parts before every upload
        (``Part.refresh_step_arrays``)."""
        self = cls.__new__(cls)
        self.num_rows = self.num_segments = self.num_wanted = batch
        self.wants_every_row = True
        self.all_decode = True
        self.decode_prefix = 0
        self.max_context = max_context          # bounds the split-key grid, not the result
        self.device = device
        groups = len(cache.groups)
        # what the parts' arrays are built from: ``batch`` segments of one row
        self.host_row_pos = np.zeros(batch, dtype=np.int32)
        self.host_seg_row0 = list(range(batch + 1))
        self.host_seg_slot = [0] * batch
        extra = self._ask(providers)
        sizes = [batch, batch, batch, batch + 1, batch, batch] + [batch * table_stride] * groups
        sizes += [array.size for _, _, array in extra]
        self.host_buffer = torch.empty(max(sum(sizes), 1), dtype=torch.int32, pin_memory=True)
        self.device_buffer = torch.zeros(max(sum(sizes), 1), dtype=torch.int32, device=device)
        views, host_views, offset = [], [], 0
        for size in sizes:
            views.append(self.device_buffer[offset:offset + size])
            host_views.append(self.host_buffer[offset:offset + size].numpy())
            offset += size
        self.token_ids, self.row_pos, self.row_seg, self.seg_row0, self.seg_slot, self.want_rows = views[:cls.FIXED]
        self.encoding_pos = self.row_pos
        self.block_tables = [v.view(batch, table_stride) for v in views[cls.FIXED:cls.FIXED + groups]]
        self._host = host_views
        self._host_tables = host_views[cls.FIXED:cls.FIXED + groups]
        self._table_stride = table_stride
        # what the parts see of a replay on the host: its positions and slots, where the upload takes them
        self.host_row_pos = host_views[1]
        self.host_seg_slot = host_views[4]
        # what never changes between replays
        rows = np.arange(batch, dtype=np.int32)
        host_views[1][:] = 0
        host_views[2][:] = rows
        host_views[3][:] = np.arange(batch + 1, dtype=np.int32)
        host_views[5][:] = rows
        self._arrays = {}
        by_part: Dict = {}
        for (key, name, array), view, host_view in zip(extra, views[cls.FIXED + groups:], host_views[cls.FIXED + groups:]):
            host_view[:] = array
            self._arrays.setdefault(key, {})[name] = view
            by_part.setdefault(key, {})[name] = host_view
        self._provider_arrays = [(part, by_part.get(part.step_arrays_key(), {})) for part in providers]
        self._position_tables = {}
        return self

    def refresh(self, entries: Sequence[StepEntry], cache: CacheManager, described=None) -> None:
        """Writes this step's tokens, positions, slots and block tables and uploads them."""
        host = self._host
        self.requests = [e.request for e in entries]
        if described is not None:
            starts, slots, natives = described[:3]
        else:
            natives = cache.natives_of(self.requests)
            starts, slots = cache.describe(self.requests, natives)
        self.wait_uploaded()
        self.new_lengths = [s + 1 for s in starts]
        host[0][:] = [int(e.tokens[0]) for e in entries]
        host[1][:] = starts
        host[4][:] = slots
        for g, rows in enumerate(self._host_tables):
            rows[:] = cache.block_table_rows(g, self.requests, stride=self._table_stride, natives=natives).reshape(-1)
        self._refresh_parts()
        self.upload()

    def wait_uploaded(self) -> None:
        """The pinned buffer is still being read until the last upload has run: wait for it
        before the buffer is written again."""
        uploaded = getattr(self, "_uploaded", None)
        if uploaded is not None:
            uploaded.synchronize()

    def upload(self) -> None:
        self.device_buffer.copy_(self.host_buffer, non_blocking=True)
        if getattr(self, "_uploaded", None) is None:
            self._uploaded = torch.cuda.Event()
        self._uploaded.record()

    def fill_from(self, scheduler, cache: CacheManager) -> int:
        """For a captured step: lets the scheduler write the plan it made last straight into the
        upload buffer (tokens, positions, slots, block tables) if that plan is one token for each
        of at most this step's number of requests and nothing else, and fills the rows behind them
        up; returns the plan's number of rows (the caller uploads). -1 (and nothing written) otherwise."""
        self.wait_uploaded()
        host = self._host
        tables = self._host_tables
        rows = scheduler.fill_decode(self.num_rows, host[0], host[1], host[4], self._table_stride,
                                     tables[0] if tables else None, self.num_rows * self._table_stride)
        if rows < 0:
            return -1
        self.fill_up(rows, cache)
        self._refresh_parts()
        return rows

    def fill_up(self, rows: int, cache: CacheManager) -> None:
        """Rows behind the plan's (a step recorded for more requests than the plan has): token 0
        at position 0 of nobody's sequence, in the cache's spare page and slot."""
        if rows == self.num_rows:
            return
        host = self._host
        host[0][rows:] = 0
        host[1][rows:] = 0
        host[4][rows:] = cache.spare_slot
        for group, table in enumerate(self._host_tables):
            table[rows * self._table_stride:] = cache.spare_pages[group]

    def position_tables(self, part):
        key = part.key()
        if key not in self._position_tables:
            self._position_tables[key] = part.tables(self)
        return self._position_tables[key]

    def cache_view(self, cache: CacheManager, entry):
        """What the mixer of schedule entry ``entry`` sees of the cache: the view its need class
        gives of the entry's storage (with this step's block-table rows, for a paged one)."""
        if entry.cache is None or entry.cache not in cache.needs:
            return CacheView(writes=False if entry.cache is None else entry.writes_cache)
        group = cache.entry_group.get(entry.cache)
        table = None if group is None else self.block_tables[group]
        return cache.view(entry.cache, table, entry.writes_cache)


class Stepper:
    """Owns the model's cache and runs steps. ``admit`` a request before its first step,
    ``release`` it when it ends."""

    def __init__(self, model: CausalLM, num_pages, max_requests: int, page_size: int = 64,
                 context_limit: Optional[int] = None):
        """``num_pages``: cache pages per page group, one number or a mapping by group
        (``CacheManager``). ``context_limit``: the most tokens one request may reach here, at most the model's
        own limit (the default). Block tables and everything sized by a sequence's length follow
        this number, not the model's: a model that allows 128,000 positions costs a run of 4,096
        no more than one that allows 4,096."""
        if not model.bound:
            raise StepError("the model has no weights yet")
        self.model = model
        self.device = model.device
        self.context_limit = min(int(context_limit or model.spec.max_positions), model.spec.max_positions)
        if self.context_limit < 1:
            raise StepError("the context limit must be positive")
        max_pages = (self.context_limit + page_size - 1) // page_size
        self.cache = CacheManager(model.cache_needs(), num_pages=num_pages, max_requests=max_requests,
                                  page_size=page_size, max_pages_per_request=max_pages, dtype=model.dtype,
                                  device=model.device)
        self.steps = 0
        self.tokens_run = 0
        self.providers = model.step_array_providers()      # parts whose index arrays travel with a step's upload
        self._staging = _Staging(self.device) if self.device.type == "cuda" else None
        # decode steps (every segment one token) are captured in a HIP graph per batch size and
        # context bucket and replayed, if every part of the model allows it
        self.use_graphs = all(block.graph_safe for block in model.layers) and model.final_norm.graph_safe
        self._graphs: Dict[tuple, "_CapturedDecode"] = {}
        self.graph_replays = 0

    def admit(self, request: Hashable) -> None:
        self.cache.admit(request)

    def release(self, request: Hashable) -> None:
        self.cache.release(request)

    def is_live(self, request: Hashable) -> bool:
        return request in self.cache.requests

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Returns float32 logits [wanted, vocab] on the device, rows in the order of the
        entries and of each entry's ``want`` (None if nothing is wanted). Raises StepError
        (naming the request at fault) or OutOfPages, having changed nothing, when an entry is
        refused or the cache cannot hold the new tokens."""
        cache = self.cache
        spec = self.model.spec
        described = check_entries(entries, cache, spec.vocab_size, self.context_limit)
        requests = [entry.request for entry in entries]
        new_lengths = [start + len(entry.tokens) for entry, start in zip(entries, described[0])]
        # reserve everything first so that a failure leaves no request half-served
        cache.reserve_all(requests, new_lengths, described[2])
        try:
            if self.use_graphs and not ops.kernel_profile_active() and all(len(entry.tokens) == 1 and entry.positions is None for entry in entries):
                return self._replay(self._decode_step(len(entries), max(new_lengths)), entries, described)
            ctx = StepContext(entries, cache, self.device, spec.vocab_size, self.context_limit, described=described,
                              providers=self.providers, staging=self._staging)
            logits = self.model.forward(ctx, cache)
        except BaseException:
            # The lengths stay where they were and the pages reserved for this step go back. What
            # the kernels that did run have written past those lengths is never read; fixed-size
            # state of the step's requests may have moved on, though: the caller has to release them.
            cache.drop_reservations(requests, described[2])
            raise
        cache.commit_all(ctx.requests, ctx.new_lengths, described[2])
        self.steps += 1
        self.tokens_run += ctx.num_rows
        return logits

    # ----- captured decode steps ----------------------------------------------------------
    def kept_pages(self, context: int) -> int:
        """The block-table width (pages) of the captured step that serves sequences of up to
        ``context`` tokens: the next power of two, at least one run of the split-key decode
        kernel, at most what the context limit needs. The split-key grid, the workspace of partial
        results and the uploaded block-table rows are sized by this, so a step costs what the live
        sequences need, and a request that grows past a bucket moves on to the next step recorded."""
        cache = self.cache
        pages = max(cache.pages_for(context), ops.DECODE_SPLIT_PAGES)
        bucket = 1 << (pages - 1).bit_length()
        return max(1, min(bucket, cache.max_pages_per_request))

    def _decode_step(self, batch: int, context: int) -> "_CapturedDecode":
        """The decode step of this many rows for sequences of up to ``context`` tokens (after the
        step), with its persistent index arrays."""
        pages = self.kept_pages(context)
        captured = self._graphs.get((batch, pages))
        if captured is None:
            cache = self.cache
            ctx = StepContext.for_decode_graph(batch, cache, self.device, max_context=pages * cache.page_size,
                                               table_stride=pages, providers=self.providers)
            captured = self._graphs[(batch, pages)] = _CapturedDecode(ctx)
        return captured

    @staticmethod
    def kept_batch(rows: int) -> int:
        """The size of the step that serves a scheduler's plan of ``rows`` decoded tokens: every
        size below 8 has a step of its own, beyond that multiples of 8 up to 64 and of 16 above
        (the sizes at which the products change kernels, 16 and 64, are among them). A serving
        run whose requests end one by one sees every batch size for a few steps only; recording
        a step for each would cost more than the rows that fill a step up."""
        if rows < 8:
            return rows
        multiple = 8 if rows <= 64 else 16
        return (rows + multiple - 1) // multiple * multiple

    def planned_decode(self, rows: int, context: int) -> Optional["_CapturedDecode"]:
        """The decode step that serves a scheduler's plan of ``rows`` single tokens whose
        sequences reach at most ``context`` tokens, or None where decode steps are not recorded."""
        return self._decode_step(self.kept_batch(rows), context) if self.use_graphs and not ops.kernel_profile_active() else None

    def _run(self, captured: "_CapturedDecode") -> None:
        """Runs the step whose index arrays have been uploaded; its logits are ``captured.logits``
        afterwards. The first time eagerly (kernels set their attributes and workspaces are
        allocated then, which a recording must not hold), the second time it is recorded (that
        runs nothing) and replayed, from then on replayed."""
        ctx = captured.ctx
        if captured.graph is None and not captured.ran:
            captured.ran = True
            ctx._position_tables = {}
            captured.logits = self.model.forward(ctx, self.cache)
            return
        if captured.graph is None:
            ctx._position_tables = {}           # the recording must hold the kernels that make them
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    captured.logits = self.model.forward(ctx, self.cache)
            torch.cuda.current_stream().wait_stream(side)
            captured.graph = graph
        captured.graph.replay()
        self.graph_replays += 1

    def replay_planned(self, captured: "_CapturedDecode", scheduler, steps: int = 1, settings_of=None):
        """Decode steps straight from the scheduler's plan (see ``StepContext.fill_from``): the
        pages are reserved by the plan and the lengths are committed when the scheduler completes
        it, so the cache manager is not asked again. Every token is the most likely one. With
        ``steps`` > 1 and a plan that is certain to repeat (``Scheduler.steps_ahead``), up to that
        many steps run back to back on the device (their pages reserved and their block tables
        uploaded before the first), each fed the tokens of the one before, and the host reads all
        of them at once: it is then asked once per turn instead of once per step. A request that
        draws one of its stop tokens on the way has run on regardless (its row costs nothing beside
        the others); the caller drops what it drew after it.
        Every token is the most likely one unless ``settings_of`` is given: called with the plan's
        requests in row order, it fills the sampling settings (float32 [rows, 4]) and generator
        states (uint64 [rows]) handed to it, and the tokens are drawn on the device.
        Returns (tokens, int32 [steps run, rows]; the plan's requests in row order; the generators'
        states after the turn, uint64 [rows], or None), or None if the plan is not a plain decode
        step (nothing has run then)."""
        ctx = captured.ctx
        cache = self.cache
        rows = ctx.fill_from(scheduler, cache)
        if rows < 0:
            return None
        ahead, natives = scheduler.steps_ahead(steps - 1, rows) if steps > 1 else (0, None)
        if natives is None or (settings_of is not None and not ahead):
            natives = scheduler.plan_requests(rows)       # (steps_ahead names them only when steps follow)
        sampling = None
        if settings_of is not None:
            sampling = captured.sampling_buffers(self.device)
            sampling.host_settings[:] = 0.0                 # the rows behind the plan's: greedy
            settings_of(list(natives[:rows]), sampling.host_settings[:rows], sampling.host_states[:rows])
            sampling.upload()
        if ahead:
            # Pages for all the steps of the turn now, and the block tables with them: a table that
            # already holds the page a later step will write to reads the same for the steps before.
            # A request whose last token comes earlier in the turn gets pages up to that token only:
            # its row runs on beside the others (that costs nothing), and what it then writes goes to
            # the spare page, which its table names behind the pages it holds.
            positions = ctx._host[1]
            stride = ctx._table_stride
            going = np.minimum(scheduler.plan_budgets(rows), ahead).astype(np.int64)     # further steps each row takes part in
            reach = positions[:rows].astype(np.int64) + 1 + going
            try:
                cache.reserve_all((), reach.tolist(), natives=natives, count=rows)
            except OutOfPages:
                ahead = 0                   # one step; the scheduler will decide who gives way
            else:
                ending = going < ahead
                for g in range(len(cache.groups)):
                    table = cache.block_table_rows(g, (), stride=stride, natives=natives, count=rows)
                    if ending.any():
                        held = (reach + cache.page_size - 1) // cache.page_size
                        behind = (np.arange(stride)[None, :] >= held[:, None]) & ending[:, None]
                        table[behind] = cache.spare_pages[g]
                    ctx._host_tables[g][:rows * stride] = table.reshape(-1)
        ctx.upload()
        # Nothing crosses to the host between the steps of a turn: the kernel that finds a step's most
        # likely tokens writes them to the turn's record and to the next step's token ids, and moves
        # every row's position on by one.
        drawn = torch.empty((ahead + 1, ctx.num_rows), dtype=torch.int32, device=self.device)
        def draw(step: int, **feed) -> None:
            if sampling is None:
                ops.argmax_rows(captured.logits, out=drawn[step], **feed)
            else:
                ops.sample_rows(captured.logits, sampling.settings, sampling.states, out=drawn[step], **feed)

        for step in range(ahead):
            self._run(captured)
            draw(step, also=ctx.token_ids, advance=ctx.row_pos)
        self._run(captured)
        draw(ahead)
        ran = ahead + 1
        self.steps += ran
        self.tokens_run += rows * ran
        tokens = drawn[:ran, :rows].cpu().numpy()
        moved_on = sampling.states[:rows].cpu().numpy().view(np.uint64) if sampling is not None else None
        return tokens, list(natives[:rows]), moved_on

    def _replay(self, captured: "_CapturedDecode", entries: Sequence[StepEntry], described=None) -> Optional[torch.Tensor]:
        cache = self.cache
        ctx = captured.ctx
        ctx.refresh(entries, cache, described)
        self._run(captured)
        cache.commit_all(ctx.requests, ctx.new_lengths, None if described is None else described[2])
        self.steps += 1
        self.tokens_run += ctx.num_rows
        # one row of logits for every wanted place, as the eager path gives them (an entry of one
        # token may name its place more than once)
        wanted = [i for i, entry in enumerate(entries) for _ in entry.want]
        if not wanted:
            return None
        if wanted == list(range(len(entries))):
            return captured.logits          # overwritten by the next replay of this batch size
        return captured.logits[wanted]


class _SamplingBuffers:
    """What the device sampler reads for a captured step's rows: settings float32 [rows, 4] and
    generator states int64 [rows], on the device and in one pinned buffer on the host."""

    def __init__(self, rows: int, device):
        self._host = torch.zeros(3 * rows, dtype=torch.int64, pin_memory=True)
        self._device = torch.zeros(3 * rows, dtype=torch.int64, device=device)
        words = self._host.numpy()
        self.host_settings = words[:2 * rows].view(np.float32).reshape(rows, 4)
        self.host_states = words[2 * rows:].view(np.uint64)
        self.settings = self._device[:2 * rows].view(torch.float32).view(rows, 4)
        self.states = self._device[2 * rows:]

    def upload(self) -> None:
        self._device.copy_(self._host, non_blocking=True)


class _CapturedDecode:
    def __init__(self, ctx: StepContext):
        self.ctx = ctx
        self.graph = None
        self.logits = None
        self.ran = False            # whether the step has run eagerly once
        self._sampling = None

    def sampling_buffers(self, device) -> _SamplingBuffers:
        if self._sampling is None:
            self._sampling = _SamplingBuffers(self.ctx.num_rows, device)
        return self._sampling
