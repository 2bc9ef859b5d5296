"""Continuous batching above the step function.

Each scheduler step builds one batch: every running request that is decoding
brings its one token, requests still in their prompt bring a portion of it, and
waiting requests are admitted first come first served while the step's token
budget, the request slots and the free pages allow. A request whose portion ends
its known tokens gets logits, a token is selected, and it finishes on a stop
token or at its length. States and reasons are the reference's
(include/microllm/inference/scheduler.h:15-27); its continuous scheduler
(src/inference/scheduler.cpp:464-1069) prefills whole prompts of equal length
into fixed slots and reserves capacity up front, so it has neither a token budget
nor a way to run out of cache.

With ``lookahead`` a step does not wait for the tokens it selects: they stay on the device, the next step takes
them from there (``StepEntry.token_from``), and the host learns them one step late, while the GPU is already at
work on that next step; what the host must decide before then (who runs, who ends at its length, who gets
pages) needs only counts, not ids. A request with stop tokens is waited for as before.

When pages run out: the running request that was admitted last is preempted. Its
pages and slot go back, it returns to the head of the waiting queue, and when it
is admitted again its prompt and the tokens it had generated are run again in
portions (recomputation); sampling draws are indexed by the number of generated
tokens, so it continues with the same stream. A request that is alone and still
cannot get pages would never fit; ``submit`` refuses such a request.
"""
from __future__ import annotations

import enum
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence

from ..cache.pages import OutOfPages
from ..sampling import NonFiniteLogits, Sampler, SamplingParams
from .batch import StepEntry

NOT_YET = -1      # in Request.generated: a token that was selected on the device and has not reached the host


class RequestState(enum.Enum):
    PENDING_PREFILL = "pending_prefill"   # waiting, or admitted and still inside its known tokens
    DECODING = "decoding"
    COMPLETED = "completed"
    CANCELLED = "cancelled"


class CompletionReason(enum.Enum):
    NONE = "none"
    LENGTH = "length"
    STOP_TOKEN = "stop_token"
    CANCELLED = "cancelled"


@dataclass(eq=False)      # a request is itself: membership and removal go by identity, not by comparing prompts
class Request:
    id: int
    prompt: List[int]
    params: SamplingParams
    arrival_step: int
    state: RequestState = RequestState.PENDING_PREFILL
    completion_reason: CompletionReason = CompletionReason.NONE
    generated: List[int] = field(default_factory=list)
    computed: int = 0            # tokens of prompt + generated whose keys and values are in the cache
    admitted: bool = False
    admission_order: int = -1
    completion_step: int = -1
    preemptions: int = 0
    submit_time: float = 0.0
    first_token_time: float = -1.0
    completion_time: float = -1.0

    @property
    def known(self) -> int:
        return len(self.prompt) + len(self.generated)

    def token_at(self, index: int) -> int:
        return self.prompt[index] if index < len(self.prompt) else self.generated[index - len(self.prompt)]

    def tokens_between(self, start: int, stop: int) -> List[int]:
        """Tokens ``start`` to ``stop - 1`` of the prompt followed by what was generated."""
        length = len(self.prompt)
        if stop <= length:
            return self.prompt[start:stop]
        if start >= length:
            return self.generated[start - length:stop - length]
        return self.prompt[start:] + self.generated[:stop - length]

    @property
    def terminal(self) -> bool:
        return self.state in (RequestState.COMPLETED, RequestState.CANCELLED)


@dataclass
class SchedulerMetrics:
    scheduler_steps: int = 0
    submitted_requests: int = 0
    completed_requests: int = 0
    cancelled_requests: int = 0
    stop_completed_requests: int = 0
    admissions: int = 0
    preemptions: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    batched_tokens: int = 0
    engine_steps: int = 0
    peak_active_requests: int = 0
    peak_held_pages: int = 0
    failed_steps: int = 0


@dataclass(eq=False)
class Pending:
    """The tokens a step selected, still on their way to the host: for whom, where each lies in its request's
    ``generated``, and the selection to ask."""
    requests: List[Request]
    places: List[int]
    selection: object

    def row_of(self, request: Request) -> Optional[int]:
        for row, candidate in enumerate(self.requests):
            if candidate is request:
                return row
        return None


@dataclass(eq=False)
class Portion:
    """What one request brings to a step."""
    request: Request
    start: int
    count: int
    wants_logits: bool


class Scheduler:
    def __init__(self, engine, max_batched_tokens: int = 2048, prefill_chunk: int = 512,
                 max_requests: Optional[int] = None, sampler: Optional[Sampler] = None, lookahead: bool = False):
        if max_batched_tokens <= 0 or prefill_chunk <= 0:
            raise ValueError("max_batched_tokens and prefill_chunk must be positive")
        self.engine = engine
        self.cache = engine.cache
        self.max_batched_tokens = max_batched_tokens
        # a cache whose windowed groups were sized for portions of some length takes no longer ones
        self.prefill_chunk = min(prefill_chunk, getattr(self.cache, "max_portion", None) or prefill_chunk)
        self.max_requests = min(max_requests or self.cache.max_requests, self.cache.max_requests)
        self.sampler = sampler or Sampler()
        self.lookahead = lookahead
        self._pending: Optional[Pending] = None
        self.requests: Dict[int, Request] = {}
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []     # in admission order
        self.metrics = SchedulerMetrics()
        self.current_step = 0
        self._next_id = 0
        self._admissions = 0

    # ---- submitting ----------------------------------------------------------------------
    def submit(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
               arrival_step: Optional[int] = None) -> int:
        params = params or SamplingParams()
        vocab = self.engine.spec.vocab_size
        params.validate(vocab)
        prompt = [int(token) for token in prompt]
        if not prompt:
            raise ValueError("a prompt needs at least one token")
        for token in prompt:
            if not 0 <= token < vocab:
                raise ValueError(f"prompt token {token} is outside the vocabulary")
        total = len(prompt) + params.max_new_tokens
        if total > self.engine.spec.max_positions:
            raise ValueError(f"prompt plus max_new_tokens is {total}, beyond max positions {self.engine.spec.max_positions}")
        for group in self.cache.groups:
            if self.cache.most_blocks(group, total, self.prefill_chunk) > group.pool.num_pages:
                raise ValueError(f"prompt plus max_new_tokens is {total} tokens, more than the cache holds "
                                 f"({group.pool.num_pages * self.cache.page_size})")
        request = Request(self._next_id, prompt, params, arrival_step if arrival_step is not None else self.current_step,
                          submit_time=time.perf_counter())
        self._next_id += 1
        self.requests[request.id] = request
        self.metrics.submitted_requests += 1
        if params.max_new_tokens == 0:   # completes at once, src/inference/scheduler.cpp:876-881
            self._finish(request, CompletionReason.LENGTH)
        else:
            self.waiting.append(request)
        return request.id

    def cancel(self, request_id: int) -> bool:
        """Terminal and idempotent: False when the request had already ended (src/inference/scheduler.cpp:885-896)."""
        if request_id not in self.requests:
            raise KeyError(f"unknown request {request_id}")
        request = self.requests[request_id]
        if request.terminal:
            return False
        if request in self.running:
            self.running.remove(request)
            self._release(request)
        else:
            self.waiting.remove(request)
        request.state = RequestState.CANCELLED
        request.completion_reason = CompletionReason.CANCELLED
        request.completion_step = self.current_step
        request.completion_time = time.perf_counter()
        self.metrics.cancelled_requests += 1
        return True

    # ---- one step ------------------------------------------------------------------------
    def has_work(self) -> bool:
        return bool(self.running or self.waiting)

    def plan(self) -> List[Portion]:
        """Decide what this step runs. Takes pages (a reservation per portion); may preempt."""
        budget = self.max_batched_tokens
        portions: List[Portion] = []
        preempted_now = False

        def portion_of(request: Request, budget_left: int) -> int:
            remaining = request.known - request.computed
            return min(remaining, self.prefill_chunk if remaining > 1 else 1, budget_left)

        # Running requests first: decodes, then prompts that are under way, each in admission order.
        ordered = sorted(self.running, key=lambda r: (r.known - r.computed > 1, r.admission_order))
        for request in ordered:
            if request not in self.running:      # preempted while an earlier one was placed
                continue
            if budget <= 0:
                break
            count = portion_of(request, budget)
            while True:
                try:
                    self.cache.reserve(self.cache.get(request.id), count)
                    break
                except OutOfPages:
                    victim = self.running[-1]
                    was_planned = [p for p in portions if p.request is victim]
                    for planned in was_planned:
                        portions.remove(planned)
                        budget += planned.count
                    self._preempt(victim)
                    preempted_now = True
                    if victim is request:
                        count = 0
                        break
            if count > 0:
                portions.append(Portion(request, request.computed, count, request.computed + count == request.known))
                budget -= count

        # Then admissions, first come first served; a request that does not fit stops the queue. None in a step
        # that had to preempt: the victim is first in the queue, and a small portion of it would fit the pages it
        # has just given back, only for the next page an older request needs to throw it out again, its prompt
        # recomputed from the first token each time. It waits for a step in which the running ones find room.
        while self.waiting and budget > 0 and len(self.running) < self.max_requests and not preempted_now:
            request = self.waiting[0]
            if request.arrival_step > self.current_step:
                break
            count = portion_of(request, budget)
            if request.preemptions > 0 and not self._room_for_all_of(request):
                break
            handle = self.cache.open(request.id)
            try:
                self.cache.reserve(handle, count)
            except OutOfPages:
                self.cache.close(request.id)
                break
            self.waiting.popleft()
            request.admitted = True
            request.admission_order = self._admissions
            self._admissions += 1
            self.metrics.admissions += 1
            self.running.append(request)
            portions.append(Portion(request, request.computed, count, request.computed + count == request.known))
            budget -= count
        return portions

    def _room_for_all_of(self, request: Request) -> bool:
        """Whether the free pages hold everything the request has to run again and its next token. A request that
        was preempted comes back only then: admitted into less, it would recompute a part of its prompt and be
        thrown out again by the next page an older request needs."""
        if not self.running:
            return True      # alone it fits: submit saw to that
        return all(self.cache.most_blocks(group, request.known + 1, self.prefill_chunk) <= group.pool.num_free
                   for group in self.cache.groups)

    def step(self) -> List[int]:
        """Run one batch; returns the ids of requests that got a token in this step."""
        portions = self.plan()
        self.metrics.scheduler_steps += 1
        self.metrics.peak_active_requests = max(self.metrics.peak_active_requests, len(self.running))
        if self.cache.groups:
            self.metrics.peak_held_pages = max(self.metrics.peak_held_pages, max(self.cache.held_pages()))
        produced: List[int] = []
        before, self._pending = self._pending, None      # what the step before selected and the host has not seen
        try:
            if portions:
                entries = []
                for portion in portions:
                    request = portion.request
                    tokens = request.tokens_between(portion.start, portion.start + portion.count)
                    token_from = None
                    if NOT_YET in tokens:
                        row = before.row_of(request) if before is not None else None
                        if portion.count == 1 and row is not None:
                            tokens, token_from = [0], row      # the step takes it from the device
                        else:                                    # a longer portion needs it here: wait for it
                            self._learn(before)
                            before = None
                            tokens = request.tokens_between(portion.start, portion.start + portion.count)
                    entries.append(StepEntry(request.id, tokens, [portion.count - 1] if portion.wants_logits else [], token_from))
                device_tokens = before.selection.device if before is not None and any(e.token_from is not None for e in entries) else None
                try:
                    if device_tokens is None:
                        logits = self.engine.step(entries, reserved=True, borrow_logits=True)
                    else:
                        logits = self.engine.step(entries, reserved=True, borrow_logits=True, device_tokens=device_tokens)
                except Exception:
                    self._step_failed(portions)
                    raise
                for portion in portions:
                    if portion.count == 1 and portion.request.state == RequestState.DECODING:
                        self.metrics.decode_tokens += 1
                    else:
                        self.metrics.prefill_tokens += portion.count
                    self.metrics.batched_tokens += portion.count
                self.metrics.engine_steps += 1
                for portion in portions:
                    portion.request.computed += portion.count
                wanting = [portion.request for portion in portions if portion.wants_logits]
                if wanting and self.lookahead and not any(r.params.stop_tokens for r in wanting):
                    # Selected, not waited for: what ends a request here is its length, which needs no id.
                    selection = self.sampler.select_later(logits, [r.params for r in wanting], [len(r.generated) for r in wanting])
                    self._pending = Pending(list(wanting), [len(r.generated) for r in wanting], selection)
                    for request in wanting:
                        request.generated.append(NOT_YET)
                        request.state = RequestState.DECODING
                        produced.append(request.id)
                        if len(request.generated) >= request.params.max_new_tokens:
                            self._complete(request, CompletionReason.LENGTH)
                elif wanting:
                    tokens = self.sampler.select(logits, [r.params for r in wanting], [len(r.generated) for r in wanting])
                    now = time.perf_counter()
                    for request, token in zip(wanting, tokens):
                        request.generated.append(int(token))
                        request.state = RequestState.DECODING
                        if request.first_token_time < 0:
                            request.first_token_time = now
                        produced.append(request.id)
                        if int(token) in request.params.stop_tokens:      # emitted, then stop
                            self._complete(request, CompletionReason.STOP_TOKEN)
                        elif len(request.generated) >= request.params.max_new_tokens:
                            self._complete(request, CompletionReason.LENGTH)
        finally:
            if before is not None:
                self._learn(before)      # its copy has long arrived: the GPU is busy with the step just launched
        self.current_step += 1
        return produced

    def _learn(self, pending: Pending) -> None:
        """The host takes the ids of a selection it did not wait for."""
        tokens = pending.selection.tokens()
        now = time.perf_counter()
        for request, place, token in zip(pending.requests, pending.places, tokens):
            if place < len(request.generated) and request.generated[place] == NOT_YET:
                request.generated[place] = int(token)
            if request.first_token_time < 0:
                request.first_token_time = now
            if request.state == RequestState.COMPLETED and request.completion_time < now and place == len(request.generated) - 1:
                request.completion_time = now      # it ended at its length before its last id was known

    def drain(self) -> None:
        """Wait for what the last step selected (``lookahead``): every generated id is then known to the host."""
        pending, self._pending = self._pending, None
        if pending is not None:
            self._learn(pending)

    def run_until_idle(self, maximum_steps: int = -1) -> None:
        """Step until nothing runs or waits; more than ``maximum_steps`` is an error
        (src/inference/scheduler.cpp:1002-1005)."""
        steps = 0
        while self.has_work():
            if 0 <= maximum_steps <= steps:
                raise RuntimeError(f"scheduler did not become idle within {maximum_steps} steps")
            self.step()
            steps += 1
        self.drain()

    # ---- endings -------------------------------------------------------------------------
    def _release(self, request: Request) -> None:
        if self.cache.requests.get(request.id) is not None:
            self.cache.close(request.id)

    def _step_failed(self, portions: List[Portion]) -> None:
        """The engine raised inside a step: nothing of the step counts. The engine has given back the pages the
        step took; the requests keep the positions they had and go on from there in the next step. Where the
        model keeps per-request state, which the failed step may have changed, every request of the step starts
        again from its first token instead, as after a preemption (the engine refuses to go on with them). The
        reference resets the rows of a failed prefill (src/inference/scheduler.cpp:763-766)."""
        self.metrics.failed_steps += 1
        if getattr(self.cache, "has_state", False):
            for portion in reversed(portions):
                if portion.request in self.running:
                    self._preempt(portion.request, failed=True)
        for portion in portions:      # reservations that the engine did not see (it raised before it came to them)
            handle = self.cache.requests.get(portion.request.id)
            if handle is not None and handle.reserved:
                self.cache.cancel_reservation(handle)

    def _preempt(self, request: Request, failed: bool = False) -> None:
        self.running.remove(request)
        self._release(request)
        request.computed = 0
        request.admitted = False
        request.state = RequestState.PENDING_PREFILL
        if not failed:
            request.preemptions += 1
            self.metrics.preemptions += 1
        self.waiting.appendleft(request)

    def _complete(self, request: Request, reason: CompletionReason) -> None:
        self.running.remove(request)
        self._release(request)
        self._finish(request, reason)

    def _finish(self, request: Request, reason: CompletionReason) -> None:
        request.state = RequestState.COMPLETED
        request.completion_reason = reason
        request.completion_step = self.current_step
        request.completion_time = time.perf_counter()
        self.metrics.completed_requests += 1
        if reason == CompletionReason.STOP_TOKEN:
            self.metrics.stop_completed_requests += 1

    # ---- looking -------------------------------------------------------------------------
    def request(self, request_id: int) -> Request:
        if request_id not in self.requests:
            raise KeyError(f"unknown request {request_id}")
        return self.requests[request_id]
