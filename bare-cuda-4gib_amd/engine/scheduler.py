"""Continuous batching above the step function.

What it keeps of the reference's scheduler (engine/include/llm/scheduler.h:15-129,
engine/src/scheduler.cpp:28-208): requests with ``id, prompt, max_new_tokens,
stop_ids, sampling, timeout_ms``; the same refusals in ``check``; FIFO admission
in which a request that does not fit blocks the ones behind it; a stop id ends a
request and *is* emitted; ``target = min(max_new_tokens, max_tokens - prompt + 1)``
(the last generated token is never run through the model); per-request random
generators; TokenEvent and the stats' names.

What it does differently: the reference runs each admitted prompt whole and
alone and then one decode pass; here every step is ONE batch under a token
budget -- one token for every request that is decoding, then portions of
prompts (at most ``prefill_chunk`` tokens of a request a step) in admission
order.  And pages are not promised for a request's whole run at admission:
they are taken as tokens arrive.  When a step's tokens do not fit the pool,
the request admitted last is preempted: its pages are given back and it goes to
the front of the waiting line with the tokens it has generated so far appended
to its prompt, to be recomputed later (its generator state and its count of
generated tokens are kept, so its output is unchanged).  A request that could
never fit the pool alone is refused at ``check``.
"""
from __future__ import annotations

import collections
import dataclasses
import time
from typing import Deque, List, Sequence

from ..errors import EngineError, OutOfPages
from ..sampling.mt19937_64 import MT19937_64
from ..sampling.params import SamplingParams, check_sampling, seed_for
from .executor import StepEntry

FINISH_NONE, FINISH_STOP, FINISH_LENGTH = "", "stop", "length"
FINISH_CANCELLED, FINISH_TIMEOUT, FINISH_ERROR = "cancelled", "timeout", "error"


@dataclasses.dataclass
class Request:
    id: int = 0
    prompt: Sequence[int] = ()
    max_new_tokens: int = 16
    stop_ids: Sequence[int] = ()          # generating any of these ends the request, e.g. EOS
    sampling: SamplingParams = dataclasses.field(default_factory=SamplingParams)
    timeout_ms: int = 0                   # from submit, waiting plus running; 0 never times out


@dataclasses.dataclass
class TokenEvent:
    """One generated token, or a request ending without one (token -1)."""
    id: int = 0
    token: int = -1
    index: int = -1                       # position among this request's generated tokens
    finish: str = FINISH_NONE


@dataclasses.dataclass
class EngineLimits:
    max_tokens: int = 0                   # per request, prompt plus generated
    max_seqs: int = 0
    kv_pages: int = 0
    page_tokens: int = 64


@dataclasses.dataclass
class SchedulerStats:
    running: int = 0
    waiting: int = 0
    kv_pages_used: int = 0
    kv_pages_total: int = 0
    steps: int = 0                        # batches run
    prefill_tokens: int = 0               # prompt tokens run through the model (recomputed ones included)
    decode_tokens: int = 0                # rows decoded, one per decoding request per step
    preemptions: int = 0
    busy_seconds: float = 0.0


class _Live:
    """A request that has been submitted: waiting, or running with a cache slot."""
    def __init__(self, request: Request, deadline: float):
        self.id = request.id
        self.tokens: List[int] = [int(t) for t in request.prompt]   # prompt + generated so far
        self.prompt_len = len(self.tokens)
        self.computed = 0                 # tokens whose keys are in the cache
        self.generated = 0
        self.target = 0
        self.stop_ids = set(int(s) for s in request.stop_ids)
        self.sampling = request.sampling
        self.rng = MT19937_64(seed_for(request.sampling))
        self.deadline = deadline
        self.admitted_at = -1             # admission counter; the largest is preempted first
        self.queued_at = 0.0              # when it joined the waiting line (the scheduler's clock)


def target_tokens(limits: EngineLimits, prompt_len: int, max_new_tokens: int) -> int:
    return min(max_new_tokens, limits.max_tokens - prompt_len + 1)


def cached_tokens(limits: EngineLimits, prompt_len: int, max_new_tokens: int) -> int:
    """Tokens of the request that ever reach the cache: the last generated one is never run."""
    return prompt_len + target_tokens(limits, prompt_len, max_new_tokens) - 1


def pages_needed(limits: EngineLimits, prompt_len: int, max_new_tokens: int) -> int:
    """Pages of a stream that keeps every token (reference: pages_needed, engine/src/scheduler.cpp:36-43)."""
    return -(-cached_tokens(limits, prompt_len, max_new_tokens) // limits.page_tokens)


def check_request(limits: EngineLimits, request: Request, cache=None, portion: int = 0) -> str:
    """Empty if the request can ever run, else why not.  What it needs of the page pools the cache
    manager says (``cache.peak_pages``: per group of streams, by the group's own rule of what is
    kept -- a windowed group needs its window and a portion, a model without per-token streams
    nothing); without a cache manager, one stream that keeps every token is assumed."""
    n = len(request.prompt)
    if n == 0:
        return "empty prompt"
    if request.max_new_tokens <= 0:
        return "max_new_tokens must be positive"
    if n > limits.max_tokens:
        return f"prompt has {n} tokens, the engine holds {limits.max_tokens} per sequence"
    if cache is None:
        pages = pages_needed(limits, n, request.max_new_tokens)
        if pages > limits.kv_pages:
            return f"request needs {pages} KV pages, the pool holds {limits.kv_pages}"
    else:
        need = cache.peak_pages(cached_tokens(limits, n, request.max_new_tokens), portion or limits.max_tokens)
        for g, pages in need.items():
            if pages > cache.groups[g].pool.num_pages:
                return f"request needs {pages} KV pages, the pool holds {cache.groups[g].pool.num_pages}"
    return check_sampling(request.sampling)


class Scheduler:
    """Not thread-safe; one thread calls everything.

    executor: the step function and its cache (``step, admit, release, has,
    cache``).  picker: chooses tokens from logits rows (``pick(logits, params,
    rngs) -> ids``).  max_batch_tokens: rows a step may hold.  prefill_chunk:
    the most prompt tokens of one request in one step.
    """

    def __init__(self, executor, picker, *, max_batch_tokens: int = 2048, prefill_chunk: int = 512,
                 clock=time.monotonic, run_ahead: bool = False, gather_ms: float = 0.0):
        """``gather_ms``: while every running request is decoding, a waiting request is admitted only after it has
        waited this long, and whoever came meanwhile with it: a step that brings a prompt portion cannot be replayed
        from a captured graph nor run ahead, so where requests come and go all the time (short prompts, long answers)
        admitting them one by one makes every other step such a step; gathered, they share one.  0 admits at once.
        Nothing is held back while nothing runs or while a prompt is under way anyway, nor while requests come so
        rarely that nobody else is to be expected within the wait (the mean gap between the last arrivals is longer
        than it): a slot that waits for company that does not come only costs.

        ``run_ahead``: while every running request is decoding and none can be admitted, the next
        step is launched with its tokens taken from what the sampling kernel has just chosen, on
        the device, before the host has read them; the host reads a step's tokens (and emits its
        events) while the next step runs.  The tokens are the same; the events of a step come out
        of the following call to step().  Needs a picker with ``pick_later`` and an executor whose
        step takes ``device_tokens``."""
        if max_batch_tokens <= 0 or prefill_chunk <= 0:
            raise EngineError("scheduler: max_batch_tokens and prefill_chunk must be positive")
        self.executor = executor
        self.picker = picker
        self.run_ahead = run_ahead
        self.gather_ms = gather_ms
        self._last_arrival = None         # when the last request was submitted, and the running mean of the gaps
        self._arrival_gap = float("inf")  # between arrivals (seconds; half of it is the newest gap)
        self._ahead = None                # (requests, picked): a step whose tokens have not been read yet
        self.max_batch_tokens = max_batch_tokens
        self.prefill_chunk = prefill_chunk
        self._clock = clock
        cache = executor.cache
        pools = [g.pool.num_pages for g in cache.groups.values()]       # (none: the model keeps nothing per token)
        self.limits = EngineLimits(max_tokens=cache.max_tokens, max_seqs=cache.max_requests,
                                   kv_pages=min(pools) if pools else 0, page_tokens=cache.page_tokens)
        self.waiting: Deque[_Live] = collections.deque()
        self.running: List[_Live] = []
        self._admissions = 0
        self._totals = SchedulerStats()
        self.vocab_size = getattr(getattr(executor, "model", None), "vocab_size", None)

    # ---- submitting and cancelling ---------------------------------------------
    def check(self, request: Request) -> str:
        cache = self.executor.cache
        error = check_request(self.limits, request, cache if hasattr(cache, "peak_pages") else None,
                              min(self.prefill_chunk, self.max_batch_tokens))
        if error:
            return error
        if self.vocab_size is not None:
            for t in request.prompt:
                if not (0 <= int(t) < self.vocab_size):
                    return f"token id {t} is outside the vocabulary [0, {self.vocab_size})"
        return ""

    def submit(self, request: Request) -> None:
        error = self.check(request)
        if error:
            raise EngineError(f"scheduler: request {request.id}: {error}")
        if any(r.id == request.id for r in self.waiting) or any(r.id == request.id for r in self.running):
            raise EngineError(f"scheduler: request {request.id}: id is already live")
        deadline = self._clock() + request.timeout_ms / 1000.0 if request.timeout_ms > 0 else float("inf")
        live = _Live(request, deadline)
        live.target = target_tokens(self.limits, live.prompt_len, request.max_new_tokens)
        live.queued_at = self._clock()
        if self._last_arrival is not None:
            gap = live.queued_at - self._last_arrival
            self._arrival_gap = gap if self._arrival_gap == float("inf") else 0.5 * (self._arrival_gap + gap)
        self._last_arrival = live.queued_at
        self.waiting.append(live)

    def cancel(self, request_id) -> bool:
        """Drops a waiting or running request and frees what it holds.  False if unknown."""
        for r in self.waiting:
            if r.id == request_id:
                self.waiting.remove(r)
                return True
        for r in self.running:
            if r.id == request_id:
                self._retire(r)
                self.running.remove(r)
                return True
        return False

    def idle(self) -> bool:
        return not self.waiting and not self.running and self._ahead is None

    def stats(self) -> SchedulerStats:
        s = dataclasses.replace(self._totals)
        s.running, s.waiting = len(self.running), len(self.waiting)
        s.kv_pages_used = self.executor.cache.pages_in_use()
        s.kv_pages_total = self.executor.cache.pages_total()
        return s

    # ---- one step ---------------------------------------------------------------
    def step(self) -> List[TokenEvent]:
        start = self._clock()
        try:
            return self._run_step()
        finally:
            self._totals.busy_seconds += self._clock() - start

    def _retire(self, r: _Live) -> None:
        if self.executor.has(r.id):
            self.executor.release(r.id)

    def _expire(self, events: List[TokenEvent]) -> None:
        now = self._clock()
        for r in [r for r in self.waiting if r.deadline <= now]:
            self.waiting.remove(r)
            events.append(TokenEvent(r.id, -1, -1, FINISH_TIMEOUT))
        for r in [r for r in self.running if r.deadline <= now]:
            self._retire(r)
            self.running.remove(r)
            events.append(TokenEvent(r.id, -1, -1, FINISH_TIMEOUT))

    def _preempt_latest(self) -> bool:
        """Give back everything the request admitted last holds and put it at the front of
        the waiting line, to be recomputed.  False if at most one request is running (a lone
        request always fits: check() saw to that)."""
        if len(self.running) <= 1:
            return False
        victim = max(self.running, key=lambda r: r.admitted_at)
        self.running.remove(victim)
        self._retire(victim)
        victim.computed = 0
        victim.queued_at = float("-inf")   # (has waited long enough: back in as soon as it fits)
        self.waiting.appendleft(victim)
        self._totals.preemptions += 1
        return True

    def _gathering(self) -> bool:
        """Whether those who wait are held back for now, to be admitted together (gather_ms)."""
        if self.gather_ms <= 0.0 or not self.waiting or not self.running:
            return False
        if any(len(r.tokens) - r.computed > 1 for r in self.running):
            return False                   # a prompt is under way: this step is no decode step anyway
        if self._arrival_gap * 1000.0 >= self.gather_ms:
            return False                   # requests come too rarely for company within the wait
        return (self._clock() - self.waiting[0].queued_at) * 1000.0 < self.gather_ms

    def plan(self) -> List[tuple]:
        """Decide this step's batch: [(live request, number of its next tokens)].  Admits
        waiting requests (taking their slot) and preempts running ones as needed; touches no
        pages."""
        cache = self.executor.cache
        preempted = False
        while True:
            budget = self.max_batch_tokens
            batch: List[tuple] = []
            # 1. one token for every request that is decoding
            for r in self.running:
                if len(r.tokens) - r.computed == 1 and budget > 0:
                    batch.append((r, 1))
                    budget -= 1
            # 2. portions of the prompts of running requests, in admission order
            for r in sorted(self.running, key=lambda r: r.admitted_at):
                left = len(r.tokens) - r.computed
                if left > 1 and budget > 0:
                    n = min(left, self.prefill_chunk, budget)
                    batch.append((r, n))
                    budget -= n
            if cache.can_reserve([(r.id, n) for r, n in batch]):
                break
            if not self._preempt_latest():
                raise OutOfPages("scheduler: a lone request does not fit the page pool")
            preempted = True
        # 3. admit waiting requests in order; one that does not fit blocks those behind it
        #    (not in a step that had to preempt: the pool is full)
        while not preempted and self.waiting and budget > 0 and cache.free_slots > 0 and not self._gathering():
            r = self.waiting[0]
            n = min(len(r.tokens) - r.computed, self.prefill_chunk, budget)
            self.executor.admit(r.id)
            if not cache.can_reserve([(q.id, m) for q, m in batch] + [(r.id, n)]):
                self.executor.release(r.id)
                break
            self.waiting.popleft()
            r.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(r)
            batch.append((r, n))
            budget -= n
        return batch

    def _run_step(self) -> List[TokenEvent]:
        events: List[TokenEvent] = []
        self._expire(events)
        if self._ahead is not None:
            # the step launched last has not been read: launch the one after it if nothing but
            # decoding goes on, then read the first while the second runs
            ahead, self._ahead = self._ahead, None
            following = self._launch_following(ahead)
            self._read(ahead, events)
            if following is not None:
                self._ahead = following
                return events
        batch = self.plan()
        if not batch:
            return events
        entries, wanted = [], []
        for r, n in batch:
            last = r.computed + n == len(r.tokens)
            entries.append(StepEntry(r.id, r.tokens[r.computed:r.computed + n], [n - 1] if last else []))
            if last:
                wanted.append(r)
            if n == 1 and r.computed >= r.prompt_len:
                self._totals.decode_tokens += 1
            else:
                self._totals.prefill_tokens += n
        logits = self.executor.step(entries)
        self._totals.steps += 1
        for r, n in batch:
            r.computed += n
        if wanted:
            if self.run_ahead:
                picked = self.picker.pick_later(logits, [r.sampling for r in wanted], [r.rng for r in wanted])
                if picked is not None:
                    self._ahead = (wanted, picked)
                    return events
            tokens = self.picker.pick(logits, [r.sampling for r in wanted], [r.rng for r in wanted])
            for r, token in zip(wanted, tokens):
                self._emit(r, int(token), events)
        return events

    def _launch_following(self, ahead):
        """The step after one whose tokens are still on the device, if it can be decided without
        them: every running request took part in that step and goes on decoding (those that reach
        their length with it leave; one that turns out to have met a stop id has run a token too
        far, into pages that its end gives back), nothing waits that could be admitted, the pages
        are there, and the tokens can be chosen on the device again.  None otherwise."""
        requests, picked = ahead
        running = {id(r) for r in self.running}
        live = sum(1 for r in requests if id(r) in running)
        if live != len(self.running) or (self.waiting and self.executor.cache.free_slots > 0 and not self._gathering()):
            return None
        rows = [i for i, r in enumerate(requests) if id(r) in running and r.generated + 1 < r.target]
        if not rows or len(rows) > self.max_batch_tokens:
            return None
        going = [requests[i] for i in rows]
        if not self.executor.cache.can_reserve([(r.id, 1) for r in going]):
            return None
        tokens = picked.tokens_for(rows)
        logits = self.executor.step([StepEntry(r.id, [0], [0]) for r in going], device_tokens=tokens)
        self._totals.steps += 1
        self._totals.decode_tokens += len(going)
        for r in going:
            r.computed += 1
        following = self.picker.pick_later(logits, [r.sampling for r in going], [r.rng for r in going])
        assert following is not None, "the same requests' tokens were chosen on the device a step ago"
        return (going, following)

    def _read(self, ahead, events: List[TokenEvent]) -> None:
        requests, picked = ahead
        running = {id(r) for r in self.running}
        for r, token in zip(requests, picked.result()):
            if id(r) in running:           # (not cancelled, expired or ended by a stop id meanwhile)
                self._emit(r, int(token), events)

    def _emit(self, r: _Live, token: int, events: List[TokenEvent]) -> None:
        e = TokenEvent(r.id, token, r.generated)
        r.generated += 1
        r.tokens.append(token)
        if token in r.stop_ids:
            e.finish = FINISH_STOP
        elif r.generated == r.target:
            e.finish = FINISH_LENGTH
        events.append(e)
        if e.finish != FINISH_NONE:
            self._retire(r)
            self.running.remove(r)
