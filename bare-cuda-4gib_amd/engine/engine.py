"""The Python entry point, in the manner of the reference's ``llm_engine_py.Engine``
(server/bindings.cc:70-107 over engine/src/async_engine.cpp): the same
constructor arguments, ``submit / cancel / poll / stop / stats`` and the same
properties, events as ``(id, token, index, finish)`` tuples and submit results as
``(status, message)`` with status ``ok | invalid | busy | unavailable``.

Who runs the scheduler is the caller's choice.  With ``worker=True`` a thread of
the engine's own does, as in the reference (async_engine.cpp:156-205): any thread
may submit, cancel and poll, tokens are generated while the caller does other
things, and ``poll`` waits up to its time-out for events.  Without, ``poll`` runs
the same turns on the caller's thread until there are events, so the GPU is only
ever touched by the thread that polls.  Either way what is submitted or cancelled
waits in an inbox for the next turn, which takes submissions before
cancellations: a cancellation right after its submission finds the request.
"""
from __future__ import annotations

import atexit
import collections
import dataclasses
import threading
import weakref
from typing import Deque, Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import EngineError
from ..sampling.device import DevicePicker
from ..sampling.params import SamplingParams
from .executor import Executor, StepEntry
from .model import load_model
from .scheduler import (FINISH_CANCELLED, FINISH_ERROR, Request, Scheduler, TokenEvent)

Event = Tuple[int, int, int, str]


def working_memory_estimate(model, max_seqs: int, max_batch_tokens: int, graphs: int, max_tokens: int = 0,
                            elem: int = 2) -> int:
    """Device bytes the engine will take beyond weights and cache while it serves, from what the model's parts
    state (Model.working_bytes): the largest step -- max_batch_tokens rows, or, where that is 0 and only memory
    limits a step, as many as one request may bring (max_tokens) -- with logits for every request, and for every
    captured decode graph its own activations and its logits [requests, vocab] in float."""
    rows = max(max_batch_tokens or max_tokens, max_seqs)
    step = model.working_bytes(rows, max_seqs, elem)
    graph = model.working_bytes(max_seqs, max_seqs, elem)
    return step + graphs * graph


def fit_kv_pages(model, max_tokens: int, max_seqs: int, page_tokens: int, dtype: torch.dtype,
                 device, headroom_bytes: int = 1 << 30, working_bytes: int = 0) -> int:
    """Pages for every request to reach max_tokens, or as many as free memory holds (less a headroom
    and what the engine will need to work: ``working_bytes``).  The weights -- both copies of every
    linear map -- are on the device already when this is asked, so free memory accounts for them.
    (Reference: fit_kv_pages, engine/src/model.cpp:259-277.)"""
    from ..cache import bytes_per_page
    per_request = -(-max_tokens // page_tokens)
    want = per_request * max_seqs
    per_page = bytes_per_page(model.cache_streams().values(), page_tokens, dtype)
    if per_page == 0:
        return want
    free, _ = torch.cuda.mem_get_info(device)
    fit = max(0, (free - headroom_bytes - working_bytes)) // per_page
    if fit < per_request:
        raise EngineError(f"free GPU memory holds {fit} cache pages, one request of {max_tokens} tokens "
                          f"needs {per_request}")
    return int(min(want, fit))


def _stop_at_exit(ref) -> None:
    engine = ref()
    if engine is not None:
        engine.stop()


class Engine:
    def __init__(self, model_path: str, max_tokens: int = 1024, max_seqs: int = 8, kv_pages: int = 0,
                 max_waiting: int = 64, *, dtype: str = "bfloat16", device: str = "cuda:0",
                 page_tokens: int = 64, max_batch_tokens: int = 2048, prefill_chunk: int = 512,
                 worker: bool = False, gather_ms: float = 0.0):
        if max_tokens <= 0 or max_seqs <= 0:
            raise EngineError("max_tokens and max_seqs must be positive")
        self.model, self.config = load_model(model_path, dtype, device)
        if max_tokens > self.model.max_seq_len:
            raise EngineError(f"max_tokens {max_tokens} is beyond the model's {self.model.max_seq_len} positions")
        rt = self.model.rt
        if kv_pages <= 0:
            working = working_memory_estimate(self.model, max_seqs, max_batch_tokens, Executor.MAX_GRAPHS, max_tokens,
                                              torch.empty((), dtype=rt.act_dtype).element_size())
            kv_pages = fit_kv_pages(self.model, max_tokens, max_seqs, page_tokens, rt.act_dtype, rt.device,
                                    working_bytes=working)
        self.executor = Executor(self.model, num_pages=kv_pages, max_requests=max_seqs,
                                 max_tokens=max_tokens, page_tokens=page_tokens,
                                 max_batch_tokens=max_batch_tokens)
        self.scheduler = Scheduler(self.executor, DevicePicker(), max_batch_tokens=max_batch_tokens,
                                   prefill_chunk=prefill_chunk, run_ahead=True, gather_ms=gather_ms)
        self._max_waiting = max_waiting
        # The inbox: what any thread hands to whoever runs the turns, and the ids not yet finished.
        self._in = threading.Condition()
        self._inbox: List[Request] = []
        self._cancels: List[int] = []
        self._live = set()
        self._failure = ""
        self._stopping = False
        self._injected = ""
        self._stats = self.scheduler.stats()
        # The outbox: events for whoever polls.
        self._out = threading.Condition()
        self._outbox: Deque[Event] = collections.deque()
        self._stopped = False
        self._thread: Optional[threading.Thread] = None
        if worker:
            self._thread = threading.Thread(target=self._loop, name="bc4g-engine", daemon=True)
            self._thread.start()
            atexit.register(_stop_at_exit, weakref.ref(self))     # the worker leaves the GPU before the interpreter goes

    @classmethod
    def from_config(cls, config: dict, seed: int = 0, dtype: str = "bfloat16", folder: Optional[str] = None,
                    **engine_args) -> "Engine":
        """An engine over random weights: the model folder (config.json, model.safetensors) is written
        from the configuration and the seed by the random-weights mode -- into ``folder``, or into a
        temporary one that lives as long as the engine -- and loaded like any other."""
        import tempfile
        from ..weights import write_random_model
        keep = None
        if folder is None:
            keep = tempfile.TemporaryDirectory(prefix="bc4g_model_")
            folder = keep.name
        write_random_model(config, seed, folder, dtype)
        engine = cls(folder, dtype=dtype, **engine_args)
        engine._model_folder = keep
        return engine

    # ---- properties ---------------------------------------------------------
    @property
    def healthy(self) -> bool:
        with self._in:
            return not self._failure

    @property
    def failure(self) -> str:
        with self._in:
            return self._failure

    @property
    def max_tokens(self) -> int:
        return self.scheduler.limits.max_tokens

    @property
    def max_seqs(self) -> int:
        return self.scheduler.limits.max_seqs

    @property
    def kv_pages(self) -> int:
        return self.scheduler.limits.kv_pages

    @property
    def vocab_size(self) -> int:
        return self.model.vocab_size

    # ---- requests -----------------------------------------------------------
    def submit(self, id: int, prompt: Sequence[int], max_new_tokens: int, stop_ids: Sequence[int] = (),
               temperature: float = 0.0, top_p: float = 1.0, top_k: int = 0, seed: int = -1,
               timeout_ms: int = 0) -> Tuple[str, str]:
        """Queues a request; returns (status, message).  temperature 0 is greedy."""
        request = Request(id=id, prompt=list(prompt), max_new_tokens=max_new_tokens, stop_ids=list(stop_ids),
                          sampling=SamplingParams(temperature, top_p, top_k, seed), timeout_ms=timeout_ms)
        with self._in:
            error = self.scheduler.check(request)          # reads limits only
            if error:
                return "invalid", error
            if self._failure:
                return "unavailable", "engine failed: " + self._failure
            if self._stopping:
                return "unavailable", "engine is stopped"
            # live: running, waiting, and not yet seen by a turn
            if self._max_waiting > 0 and len(self._live) >= self.max_seqs + self._max_waiting:
                return "busy", f"{len(self._live)} requests already in flight"
            if id in self._live:
                return "invalid", f"request id {id} is already in use"
            self._live.add(id)
            self._inbox.append(request)
            self._in.notify()
        return "ok", ""

    def cancel(self, id: int) -> None:
        """Ends a request early; it then gets one last event with finish 'cancelled'."""
        with self._in:
            self._cancels.append(id)
            self._in.notify()

    def poll(self, timeout_ms: int = 100) -> List[Event]:
        """The events since the last poll: a list of (id, token, index, finish) tuples.  With a worker:
        waits up to timeout_ms for some; empty on time-out or once stopped.  Without: runs turns on this
        thread until there are events or nothing is left to do."""
        if self._thread is None:
            while True:
                with self._out:
                    if self._outbox or self._stopped:
                        break
                if not self._turn():
                    break
        with self._out:
            if self._thread is not None:
                self._out.wait_for(lambda: self._outbox or self._stopped, max(0, timeout_ms) / 1000.0)
            out = list(self._outbox)
            self._outbox.clear()
        return out

    def idle(self) -> bool:
        """Nothing submitted is unfinished and no event waits to be polled."""
        with self._in:
            busy = bool(self._live)
        with self._out:
            return not busy and not self._outbox

    def stop(self) -> None:
        """Stops the worker, if there is one; waiting and running requests are dropped."""
        with self._in:
            already = self._stopping
            self._stopping = True
            self._in.notify_all()
        if self._thread is not None and self._thread is not threading.current_thread():
            self._thread.join()
        if not already:
            for r in list(self.scheduler.running) + list(self.scheduler.waiting):
                self.scheduler.cancel(r.id)
            with self._in:
                self._inbox.clear()
                self._cancels.clear()
                self._live.clear()
        with self._out:
            self._stopped = True
            self._out.notify_all()

    def stats(self) -> Dict[str, object]:
        """The scheduler's figures as of its last step; waiting also counts requests no turn has seen yet."""
        with self._in:
            snapshot = self._stats if self._thread is not None else self.scheduler.stats()
            out = dataclasses.asdict(snapshot)
            out["waiting"] += len(self._inbox)
        return out

    def _fail_for_test(self, message: str) -> None:
        """Makes the next turn fail, to exercise the failure path."""
        with self._in:
            self._injected = message
            self._in.notify()

    # ---- the step function, for programs that bring their own tokens ------------
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        for e in entries:
            if not self.executor.has(e.request):
                self.executor.admit(e.request)
        return self.executor.step(entries)

    def release(self, request) -> None:
        self.executor.release(request)

    # ---- internals -----------------------------------------------------------
    def _turn(self) -> bool:
        """One turn of the serving loop, on whichever thread runs it (the only one that touches the scheduler
        and the GPU): takes in what was submitted and cancelled since the last, runs one scheduler step if there
        is work, keeps the scheduler's figures.  False if there was nothing to do.  An error ends every live
        request with 'error'; the engine refuses new work from then on."""
        with self._in:
            if self._stopping or self._failure:
                return False
            injected = self._injected
            requests, self._inbox = self._inbox, []
            cancels, self._cancels = self._cancels, []
        if not (requests or cancels or injected) and self.scheduler.idle():
            return False
        try:
            if injected:
                raise EngineError(injected)
            for r in requests:
                self.scheduler.submit(r)
            self._publish([TokenEvent(id, -1, -1, FINISH_CANCELLED) for id in cancels if self.scheduler.cancel(id)])
            if not self.scheduler.idle():
                self._publish(self.scheduler.step())
            snapshot = self.scheduler.stats()
            with self._in:
                self._stats = snapshot
        except Exception as e:
            self._fail_all(str(e))
        return True

    def _loop(self) -> None:
        """The worker: sleeps only when there is nothing to decode and nothing new."""
        torch.cuda.set_device(self.model.rt.device)
        decoding = False
        while True:
            with self._in:
                self._in.wait_for(lambda: self._stopping or self._failure or self._inbox or self._cancels
                                  or self._injected or decoding)
                if self._stopping or self._failure:
                    return
            self._turn()
            decoding = not self.scheduler.idle()

    def _publish(self, events: List[TokenEvent]) -> None:
        if not events:
            return
        with self._in:
            for e in events:
                if e.finish:
                    self._live.discard(e.id)
        with self._out:
            self._outbox.extend((e.id, e.token, e.index, e.finish) for e in events)
            self._out.notify_all()

    def _fail_all(self, message: str) -> None:
        with self._in:
            self._failure = message
            ids = sorted(self._live)
            self._live.clear()
            self._inbox.clear()
            self._cancels.clear()
            self._in.notify_all()
        with self._out:
            self._outbox.extend((id, -1, -1, FINISH_ERROR) for id in ids)
            self._out.notify_all()


def generate_batch(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
                   **sampling) -> List[List[int]]:
    """All prompts through the scheduler, ids 0..n-1 (reference: Model::generate_batch,
    engine/src/model.cpp:693-717)."""
    out: List[List[int]] = [[] for _ in prompts]
    for i, p in enumerate(prompts):
        status, message = engine.submit(i, p, max_new_tokens, **sampling)
        if status != "ok":
            raise EngineError(f"prompt {i}: {message}")
    done = 0
    while done < len(prompts):
        events = engine.poll()
        if not events and engine.idle():
            break
        for id, token, index, finish in events:
            if token >= 0:
                out[id].append(token)
            if finish:
                if finish == "error":
                    raise EngineError(engine.failure)
                done += 1
    return out
