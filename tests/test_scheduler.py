"""The scheduler's decisions, on the host, with a stand-in for the step function whose logits
depend only on a request's own tokens (so outputs must not depend on batching, portions or
preemption).  Scenarios after engine/tests/test_scheduler.cu:122-255."""
import hashlib

import numpy as np
import pytest
import torch

from bare_cuda_4gib_amd.cache import CacheManager, PagedKV
from bare_cuda_4gib_amd.engine.executor import StepEntry
from bare_cuda_4gib_amd.engine.scheduler import Request, Scheduler, check_request, EngineLimits
from bare_cuda_4gib_amd.errors import EngineError
from bare_cuda_4gib_amd.sampling import SamplingParams, sample_token

VOCAB = 50


def fake_logits(tokens):
    digest = hashlib.sha256(np.asarray(tokens, dtype=np.int64).tobytes()).digest()
    rng = np.random.default_rng(int.from_bytes(digest[:8], "little"))
    return rng.normal(size=VOCAB).astype(np.float32) * 3.0


class FakeExecutor:
    """Keeps a real cache manager (so pages run out for real) and checks that tokens arrive in
    order, each exactly once per (re)computation."""
    def __init__(self, num_pages=8, page_tokens=4, max_requests=3, max_tokens=32, streams=None):
        self.cache = CacheManager(streams if streams is not None else {0: PagedKV(1, 2)}, page_tokens=page_tokens, num_pages=num_pages,
                                  max_requests=max_requests, max_tokens=max_tokens, dtype=torch.float32, device="cpu")
        self.history = {}
        self.batches = []
        self.ahead_steps = 0

    def admit(self, rid):
        self.history[rid] = []
        return self.cache.admit(rid)

    def release(self, rid):
        self.cache.release(rid)
        del self.history[rid]

    def has(self, rid):
        return self.cache.has(rid)

    def step(self, entries, device_tokens=None):
        if device_tokens is not None:      # (here: a list that stands for the ids on the device)
            assert len(device_tokens) == len(entries) and all(e.tokens == [0] for e in entries)
            entries = [StepEntry(e.request, [t], e.want) for e, t in zip(entries, device_tokens)]
            self.ahead_steps += 1
        self.cache.reserve([(e.request, len(e.tokens)) for e in entries])
        self.batches.append([(e.request, len(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert len(self.history[e.request]) == self.cache.length(e.request)
            self.history[e.request].extend(e.tokens)
            self.cache.advance(e.request, len(e.tokens))
            for w in e.want:
                rows.append(fake_logits(self.history[e.request][:self.cache.length(e.request) - len(e.tokens) + w + 1]))
        return torch.tensor(np.stack(rows)) if rows else None


class HostPicker:
    def pick(self, logits, params, rngs):
        return [sample_token(logits[i].numpy(), p, r) for i, (p, r) in enumerate(zip(params, rngs))]

    def pick_later(self, logits, params, rngs):
        """What DevicePicker.pick_later gives, with a list in the place of the device tensor; rows
        with top-k or top-p cannot be chosen "on the device" here either."""
        if any(p.filtered() and not p.greedy() for p in params):
            return None
        tokens = self.pick(logits, params, rngs)

        class Later:
            def tokens_for(self, rows):
                return [tokens[i] for i in rows]

            def result(self):
                return tokens
        return Later()


def expected_greedy(prompt, n, stop=()):
    tokens, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(fake_logits(tokens)))
        out.append(t)
        tokens.append(t)
        if t in stop:
            break
    return out


def run(sched, max_steps=500):
    out, finish = {}, {}
    for _ in range(max_steps):
        if sched.idle():
            break
        for e in sched.step():
            if e.token >= 0:
                assert e.index == len(out.setdefault(e.id, []))
                out[e.id].append(e.token)
            if e.finish:
                finish[e.id] = e.finish
    assert sched.idle()
    return out, finish


def make(**kw):
    sched_kw = {k: kw.pop(k) for k in ("max_batch_tokens", "prefill_chunk", "clock", "run_ahead", "gather_ms") if k in kw}
    ex = FakeExecutor(**kw)
    return Scheduler(ex, HostPicker(), **{"max_batch_tokens": 16, "prefill_chunk": 6, **sched_kw}), ex


def prompt(n, seed):
    return [int(x) for x in np.random.default_rng(seed).integers(0, VOCAB, n)]


def test_outputs_do_not_depend_on_batching_and_budget_is_kept():
    sched, ex = make(num_pages=24)
    prompts = {i: prompt(n, i) for i, n in enumerate([5, 13, 1, 9, 7])}
    for i, p in prompts.items():
        sched.submit(Request(id=i, prompt=p, max_new_tokens=6))
    out, finish = run(sched)
    for i, p in prompts.items():
        assert out[i] == expected_greedy(p, 6) and finish[i] == "length"
    for batch in ex.batches:
        assert sum(n for _, n in batch) <= 16 and all(n <= 6 for _, n in batch)
        assert len(batch) <= 3                                         # slots
    assert any(len(b) > 1 and any(n > 1 for _, n in b) and any(n == 1 for _, n in b) for b in ex.batches), \
        "portions of prompts beside decoded tokens were expected in one batch"
    s = sched.stats()
    assert s.prefill_tokens == sum(len(p) for p in prompts.values()) and s.decode_tokens == 5 * 5
    assert s.kv_pages_used == 0 and s.running == 0 and s.waiting == 0 and s.preemptions == 0
    assert ex.cache.free_slots == 3


def test_admission_is_in_order_and_the_head_blocks():
    sched, ex = make(num_pages=4, max_tokens=16, prefill_chunk=16, max_batch_tokens=32)   # 16 tokens of pool
    sched.submit(Request(id=0, prompt=prompt(9, 0), max_new_tokens=2))    # 3 pages
    sched.submit(Request(id=1, prompt=prompt(9, 1), max_new_tokens=2))    # 3 pages: must wait for 0 to end
    sched.submit(Request(id=2, prompt=prompt(2, 2), max_new_tokens=2))    # would fit beside 0, but waits behind 1
    first_seen = []
    while not sched.idle():
        sched.step()
        for rid, _ in ex.batches[-1]:
            if rid not in first_seen:
                first_seen.append(rid)
    assert first_seen == [0, 1, 2]
    assert all(0 not in [r for r, _ in b] or 1 not in [r for r, _ in b] for b in ex.batches)


def test_stop_ids_budgets_and_prefill_only():
    sched, _ = make()
    p = prompt(7, 3)
    free_run = expected_greedy(p, 7)
    stop = free_run[3]
    sched.submit(Request(id=0, prompt=p, max_new_tokens=7))
    sched.submit(Request(id=1, prompt=p, max_new_tokens=7, stop_ids=[stop]))
    sched.submit(Request(id=2, prompt=p, max_new_tokens=1))
    out, finish = run(sched)
    assert out[0] == free_run and finish[0] == "length"
    first = free_run.index(stop)
    assert out[1] == free_run[:first + 1] and finish[1] == "stop"         # the stop token is emitted
    assert out[2] == free_run[:1] and finish[2] == "length"


def test_target_is_capped_by_max_tokens():
    sched, _ = make(num_pages=8, max_tokens=12)
    p = prompt(10, 4)
    sched.submit(Request(id=0, prompt=p, max_new_tokens=50))
    out, finish = run(sched)
    assert len(out[0]) == 12 - 10 + 1 and finish[0] == "length"           # the last token is never cached


def test_check_refusals():
    limits = EngineLimits(max_tokens=32, max_seqs=3, kv_pages=4, page_tokens=4)
    assert check_request(limits, Request(prompt=[], max_new_tokens=1)) == "empty prompt"
    assert "positive" in check_request(limits, Request(prompt=[1], max_new_tokens=0))
    assert "holds 32 per sequence" in check_request(limits, Request(prompt=[1] * 33, max_new_tokens=1))
    assert "KV pages" in check_request(limits, Request(prompt=[1] * 10, max_new_tokens=8))
    assert check_request(limits, Request(prompt=[1] * 10, max_new_tokens=7)) == ""
    assert "top_p" in check_request(limits, Request(prompt=[1], max_new_tokens=1, sampling=SamplingParams(top_p=0.0)))
    sched, _ = make()
    with pytest.raises(EngineError):
        sched.submit(Request(id=0, prompt=[], max_new_tokens=1))
    sched.submit(Request(id=0, prompt=[1], max_new_tokens=1))
    with pytest.raises(EngineError):
        sched.submit(Request(id=0, prompt=[1], max_new_tokens=1))          # id already live


def test_cancel_running_and_waiting():
    sched, ex = make(max_requests=1)
    sched.submit(Request(id=0, prompt=prompt(4, 0), max_new_tokens=20))
    sched.submit(Request(id=1, prompt=prompt(4, 1), max_new_tokens=3))
    sched.step(), sched.step()
    assert sched.cancel(1) and sched.cancel(0) and not sched.cancel(5)
    assert sched.idle() and ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 1


def test_sampling_seeds():
    def sample_run(seed, others=0, temperature=0.9, top_p=1.0):
        sched, _ = make(num_pages=24)
        sched.submit(Request(id=0, prompt=prompt(5, 9), max_new_tokens=8,
                             sampling=SamplingParams(temperature=temperature, top_p=top_p, seed=seed)))
        for j in range(others):
            sched.submit(Request(id=10 + j, prompt=prompt(6, 20 + j), max_new_tokens=8,
                                 sampling=SamplingParams(temperature=1.3, seed=99 + j)))
        return run(sched)[0][0]
    assert sample_run(7) == sample_run(7, others=2)                       # alone == batched
    assert sample_run(7) != sample_run(8)
    assert sample_run(7, top_p=1e-6) == expected_greedy(prompt(5, 9), 8)  # a vanishing nucleus is greedy


def test_timeouts_with_a_stepped_clock():
    now = [0.0]
    sched, ex = make(max_requests=1, clock=lambda: now[0])
    sched.submit(Request(id=0, prompt=prompt(4, 0), max_new_tokens=30, timeout_ms=50))
    sched.submit(Request(id=1, prompt=prompt(4, 1), max_new_tokens=2, timeout_ms=20))   # expires while waiting
    sched.submit(Request(id=2, prompt=prompt(4, 2), max_new_tokens=2))
    sched.step()
    now[0] = 0.03
    events = sched.step()
    assert [(e.id, e.token, e.finish) for e in events if e.finish] == [(1, -1, "timeout")]
    now[0] = 0.06
    events = sched.step()
    assert (0, -1, "timeout") in [(e.id, e.token, e.finish) for e in events]
    tokens = [e.token for e in events if e.id == 2]
    while not sched.idle():
        tokens += [e.token for e in sched.step() if e.id == 2]
    assert tokens == expected_greedy(prompt(4, 2), 2) and ex.cache.pages_in_use() == 0


def test_when_pages_run_out_the_latest_request_is_recomputed():
    # 3 requests of 6 + 10 tokens each need 4 pages each at the end; the pool has 9.
    sched, ex = make(num_pages=9, max_tokens=32)
    prompts = {i: prompt(6, 30 + i) for i in range(3)}
    for i, p in prompts.items():
        sched.submit(Request(id=i, prompt=p, max_new_tokens=10, sampling=SamplingParams(temperature=0.7, seed=i)))
    out, finish = run(sched)
    assert sched.stats().preemptions >= 1
    ref_sched, _ = make(num_pages=24, max_tokens=32)
    for i, p in prompts.items():
        ref_sched.submit(Request(id=i, prompt=p, max_new_tokens=10, sampling=SamplingParams(temperature=0.7, seed=i)))
    ref_out, _ = run(ref_sched)
    assert out == ref_out and set(finish.values()) == {"length"}
    assert ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3
    assert max(g.pool.high_water_mark for g in ex.cache.groups.values()) <= 9
    assert sched.stats().prefill_tokens > 18                              # recomputed tokens are counted


@pytest.mark.parametrize("temperature", [0.0, 0.9])
def test_running_ahead_changes_nothing_but_when_events_come(temperature):
    """With run_ahead the step after a decode step is launched before the host has read the first
    one's tokens: same tokens, same finishes, same pages given back -- with requests that end by a
    stop id (one step too far on the device), by length, one cancelled while a step is unread,
    others admitted when a slot frees, and under preemption."""
    def scenario(run_ahead):
        sched, ex = make(num_pages=8, max_requests=3, max_tokens=32, run_ahead=run_ahead)   # pages for 32 tokens
        prompts = {i: prompt(n, 10 + i) for i, n in enumerate([5, 9, 3, 7, 2])}
        free_run = expected_greedy(prompts[1], 12)
        for i, p in prompts.items():
            sched.submit(Request(id=i, prompt=p, max_new_tokens=[12, 12, 20, 9, 15][i],
                                 stop_ids=[free_run[5]] if i == 1 and temperature == 0.0 else [],
                                 sampling=SamplingParams(temperature=temperature, seed=i)))
        out, finish, steps = {}, {}, 0
        while not sched.idle():
            steps += 1
            assert steps < 400
            for e in sched.step():
                if e.token >= 0:
                    assert e.index == len(out.setdefault(e.id, []))
                    out[e.id].append(e.token)
                if e.finish:
                    finish[e.id] = e.finish
            if len(out.get(2, [])) == 6 and 2 not in finish and sched.cancel(2):
                finish[2] = "cancelled here"
        assert ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3
        return out, finish, ex, sched.stats()

    plain_out, plain_finish, _, plain_stats = scenario(False)
    out, finish, ex, stats = scenario(True)
    assert ex.ahead_steps > 10, "steps were expected to be launched from tokens the host had not read"
    cancelled = out.pop(2), plain_out.pop(2)
    assert cancelled[0][:6] == cancelled[1][:6]            # (how many more it got before the cancel may differ)
    assert out == plain_out and finish == plain_finish
    # (a request that runs one token too far, or is cancelled a step later, may tip a page decision:
    # the number of preemptions may differ, the tokens may not)
    assert stats.preemptions > 0 and plain_stats.preemptions > 0
    if temperature == 0.0:
        assert finish[1] == "stop" and len(out[1]) == 6


def test_running_ahead_leaves_rows_for_the_host_alone():
    """A request with top-k cannot have its tokens chosen on the device: no step runs ahead."""
    sched, ex = make(num_pages=12, run_ahead=True)
    sched.submit(Request(id=0, prompt=prompt(4, 1), max_new_tokens=8, sampling=SamplingParams(temperature=0.7, top_k=5, seed=3)))
    sched.submit(Request(id=1, prompt=prompt(6, 2), max_new_tokens=8))
    out, finish = run(sched)
    assert ex.ahead_steps == 0 and len(out[0]) == 8 and out[1] == expected_greedy(prompt(6, 2), 8)


def test_a_windowed_model_runs_in_a_pool_smaller_than_its_requests():
    """Every stream of the model keeps a window of 6 tokens only: a request of 30 tokens needs the window's
    pages and a portion's, not 30 tokens' worth, and is admitted and run in a pool of 3 pages (12 tokens);
    what it may need at most is the cache manager's answer, by the stream's own rule."""
    windowed = {0: PagedKV(1, 2, window=6), 1: PagedKV(1, 2, window=6)}
    sched, ex = make(num_pages=3, max_tokens=32, prefill_chunk=4, streams=windowed)
    assert ex.cache.peak_pages(29, 4) == {("window", 6): 3}
    p = prompt(20, 11)
    sched.submit(Request(id=0, prompt=p, max_new_tokens=10))
    out, finish = run(sched)
    assert out[0] == expected_greedy(p, 10) and finish[0] == "length"
    assert ex.cache.groups[("window", 6)].pool.high_water_mark == 3 and sched.stats().preemptions == 0
    # a portion too large for the pool beside the window is still refused, with the pool's size in the message
    wide, _ = make(num_pages=5, max_tokens=32, prefill_chunk=16, streams=windowed)
    assert "needs 6 KV pages, the pool holds 5" in wide.check(Request(id=1, prompt=prompt(20, 1), max_new_tokens=10))
    # beside a stream that keeps everything the request is held to that stream's need
    both, _ = make(num_pages=5, max_tokens=32, prefill_chunk=4, streams={0: PagedKV(1, 2), 1: PagedKV(1, 2, window=6)})
    assert "needs 8 KV pages" in both.check(Request(id=2, prompt=prompt(20, 2), max_new_tokens=10))


def test_a_model_that_keeps_nothing_per_token_needs_no_pages():
    from bare_cuda_4gib_amd.cache import FixedState
    sched, ex = make(num_pages=0, max_tokens=32, streams={0: FixedState((3,))})
    assert sched.limits.kv_pages == 0 and ex.cache.peak_pages(31, 6) == {}
    prompts = {i: prompt(n, 20 + i) for i, n in enumerate([9, 3, 14, 2])}
    for i, p in prompts.items():
        sched.submit(Request(id=i, prompt=p, max_new_tokens=5))
    out, finish = run(sched)
    for i, p in prompts.items():
        assert out[i] == expected_greedy(p, 5) and finish[i] == "length"
    assert sched.stats().preemptions == 0 and ex.cache.free_slots == 3


@pytest.mark.parametrize("run_ahead", [False, True])
def test_arrivals_are_gathered_while_others_decode(run_ahead):
    """gather_ms: a request that arrives while others decode waits until the first of the waiting has waited that
    long, and goes in together with those that came meanwhile, in one step -- so the steps between stay decode
    steps (which an engine replays from graphs and runs ahead).  Nothing is held back while nothing runs or while a
    prompt is under way; a request that lost its pages is not made to wait again; and the tokens are the same."""
    now = [0.0]

    def build(gather_ms):
        now[0] = 0.0
        return make(num_pages=64, max_requests=6, max_tokens=64, clock=lambda: now[0], run_ahead=run_ahead, gather_ms=gather_ms)

    prompts = {i: prompt(3 + i, 50 + i) for i in range(5)}

    def serve(gather_ms):
        sched, ex = build(gather_ms)
        out, finish, admitted_in = {}, {}, {}
        sched.submit(Request(id=0, prompt=prompts[0], max_new_tokens=30))       # nothing runs: in at once
        arrivals = {3: 1, 4: 2, 9: 3, 20: 4}                                     # step -> request that arrives before it
        for step in range(200):
            if step in arrivals:
                sched.submit(Request(id=arrivals[step], prompt=prompts[arrivals[step]], max_new_tokens=8))
            if sched.idle():
                break
            before = len(ex.batches)
            for e in sched.step():
                if e.token >= 0:
                    out.setdefault(e.id, []).append(e.token)
                if e.finish:
                    finish[e.id] = e.finish
            for batch in ex.batches[before:]:
                for rid, n in batch:
                    admitted_in.setdefault(rid, len(ex.batches))
            now[0] += 0.001                                                      # a millisecond a step
        assert sched.idle() and len(finish) == 5
        return out, admitted_in, ex.batches

    plain_out, plain_in, plain_batches = serve(0.0)
    out, admitted_in, batches = serve(5.0)
    assert out == plain_out == {i: expected_greedy(prompts[i], 30 if i == 0 else 8) for i in range(5)}
    assert plain_in[1] < plain_in[2] < plain_in[3]                               # one by one without gathering
    assert admitted_in[1] == admitted_in[2] and admitted_in[2] < admitted_in[3]  # 1 and 2 together: 2 came while 1 waited
    assert admitted_in[1] - plain_in[1] >= 4                                     # ... five milliseconds after 1 came
    mixed = lambda bs: sum(1 for b in bs if any(n > 1 for _, n in b))
    assert mixed(batches) < mixed(plain_batches)                                 # fewer steps that bring a prompt portion

    # nothing runs: nobody is held back, whatever the clock says
    sched, ex = build(1000.0)
    sched.submit(Request(id=7, prompt=prompts[1], max_new_tokens=2))
    sched.step()
    assert ex.batches and ex.batches[0] == [(7, len(prompts[1]))]
    # a long prompt under way: who comes now rides along at once
    sched, ex = build(1000.0)
    sched.submit(Request(id=1, prompt=prompt(20, 1), max_new_tokens=2))
    sched.step()
    sched.submit(Request(id=2, prompt=prompts[2], max_new_tokens=2))
    sched.step()
    assert (2, len(prompts[2])) in ex.batches[1]


def test_rare_arrivals_are_not_held_back():
    """Where requests come further apart than the wait (the running mean of the last gaps), nobody is to be expected
    for company: the arrival goes in with the next step, as without gathering."""
    now = [0.0]
    sched, ex = make(num_pages=64, max_requests=6, max_tokens=64, clock=lambda: now[0], gather_ms=5.0)
    sched.submit(Request(id=0, prompt=prompt(3, 1), max_new_tokens=60))
    for step in range(100):
        if step in (10, 40, 70):                                                  # thirty milliseconds apart
            sched.submit(Request(id=step, prompt=prompt(4, step), max_new_tokens=3))
            sched.step()
            assert (step, 4) in ex.batches[-1], f"the arrival before step {step} was held back"
        else:
            sched.step()
        now[0] += 0.001
    # ... and once they come in a burst again, they are gathered again
    burst = {}
    for i, rid in enumerate((200, 201, 202, 203)):
        sched.submit(Request(id=rid, prompt=prompt(4, rid), max_new_tokens=3))
        sched.step()
        now[0] += 0.001
        burst[rid] = any(r == rid for r, _ in ex.batches[-1])
    assert burst[200] and not burst[203]                                          # (by the fourth the mean gap is below the wait)


def test_a_request_that_lost_its_pages_is_not_made_to_wait_again():
    now = [0.0]
    sched, ex = make(num_pages=5, page_tokens=4, max_requests=3, max_tokens=20, clock=lambda: now[0], gather_ms=50.0)
    for i in range(2):
        sched.submit(Request(id=i, prompt=prompt(7, 80 + i), max_new_tokens=8))
    out, finish = {}, {}
    for step in range(300):
        if sched.idle():
            break
        for e in sched.step():
            if e.token >= 0:
                out.setdefault(e.id, []).append(e.token)
            if e.finish:
                finish[e.id] = e.finish
        now[0] += 0.001
    assert sched.idle() and sched.stats().preemptions >= 1
    assert out == {i: expected_greedy(prompt(7, 80 + i), 8) for i in range(2)}
    victim_back = [i for i, b in enumerate(ex.batches) if any(rid == 1 and n > 1 for rid, n in b)]
    assert len(victim_back) >= 2                                                 # its prompt ran twice
