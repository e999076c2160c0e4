"""Serving schedules on the GPU that the other engine tests do not reach: a live count that wanders
(captured graphs of a few sizes, filled up with rows that stand for no request), a request that meets a
stop id while the step after it is already running into pages its end gives back, sampled tokens
against the law on the engine's own logits, and the executor's refusal of more tokens than the model
has positions."""
import numpy as np
import pytest
import torch

import helpers
from plain_llama import PlainLlama, argmax_lowest

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(rtol=1e-4, atol=2e-6), "bfloat16": dict(rtol=2e-2, atol=6e-3)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("serving")
    return lambda name, dtype, variant="ones": helpers.make_model_dir(tmp, name, dtype, variant=variant)


def record_steps(engine):
    """Wraps the engine's step function: every step's entries (request, position of each wanted row) with
    a copy of the logits it returned, and the requests' cached lengths as the step found them."""
    ex = engine.executor
    real = ex.step
    log = []

    def step(entries, device_tokens=None):
        rows = [(e.request, ex.length(e.request) + int(w)) for e in entries for w in e.want]
        before = {e.request: ex.length(e.request) for e in entries}
        group = next(iter(ex.cache.groups), None)
        logits = real(entries, device_tokens=device_tokens)
        log.append(dict(rows=rows, logits=None if logits is None else logits.float().cpu().numpy().copy(),
                        before=before, ahead=device_tokens is not None, n=len(entries),
                        pages={e.request: [p for p in ex.cache.table(group, e.request) if p >= 0] for e in entries} if group is not None else {},
                        decode=all(len(e.tokens) == 1 for e in entries)))
        return logits
    ex.step = step
    return log


def drain(engine, n_requests):
    out, finish = {}, {}
    while len(finish) < n_requests:
        events = engine.poll()
        assert events or not engine.idle(), "the engine went idle before every request had finished"
        for id, tok, idx, fin in events:
            if tok >= 0:
                assert idx == len(out.setdefault(id, []))
                out[id].append(tok)
            if fin:
                finish[id] = fin
    return out, finish


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_wandering_live_count_needs_few_graphs(folders, dtype):
    """Thirty requests whose lengths are spread from 4 to 62 new tokens, 24 live at a time: as they end one by
    one and the waiting ones come in, the number of decoding requests takes nearly every value from 24 down to 1.
    Decode steps run in graphs of 1..8, 12, 16 and 24 rows -- a step of 19 requests in the graph of 24, the
    rows beyond its own standing for no request -- so eleven graphs serve what would else be twenty-four.
    The tokens are those of the same engine without graphs (32-bit: the same ids; bfloat16: each within a
    rounding of the plain argmax), and the plain implementation's."""
    from bare_cuda_4gib_amd.engine import Engine
    cfg, _ = helpers.TINY["A"]
    folder = folders("A", dtype)
    plain = PlainLlama(folder)
    n = 30
    prompts = [helpers.random_ids(3 + (7 * i) % 23, cfg["vocab_size"], 3000 + i) for i in range(n)]
    new = [4 + 2 * i for i in range(n)]
    runs = {}
    for graphs in (True, False):
        engine = Engine(folder, max_tokens=96, max_seqs=24, kv_pages=0, dtype=dtype, page_tokens=16, prefill_chunk=32,
                        max_batch_tokens=128, max_waiting=0)
        engine.executor.use_graphs = engine.executor.use_graphs and graphs
        assert engine.executor.use_graphs == graphs
        log = record_steps(engine)
        for i in range(n):
            assert engine.submit(i, prompts[i], new[i])[0] == "ok"
        out, finish = drain(engine, n)
        assert all(finish[i] == "length" and len(out[i]) == new[i] for i in range(n))
        runs[graphs] = out
        if graphs:
            counts = {s["n"] for s in log if s["decode"]}
            assert len(counts) >= 18 and max(counts) >= 20 and min(counts) == 1, f"the live count was meant to wander, took {sorted(counts)}"
            assert any(c not in engine.executor.GRAPH_ROWS for c in counts), "no step needed rows that stand for no request"
            keys = sorted(engine.executor._graphs)
            assert engine.executor.captures == len(keys) <= 11 < len(counts), f"{engine.executor.captures} captures for {keys}"
            assert {k[0] for k in keys} <= {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24}
        assert engine.stats()["kv_pages_used"] == 0
    margin = 0.0 if dtype == "float32" else 2e-2
    for i in range(n):
        for which in (True, False):
            full = plain.logits(prompts[i] + runs[which][i])
            for j, tok in enumerate(runs[which][i]):
                row = full[len(prompts[i]) - 1 + j]
                assert float(row.max() - row[tok]) <= margin + 1e-6, \
                    f"request {i}, token {j} (graphs {which}): {tok} lies below the plain best {argmax_lowest(row)}"
    if dtype == "float32":
        assert runs[True] == runs[False]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_stop_id_met_while_the_next_step_already_runs(folders, dtype):
    """Two slots, so the third request can only come in once the first has ended.  Request 0 is stopped by a
    token that it would generate freely a few steps in; the engine launches a decode step before it has read the
    ids of the one before, so request 0 runs one token beyond its stop, into pages that its end then gives back
    and that request 2 takes over at once (the pool hands out first what was freed last).  The tokens of all
    three and the logits of the neighbour (request 1, beside request 0 all the time) and of request 2 (in
    request 0's pages) are the plain implementation's."""
    from bare_cuda_4gib_amd.engine import Engine
    cfg, _ = helpers.TINY["A"]                      # (an output head of its own: greedy tokens that vary)
    vocab = cfg["vocab_size"]
    folder = folders("A", dtype, "spread")
    plain = PlainLlama(folder)
    prompts = [helpers.random_ids(n, vocab, 4100 + n) for n in (20, 30, 40)]
    new = [30, 26, 10]
    free_run = plain.greedy(prompts[0], 12)
    stops = [j for j in range(3, 10) if free_run[j] not in free_run[:j]]
    assert stops, f"pick other seeds: no token of {free_run} first appears between the fourth and the tenth place"
    at = stops[0]                                   # request 0 ends with its (at + 1)-th token
    stop = free_run[at]
    engine = Engine(folder, max_tokens=96, max_seqs=2, kv_pages=8, dtype=dtype, page_tokens=16, prefill_chunk=64,
                    max_batch_tokens=128)
    log = record_steps(engine)
    assert engine.submit(0, prompts[0], new[0], stop_ids=[stop])[0] == "ok"
    assert engine.submit(1, prompts[1], new[1])[0] == "ok"
    assert engine.submit(2, prompts[2], new[2])[0] == "ok"
    out, finish = drain(engine, 3)
    assert finish == {0: "stop", 1: "length", 2: "length"}
    # request 0 was run one token too far: if every step waited for the ids of the one before, its at + 1 generated
    # tokens would make prompt + at cached ones at most (the last generated token is never run); a step found it
    # with that many and ran one more
    assert any(s["ahead"] for s in log), "no step was launched ahead of the ids before it"
    assert max(s["before"].get(0, 0) for s in log) == len(prompts[0]) + at, "request 0 was not run beyond its stop token"
    # request 2 came in only after request 0 had ended
    first_2 = min(i for i, s in enumerate(log) if 2 in s["before"])
    last_0 = max(i for i, s in enumerate(log) if 0 in s["before"])
    assert first_2 > last_0 and set(log[first_2]["pages"][2]) >= set(log[last_0]["pages"][0]), "request 2 was meant to get request 0's pages"
    margin = 0.0 if dtype == "float32" else 2e-2
    if dtype == "float32":
        assert out[0] == free_run[:at + 1] and out[1] == plain.greedy(prompts[1], new[1]) and out[2] == plain.greedy(prompts[2], new[2])
    full = {i: plain.logits(prompts[i] + out[i]).numpy() for i in range(3)}
    for i in range(3):
        for j, tok in enumerate(out[i]):
            row = full[i][len(prompts[i]) - 1 + j]
            assert float(row.max() - row[tok]) <= margin + 1e-6, f"request {i}, token {j}: {tok} lies below the plain best"
    got, where = {}, {}
    for k, s in enumerate(log):
        for r, (rid, pos) in enumerate(s["rows"]):
            if rid in (1, 2) and pos < len(prompts[rid]) + len(out[rid]):
                got[(k, r)], where[(k, r)] = s["logits"][r], (rid, pos)
    assert len(where) >= new[1] + new[2]
    helpers.compare_with_plain(got, where, full, label=f"beside and after a stopped request, {dtype}", **TOL[dtype])
    assert engine.stats()["kv_pages_used"] == 0


@pytest.mark.parametrize("filters", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sampled_tokens_are_the_law_on_the_engine_s_own_logits(folders, dtype, filters):
    """Three requests in one mixed batch, each with a temperature -- and, with `filters`, one with a top-k, one
    with a top-p, one with both, which the device draws by the law for filtered rows, the step after running
    ahead all the same: every id the engine draws on the device is, exactly, the id that the host's sampler (the
    reference's law) draws from the very logits row the step returned, with the request's own generator -- in
    bfloat16 too, where the logits' tolerance against the plain implementation is wider than a token's share of
    the running sum and that comparison cannot bite."""
    from bare_cuda_4gib_amd.engine import Engine
    from bare_cuda_4gib_amd.sampling import MT19937_64, SamplingParams, sample_token
    folder = folders("B", dtype, "spread")
    prompts = [helpers.random_ids(n, 384, 40 + n) for n in (5, 64, 130)]
    how = [dict(temperature=0.8), dict(temperature=0.8), dict(temperature=0.8)]
    if filters:
        how = [dict(temperature=0.8, top_k=7), dict(temperature=1.3, top_p=0.8), dict(temperature=1.0, top_k=40, top_p=0.95)]
    engine = Engine(folder, max_tokens=256, max_seqs=3, kv_pages=0, dtype=dtype, page_tokens=16, prefill_chunk=32,
                    max_batch_tokens=96)
    log = record_steps(engine)
    for i, p in enumerate(prompts):
        assert engine.submit(i, p, 24, seed=4 + i, **how[i])[0] == "ok"
    out, _ = drain(engine, 3)
    assert any(s["ahead"] for s in log)                 # steps were launched before the tokens of the last had been read
    rngs = {i: MT19937_64(4 + i) for i in range(3)}
    drawn = {i: [] for i in range(3)}
    for s in log:                                # the steps in order: a request's k-th wanted row gets its generator's k-th number
        for r, (rid, pos) in enumerate(s["rows"]):
            if len(drawn[rid]) < 24:
                drawn[rid].append(sample_token(s["logits"][r], SamplingParams(**how[rid]), rngs[rid]))
    assert drawn == out
    assert len(set(out[2])) > 3
    # the check bites: another request's generator gives other ids from the same rows
    other = MT19937_64(4 + 2)
    rows_1 = [s["logits"][r] for s in log for r, (rid, _) in enumerate(s["rows"]) if rid == 1][:24]
    assert [sample_token(row, SamplingParams(**how[1]), other) for row in rows_1] != out[1]


def test_more_tokens_than_the_model_has_positions_are_refused(folders):
    """(Reference: Model::load refuses max_tokens beyond max_seq_len, engine/src/model.cpp:429-433.)"""
    from bare_cuda_4gib_amd.engine import Executor, load_model
    from bare_cuda_4gib_amd.errors import EngineError
    model, cfg = load_model(folders("A", "float32"), "float32")
    assert model.max_seq_len == helpers.TINY_A["max_position_embeddings"] == 128
    Executor(model, num_pages=2, max_requests=1, max_tokens=128, page_tokens=64)
    with pytest.raises(EngineError, match="beyond the model's 128 positions"):
        Executor(model, num_pages=3, max_requests=1, max_tokens=129, page_tokens=64)
    # the replay program alone may ask for more (it feeds given ids and serves nobody)
    Executor(model, num_pages=3, max_requests=1, max_tokens=129, page_tokens=64, beyond_positions=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_worker_thread_serves_while_the_callers_do_other_things(folders, dtype):
    """With a worker of its own the engine is the reference's (engine/src/async_engine.cpp:22-205): any thread
    submits, tokens are generated while nobody polls, poll waits up to its time-out and no longer, a cancelled
    request gets its last event and gives its pages back, a failure ends every live request with 'error', and
    stop joins the worker.  The tokens are those of the engine whose turns the polling thread runs."""
    import threading
    import time
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder = folders("A", dtype, "spread")
    vocab = helpers.TINY_A["vocab_size"]
    prompts = [helpers.random_ids(n, vocab, 70 + n) for n in (3, 40, 17, 64, 9)]
    args = dict(max_tokens=128, max_seqs=3, dtype=dtype, page_tokens=16, prefill_chunk=32, max_batch_tokens=96)
    inline = generate_batch(Engine(folder, **args), prompts, 20)

    engine = Engine(folder, worker=True, **args)
    t0 = time.monotonic()
    assert engine.poll(60) == [] and 0.05 <= time.monotonic() - t0 < 1.0        # nothing to wait for but the time
    with engine._in:                                   # all five before the worker's next turn, as before the first poll
        assert [engine.submit(i, p, 20) for i, p in enumerate(prompts)] == [("ok", "")] * 5
    assert engine.submit(1, prompts[1], 20)[0] == "invalid"                      # id in use
    deadline = time.monotonic() + 60
    while engine._live:                                                          # nobody polls; the worker goes on
        assert time.monotonic() < deadline, "the worker does not generate by itself"
        time.sleep(0.01)
    assert len(engine._outbox) >= 5 * 20
    out = {i: [] for i in range(5)}
    finish = {}
    while len(finish) < 5:
        events = engine.poll(1000)
        assert events, "a second without an event"
        for id, tok, idx, fin in events:
            if tok >= 0:
                assert idx == len(out[id])
                out[id].append(tok)
            if fin:
                finish[id] = fin
    assert [out[i] for i in range(5)] == inline and set(finish.values()) == {"length"}
    assert engine.idle() and engine.stats()["kv_pages_used"] == 0 and engine.stats()["waiting"] == 0

    # a request from another thread, cancelled while it runs
    results = []
    other = threading.Thread(target=lambda: results.append(engine.submit(7, prompts[2], 100)))
    other.start()
    other.join()
    assert results == [("ok", "")]
    first = engine.poll(5000)
    assert first and first[0][:1] == (7,) and first[0][3] == ""
    engine.cancel(7)
    engine.cancel(99)                                                             # no such request: nothing happens
    seen = []
    while not any(e[3] for e in seen):
        got = engine.poll(5000)
        assert got, "the cancellation never arrived"
        seen += got
    assert seen[-1] == (7, -1, -1, "cancelled") and len(seen) < 100
    while engine.stats()["kv_pages_used"]:
        assert time.monotonic() < deadline + 60
        time.sleep(0.01)
    assert engine.idle()

    # a failure on the worker's thread
    assert engine.submit(8, prompts[3], 60)[0] == "ok" and engine.submit(9, prompts[0], 60)[0] == "ok"
    engine._fail_for_test("injected")
    seen = []
    while sum(1 for e in seen if e[3] == "error") < 2:
        got = engine.poll(5000)
        assert got, "the failure must surface"
        seen += got
    assert [e[:3] for e in seen if e[3] == "error"] == [(8, -1, -1), (9, -1, -1)]
    assert not engine.healthy and "injected" in engine.failure
    assert engine.submit(10, [1], 1) == ("unavailable", "engine failed: injected")
    engine._thread.join(10)
    assert not engine._thread.is_alive()                                          # the worker ends with the failure
    engine.stop()
    assert engine.poll(10_000) == []                                              # stopped: no waiting

    # stop with work in flight
    engine = Engine(folder, worker=True, **args)
    assert engine.submit(1, prompts[3], 60)[0] == "ok"
    assert engine.poll(5000)
    engine.stop()
    assert not engine._thread.is_alive() and engine.submit(2, [1], 1) == ("unavailable", "engine is stopped")
    engine.poll(0)
    t0 = time.monotonic()
    assert engine.poll(10_000) == [] and time.monotonic() - t0 < 1.0
    assert engine.executor.cache.pages_in_use() == 0
