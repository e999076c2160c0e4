"""The engine above the step function on the GPU: long decoding, the first tokens of a sequence,
greedy generation through the entry point and the command line, batching and preemption."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
from plain_llama import PlainLlama, argmax_lowest

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(rtol=1e-4, atol=2e-6), "bfloat16": dict(rtol=2e-2, atol=6e-3)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return lambda name, dtype, variant="ones": helpers.make_model_dir(tmp, name, dtype, variant=variant)


def follow_with_plain(plain, prompt, tokens, margin):
    """The engine's tokens, checked step by step against the plain logits of the engine's own
    sequence: each chosen token must be the plain argmax, or within `margin` of it (a near-tie
    that rounding may turn)."""
    ids = list(prompt)
    full = plain.logits(ids + list(tokens))
    for i, tok in enumerate(tokens):
        row = full[len(prompt) - 1 + i]
        gap = float(row.max() - row[tok])
        assert gap <= margin, f"token {i} ({tok}) lies {gap:.4g} below the plain best {argmax_lowest(row)}"


@pytest.mark.parametrize("variant", ["ones", "spread"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype, variant):
    """A short prompt, then several hundred tokens one by one (captured graphs, many pages)."""
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    folder = folders("C", dtype, variant)
    ids = helpers.random_ids(400, helpers.TINY_C["vocab_size"], 77)
    plain = PlainLlama(folder).logits(ids).numpy()
    model, _ = load_model(folder, dtype)
    ex = Executor(model, num_pages=26, max_requests=2, max_tokens=416, page_tokens=16, poison=True)
    ex.cache.shuffle_free_pages(3)
    ex.admit("r")
    got = {}
    rows = ex.step([StepEntry("r", ids[:3], [0, 1, 2])]).cpu().numpy()      # the first tokens of a sequence
    got.update({p: rows[p] for p in range(3)})
    for p in range(3, 400):
        got[p] = ex.step([StepEntry("r", [ids[p]], [0])]).cpu().numpy()[0]
    where = {(0, p): ("r", p) for p in range(400)}
    helpers.compare_with_plain({(0, p): got[p] for p in range(400)}, where, {"r": plain}, label=f"long {dtype}", **TOL[dtype])


@pytest.mark.parametrize("variant", ["ones", "spread"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_norms_prepared_by_the_product_before(folders, monkeypatch, name, variant):
    """In bfloat16 the product that adds into the residual stream prepares the norm that the next
    attention begins with (and, from 64 rows on, the feed-forward's): the path is taken -- the
    preparing kernel runs once a layer and step, none where no layer follows -- and the logits are
    those of the path without it up to rounding, and the plain implementation's, for decoded tokens
    alone, for 64 rows in a step (both norms prepared) and for portions beside decoded tokens."""
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.engine import Executor, load_model
    from bare_cuda_4gib_amd.parts.attention import CausalAttention
    from bare_cuda_4gib_amd.parts.feedforward import SwiGLU
    cfg = helpers.TINY[name][0]
    folder = folders(name, "bfloat16", variant)
    requests = {f"r{i}": helpers.random_ids(n, cfg["vocab_size"], 500 + i) for i, n in enumerate([75, 20, 9])}
    plain = PlainLlama(folder)
    plain_logits = {rid: plain.logits(ids).numpy() for rid, ids in requests.items()}
    model, _ = load_model(folder, "bfloat16")
    at = {rid: 0 for rid in requests}

    def entry(rid, n):
        e = {"id": rid, "tokens": requests[rid][at[rid]:at[rid] + n], "want": list(range(n)), "_start": at[rid]}
        at[rid] += n
        return e
    plan = [[("r0", 64)], [("r0", 1)], [("r0", 1), ("r1", 18)], [("r0", 1), ("r1", 1), ("r2", 9)], [("r0", 1), ("r1", 1)], [("r0", 1)]]
    steps = [{"step": i, "entries": [entry(rid, n) for rid, n in group], "end": []} for i, group in enumerate(plan)]
    steps, where = helpers._finish(steps)
    calls = []
    real = ops.gemm_accumulate_emit
    monkeypatch.setattr(ops, "gemm_accumulate_emit", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])

    def run():
        ex = Executor(model, num_pages=12, max_requests=4, max_tokens=128, page_tokens=16, poison=True, use_graphs=False)
        return helpers.replay_in_process(ex, steps)
    with_prepared = run()
    layers = cfg["num_hidden_layers"]
    assert len(calls) >= len(steps) * (layers - 1) and any(m >= 64 for m in calls) and any(m == 1 for m in calls)
    n_with = len(calls)
    monkeypatch.setattr(CausalAttention, "wants_prepared_norm", lambda self, n: False)
    monkeypatch.setattr(SwiGLU, "wants_prepared_norm", lambda self, n: False)
    without = run()
    assert len(calls) == n_with, "nothing is prepared for parts that do not want it"
    helpers.compare_with_plain(with_prepared, where, plain_logits, label=f"prepared norms {name}", **TOL["bfloat16"])
    for key in with_prepared:
        torch.testing.assert_close(torch.from_numpy(with_prepared[key]), torch.from_numpy(without[key]), rtol=2e-2, atol=4e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoded_tokens_at_long_contexts_beside_prompt_portions(folders, dtype):
    """Requests with hundreds of cached tokens decode one token each in the same step in which others
    bring portions of their prompts: in bfloat16 the decoded rows then get an attention launch of their
    own (keys cut between a workgroup's waves and over workgroups) into the same output as the
    portions' launch.  Every row's logits against the plain implementation; one decoding request
    stays below the context at which that happens and goes with the portions."""
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    folder = folders("C", dtype)
    vocab = helpers.TINY_C["vocab_size"]
    plain = PlainLlama(folder)
    model, _ = load_model(folder, dtype)
    ex = Executor(model, num_pages=80, max_requests=6, max_tokens=512, page_tokens=16, poison=True)
    ex.cache.shuffle_free_pages(9)
    ids = {"far": helpers.random_ids(460, vocab, 1), "mid": helpers.random_ids(300, vocab, 2),
           "near": helpers.random_ids(40, vocab, 3), "p1": helpers.random_ids(90, vocab, 4),
           "p2": helpers.random_ids(37, vocab, 5)}
    want = {r: plain.logits(t).numpy() for r, t in ids.items()}
    done = {"far": 450, "mid": 290, "near": 30, "p1": 0, "p2": 0}
    for r in ("far", "mid", "near"):
        ex.admit(r)
        ex.step([StepEntry(r, ids[r][:done[r]], [])])
    ex.admit("p1"), ex.admit("p2")
    portions = {"p1": [33, 2, 40, 15], "p2": [5, 20, 12]}
    tol = TOL[dtype]
    for step in range(4):
        entries, rows = [], []
        for r in ("p1", "far", "near", "p2", "mid"):
            n = 1 if r in ("far", "mid", "near") else (portions[r][step] if step < len(portions[r]) else 0)
            if n == 0:
                continue
            entries.append(StepEntry(r, ids[r][done[r]:done[r] + n], list(range(n))))
            rows += [(r, done[r] + i) for i in range(n)]
            done[r] += n
        got = ex.step(entries).float().cpu().numpy()
        for row, (r, pos) in enumerate(rows):
            w = want[r][pos]
            assert abs(got[row] - w).max() <= tol["atol"] + tol["rtol"] * abs(w).max(), f"step {step}: {r} at {pos}"


@pytest.mark.parametrize("graphs", [True, False])
def test_tokens_taken_on_the_device_give_the_same_sequence(folders, graphs):
    """Decoding with every step's tokens taken from the ids the step before chose, on the device
    (the host sees them a step late), gives the ids of decoding with the host in between."""
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    folder = folders("B", "bfloat16")
    model, _ = load_model(folder, "bfloat16")
    vocab = helpers.TINY_B["vocab_size"]
    prompts = [helpers.random_ids(n, vocab, 60 + n) for n in (5, 17, 2)]

    def start():
        ex = Executor(model, num_pages=12, max_requests=3, max_tokens=64, page_tokens=16)
        ex.use_graphs = ex.use_graphs and graphs
        first = []
        for i, ids in enumerate(prompts):
            ex.admit(i)
            first.append(int(ops.argmax(ex.step([StepEntry(i, ids, [len(ids) - 1])]))[0]))
        return ex, first

    ex, last = start()
    by_host = []
    for _ in range(30):
        last = ops.argmax(ex.step([StepEntry(i, [last[i]], [0]) for i in range(3)])).tolist()
        by_host.append(last)
    ex, first = start()
    ids = torch.tensor(first, dtype=torch.int32, device="cuda:0")
    entries = [StepEntry(i, [0], [0]) for i in range(3)]
    on_device = []
    for _ in range(30):
        ids = ops.argmax(ex.step(entries, device_tokens=ids))
        on_device.append(ids)                       # read only after everything has been launched
    assert [t.tolist() for t in on_device] == by_host
    with pytest.raises(Exception, match="device_tokens"):
        ex.step(entries[:2], device_tokens=ids)


def test_decode_step_description_from_the_arrays_by_slot(folders):
    """A step of decoded tokens is described to the device from the cache manager's arrays by slot;
    the description is, number for number, the one the general builder makes -- for requests of
    different lengths, in another order than their slots, across page edges, with one left out."""
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    folder = folders("A", "bfloat16")
    model, _ = load_model(folder, "bfloat16")
    ex = Executor(model, num_pages=40, max_requests=6, max_tokens=96, page_tokens=16)
    assert ex.use_graphs
    vocab = helpers.TINY_A["vocab_size"]
    names = ["a", "b", "c", "d", "e"]
    for i, r in enumerate(names):
        ex.admit(r)
        ex.step([StepEntry(r, helpers.random_ids(3 + 6 * i, vocab, 40 + i), [])])
    ex.release("b")
    ex.admit("f")
    ex.step([StepEntry("f", helpers.random_ids(15, vocab, 50), [])])
    width = ex.cache.max_pages_per_request
    for step in range(40):
        order = [r for r in ("e", "a", "f", "d", "c") if not (r == "d" and step % 3 == 0)]
        entries = [StepEntry(r, [(7 * step + j) % vocab], [0]) for j, r in enumerate(order)]
        ex.cache.reserve([(e.request, 1) for e in entries])
        want = ex._host_arrays(entries, table_width=width, all_logits=True)[0].tolist()
        ex.step(entries)
        used = [slot for slot in ex._graphs.values() if slot["next"] and len(slot["rows"]) == len(entries)]
        latest = [s["ring"][(s["next"] - 1) % len(s["ring"])][1].tolist() for s in used]
        assert want in latest, f"step {step}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_one_by_one(folders, dtype):
    """Positions 0, 1, 2, ... each as a step of its own: one key, then two, then three."""
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    folder = folders("A", dtype)
    ids = helpers.random_ids(6, 256, 5)
    plain = PlainLlama(folder).logits(ids).numpy()
    model, _ = load_model(folder, dtype)
    ex = Executor(model, num_pages=1, max_requests=1, max_tokens=64, page_tokens=64)
    ex.admit(0)
    got = {(0, p): ex.step([StepEntry(0, [ids[p]], [0])]).cpu().numpy()[0] for p in range(6)}
    helpers.compare_with_plain(got, {(0, p): ("r", p) for p in range(6)}, {"r": plain}, label="first", **TOL[dtype])


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    cfg, _ = helpers.TINY[name]
    folder = folders(name, dtype)
    plain = PlainLlama(folder)
    prompts = [helpers.random_ids(n, cfg["vocab_size"], 10 + n) for n in (1, 7, 33)]   # the first tiny configuration's workload
    engine = Engine(folder, max_tokens=64, max_seqs=3, kv_pages=0, dtype=dtype, page_tokens=16, prefill_chunk=16)
    assert engine.vocab_size == cfg["vocab_size"] and engine.max_seqs == 3 and engine.healthy
    together = generate_batch(engine, prompts, 16)
    margin = 0.0 if dtype == "float32" else 2e-2
    for p, toks in zip(prompts, together):
        assert len(toks) == 16
        follow_with_plain(plain, p, toks, margin + 1e-6)
    if dtype == "float32":
        assert together == [plain.greedy(p, 16) for p in prompts]
    alone = [generate_batch(engine, [p], 16)[0] for p in prompts]
    if dtype == "float32":
        assert alone == together, "a request's tokens must not depend on what else is in the batch"
    else:
        # other row counts may choose other kernels, which differ by rounding: a request alone may turn a
        # near-tie the other way, so its tokens are held to the plain logits of its own sequence, like the batch's
        # (the reference re-scores such a divergence by its logit gap too, bench/src/batch_check_main.cc:110-148)
        for p, toks in zip(prompts, alone):
            assert len(toks) == 16
            follow_with_plain(plain, p, toks, margin + 1e-6)
    stats = engine.stats()
    assert stats["kv_pages_used"] == 0 and stats["running"] == 0 and stats["prefill_tokens"] == 2 * sum(map(len, prompts))


def test_engine_from_a_configuration_and_a_seed(folders):
    """Engine.from_config writes the model folder by the random-weights mode and loads it: the
    same tokens as the engine over the folder the tests wrote with the same seed."""
    from bare_cuda_4gib_amd.engine.engine import Engine, generate_batch
    cfg, seed = helpers.TINY["A"]
    prompts = [helpers.random_ids(n, cfg["vocab_size"], 90 + n) for n in (3, 11)]
    over_folder = generate_batch(Engine(folders("A", "bfloat16"), max_tokens=32, max_seqs=2), prompts, 8)
    fresh = Engine.from_config(cfg, seed, "bfloat16", max_tokens=32, max_seqs=2)
    assert generate_batch(fresh, prompts, 8) == over_folder


def test_entry_point_statuses_and_failure_path(folders):
    from bare_cuda_4gib_amd.engine import Engine
    engine = Engine(folders("A", "bfloat16"), max_tokens=32, max_seqs=1, max_waiting=1, page_tokens=16)
    assert engine.submit(1, [], 4)[0] == "invalid"
    assert engine.submit(1, [1] * 40, 4)[0] == "invalid"
    assert engine.submit(1, [999], 4)[0] == "invalid"                              # outside the vocabulary
    assert engine.submit(1, [1, 2], 4, temperature=-1.0)[0] == "invalid"
    assert engine.submit(1, [1, 2, 3], 4) == ("ok", "")
    assert engine.submit(1, [1, 2, 3], 4)[0] == "invalid"                          # id in use
    assert engine.submit(2, [4, 5], 4, stop_ids=[7])[0] == "ok"
    assert engine.submit(3, [4, 5], 4)[0] == "busy"                                # max_seqs + max_waiting live
    events = engine.poll()
    assert events and events[0][0] == 1 and events[0][2] == 0 and events[0][3] == ""
    engine.cancel(2)
    assert (2, -1, -1, "cancelled") in engine.poll() + engine.poll()
    engine._fail_for_test("injected")
    while True:
        ev = engine.poll()
        if any(e[3] == "error" for e in ev):
            assert ev[-1][:3] == (1, -1, -1)
            break
        assert ev, "the failure must surface"
    assert not engine.healthy and "injected" in engine.failure
    assert engine.submit(9, [1], 1)[0] == "unavailable"


def follow_sampled_with_plain(plain, prompt, tokens, temperature, seed, logit_tol):
    """The engine's sampled tokens, checked step by step against the law (engine/src/sampler.cpp:39-61)
    applied to the plain logits of the engine's own sequence: weights exp((l - max) / T), their running
    sum in vocabulary order, and u * total with u from a fresh generator of the request's seed.  The
    engine's token must be the one in whose stretch of the running sum u * total falls -- or one next
    to it when u * total lies so close to the stretch's edge that the rounding of the engine's logits
    (logit_tol: rtol and atol of the logits in this precision) can move the edge across it.  Returns how
    many tokens were exactly the plain choice."""
    from bare_cuda_4gib_amd.sampling import MT19937_64
    rng = MT19937_64(seed)
    full = plain.logits(list(prompt) + list(tokens)).numpy()
    exact = 0
    for i, tok in enumerate(tokens):
        row = full[len(prompt) - 1 + i]
        w = np.exp((row - row.max()) / temperature)
        cum = np.cumsum(w)
        total = cum[-1]
        target = rng.uniform() * total
        want = int(np.nonzero(target - cum < 0.0)[0][0])
        exact += tok == want
        # a logit off by e moves its weight by a factor exp(e / T): every edge of the running sum by at most
        # 2 e / T of the total (the maximum's own error included)
        margin = 2.0 * (logit_tol["rtol"] * float(np.abs(row).max()) + logit_tol["atol"]) / temperature * total
        low = cum[tok - 1] if tok > 0 else 0.0
        assert low - margin <= target < cum[tok] + margin, (
            f"token {i}: the engine drew {tok}, the law gives {want} (u * total = {target:.6g}, the engine's token "
            f"spans [{low:.6g}, {cum[tok]:.6g}), margin {margin:.3g})")
    return exact


def test_sampled_tokens_follow_the_law_on_the_plain_logits(folders):
    """Configuration B's workload -- prompts of 5, 64 and 130 tokens as one mixed batch with 32-token
    portions, 24 tokens each at temperature 0.8: every token the engine draws is the one the sampling
    law gives on the plain implementation's logits for the request's own generator (the k-th token
    uses the generator's k-th number, whatever else is in the batch).  In 32-bit the check is sharp
    (a token spans 1/384 of the running sum, the margin is a fifteenth of that): a draw from another
    request's row, with another request's generator or with the temperature applied twice gives
    other tokens, which the test shows.  (In bfloat16 the logits' tolerance would make the margin wider
    than a token: there the draw is held, exactly, to the law on the engine's own logits instead,
    test_serving_gpu.py::test_sampled_tokens_are_the_law_on_the_engine_s_own_logits.)"""
    dtype = "float32"
    from bare_cuda_4gib_amd.engine import Engine
    folder = folders("B", dtype, "spread")
    plain = PlainLlama(folder)
    prompts = [helpers.random_ids(n, 384, 40 + n) for n in (5, 64, 130)]
    engine = Engine(folder, max_tokens=256, max_seqs=3, kv_pages=0, dtype=dtype, page_tokens=16, prefill_chunk=32,
                    max_batch_tokens=96)
    for i, p in enumerate(prompts):
        assert engine.submit(i, p, 24, temperature=0.8, seed=4 + i)[0] == "ok"
    out = {}
    while len(out) < 3 or any(len(v) < 24 for v in out.values()):
        for id, tok, idx, fin in engine.poll():
            out.setdefault(id, []).append(tok)
    exact = sum(follow_sampled_with_plain(plain, prompts[i], out[i], 0.8, 4 + i, TOL[dtype]) for i in range(3))
    assert exact >= 66, f"only {exact} of 72 tokens are the plain choice"
    # the check bites: the same tokens against another request's generator, a temperature applied
    # twice, or another request's tokens (its rows) fail
    with pytest.raises(AssertionError):
        follow_sampled_with_plain(plain, prompts[1], out[1], 0.8, 4 + 2, TOL[dtype])
    with pytest.raises(AssertionError):
        follow_sampled_with_plain(plain, prompts[1], out[1], 0.8 * 0.8, 4 + 1, TOL[dtype])
    with pytest.raises(AssertionError):
        follow_sampled_with_plain(plain, prompts[1], out[2], 0.8, 4 + 2, TOL[dtype])


def test_sampling_and_preemption_on_the_device(folders):
    """Temperature sampling on the device: a seed gives the same tokens alone, batched, and when the
    pool is so small that requests are preempted and recomputed."""
    from bare_cuda_4gib_amd.engine import Engine, generate_batch
    folder = folders("B", "float32", "spread")
    prompts = [helpers.random_ids(n, 384, 40 + n) for n in (5, 64, 130)]            # the second tiny configuration's workload
    def run(kv_pages, which):
        engine = Engine(folder, max_tokens=256, max_seqs=3, kv_pages=kv_pages, dtype="float32", page_tokens=16,
                        prefill_chunk=32, max_batch_tokens=96)
        out = {}
        for i in which:
            assert engine.submit(i, prompts[i], 24, temperature=0.8, seed=4 + i)[0] == "ok"
        while len(out) < len(which) or any(len(v) < 24 for v in out.values()):
            for id, tok, idx, fin in engine.poll():
                out.setdefault(id, []).append(tok)
        return out, engine.stats()
    roomy, _ = run(0, [0, 1, 2])
    tight, stats = run(13, [0, 1, 2])                                               # 208 tokens of pool for 5+64+130+3*23
    assert stats["preemptions"] >= 1 and stats["kv_pages_used"] == 0
    assert tight == roomy
    assert run(0, [1])[0][1] == roomy[1]
    again, _ = run(0, [0, 1, 2])
    assert again == roomy and len(set(roomy[2])) > 3                                # repeatable, and really sampled


def test_command_line(folders, tmp_path):
    folder = folders("A", "float32")
    prompt = helpers.random_ids(7, 256, 1)
    proc = subprocess.run([sys.executable, os.path.join(helpers.ROOT, "bin", "llm-infer"), "--model", folder,
                           "--prompt", ",".join(map(str, prompt)), "--tokens", "5", "--dtype", "float32",
                           "--page-tokens", "16", "--kv-pages", "3"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    assert lines[0].startswith("[llm] 2 layers, hidden 64, vocab 256") and lines[1].split() == ["prompt:"] + [str(t) for t in prompt]
    assert "(3 pages, max batch 1)" in lines[0]
    assert [int(t) for t in lines[2].split()[1:]] == PlainLlama(folder).greedy(prompt, 5)
    bad = subprocess.run([sys.executable, os.path.join(helpers.ROOT, "bin", "llm-infer"), "--model", str(tmp_path / "none"),
                          "--prompt", "1,2"], capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "config.json" in bad.stderr


def test_missing_kernel_library_fails_loudly(monkeypatch):
    from bare_cuda_4gib_amd.csrc import build, library
    from bare_cuda_4gib_amd.errors import KernelError
    monkeypatch.setattr(library, "_lib", None)
    monkeypatch.setattr(build, "LIB_PATH", "/nonexistent/libbc4g.so")
    with pytest.raises(KernelError):
        library.load(build_if_missing=False)


def test_cpu_tensors_are_refused():
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.errors import KernelError
    with pytest.raises(KernelError):
        ops.rmsnorm(torch.zeros(2, 8), torch.ones(8), 1e-5, torch.float32)
