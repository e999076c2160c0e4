"""Replay on the GPU against the plain implementation: each request alone and whole; most of it
in one step and the last 32 tokens one by one; in portions of changing size down to two tokens;
and mixed, up to four live requests with so few pages that they are used again -- in 32-bit and
in bfloat16, for every tiny configuration, on folders whose norm scales are all 1.0 (the benchmark's
configurations) and on folders whose norm scales are drawn around 1.0, a draw for every norm, with
peaked attention (a scale that reaches the wrong norm, or none, changes these logits)."""
import pytest

import helpers
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu

# Tolerances, fixed beforehand.  32-bit: the engine's float arithmetic against float64, logits
# of magnitude ~0.2.  bfloat16: activations between kernels carry 8 bits, logits of magnitude
# ~0.2 come out within a few 1e-3.
TOL = {"float32": dict(rtol=1e-4, atol=2e-6), "bfloat16": dict(rtol=2e-2, atol=6e-3)}
LENGTHS = {"A": [1, 7, 33, 100, 128], "B": [5, 64, 130, 201], "C": [2, 77, 150, 260]}


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """name, dtype, variant -> (model folder, requests, plain logits per request)."""
    tmp = tmp_path_factory.mktemp("models")
    cache = {}

    def get(name, dtype, variant="ones"):
        key = (name, dtype, variant)
        if key not in cache:
            cfg, _ = helpers.TINY[name]
            folder = helpers.make_model_dir(tmp, name, dtype, variant=variant)
            requests = {f"r{i}": helpers.random_ids(n, cfg["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS[name])}
            plain = PlainLlama(folder)
            logits = {rid: plain.logits(ids).numpy() for rid, ids in requests.items()}
            cache[key] = (folder, requests, logits)
        return cache[key]
    return get


def _executor(folder, dtype, num_pages, page_tokens):
    """An executor whose requests may grow to the model's positions (the longest request of every configuration
    is as long as, or a little shorter than, that)."""
    from bare_cuda_4gib_amd.engine import Executor, load_model
    model, _ = load_model(folder, dtype, "cuda:0")
    max_tokens = model.max_seq_len
    ex = Executor(model, num_pages=num_pages, max_requests=6, max_tokens=max_tokens, page_tokens=page_tokens,
                  poison=True)
    ex.cache.shuffle_free_pages(7)
    return ex


CASES = [(n, d, v) for v in ("ones", "spread") for n in ("A", "B", "C") for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype,variant", CASES)
def test_whole(setups, name, dtype, variant):
    folder, requests, plain = setups(name, dtype, variant)
    steps, where = helpers.trace_whole(requests)
    ex = _executor(folder, dtype, num_pages=20, page_tokens=16)
    got = helpers.replay_in_process(ex, steps)
    helpers.compare_with_plain(got, where, plain, label=f"whole {name} {dtype} {variant}", **TOL[dtype])
    assert ex.cache.pages_in_use() == 0


@pytest.mark.parametrize("name,dtype,variant", CASES)
def test_tail_one_by_one(setups, name, dtype, variant):
    folder, requests, plain = setups(name, dtype, variant)
    steps, where = helpers.trace_tail_one_by_one(requests, tail=32)
    ex = _executor(folder, dtype, num_pages=20, page_tokens=16)
    got = helpers.replay_in_process(ex, steps)
    helpers.compare_with_plain(got, where, plain, label=f"tail {name} {dtype} {variant}", **TOL[dtype])


@pytest.mark.parametrize("name,dtype,variant", CASES)
def test_portions(setups, name, dtype, variant):
    folder, requests, plain = setups(name, dtype, variant)
    steps, where = helpers.trace_portions(requests, seed=3)
    ex = _executor(folder, dtype, num_pages=20, page_tokens=16)
    got = helpers.replay_in_process(ex, steps)
    helpers.compare_with_plain(got, where, plain, label=f"portions {name} {dtype} {variant}", **TOL[dtype])


@pytest.mark.parametrize("name,dtype,variant", CASES)
def test_mixed_few_pages(setups, name, dtype, variant):
    folder, requests, plain = setups(name, dtype, variant)
    page = 16
    steps, where, peak = helpers.trace_mixed(requests, seed=11, max_live=4, page_tokens=page)
    ex = _executor(folder, dtype, num_pages=peak // page, page_tokens=page)
    got = helpers.replay_in_process(ex, steps)
    helpers.compare_with_plain(got, where, plain, label=f"mixed {name} {dtype} {variant}", **TOL[dtype])
    assert ex.cache.pages_in_use() == 0
    pool = next(iter(ex.cache.groups.values())).pool
    assert pool.high_water_mark == pool.num_pages, "the pool was meant to be used up"


@pytest.mark.parametrize("dtype,variant", [("float32", "ones"), ("bfloat16", "spread")])
def test_trace_run_program(setups, tmp_path, dtype, variant):
    """The program itself (64-token pages, a pool just big enough), on the mixed trace."""
    folder, requests, plain = setups("B", dtype, variant)
    steps, where, peak = helpers.trace_mixed(requests, seed=5, max_live=4, page_tokens=64)
    got = helpers.replay_subprocess(folder, dtype, steps, str(tmp_path / "out"), peak, helpers.TINY_B["vocab_size"])
    helpers.compare_with_plain(got, where, plain, label=f"trace_run B {dtype}", **TOL[dtype])
