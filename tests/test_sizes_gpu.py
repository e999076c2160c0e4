"""Sizes at the edges of what the kernels take, each through the whole engine against the plain
implementation: a query group wider than one 16-row tile, the largest head sizes, a width and
head size that the matrix-core kernels refuse (so the plain kernels serve), feed-forward and
vocabulary sizes that are multiples of nothing, small and large pages."""
import os

import pytest

import helpers
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu

# The tolerances of the replay tests, which were set for logits of magnitude ~0.2: the wider
# configuration below draws its weights with half the spread so that its logits are of that size too.
TOL = {"float32": dict(rtol=1e-4, atol=2e-6), "bfloat16": dict(rtol=2e-2, atol=6e-3)}
STD = {"big_pages": 0.01}


def _cfg(**kw):
    base = dict(architectures=["LlamaForCausalLM"], model_type="llama", rope_theta=10000.0, rms_norm_eps=1e-5,
                max_position_embeddings=256, tie_word_embeddings=False, num_hidden_layers=2)
    base.update(kw)
    return base


SIZES = {
    # 32 query heads on one key/value head: two 16-row tiles per token; width != heads * head_dim
    "wide_group": (_cfg(vocab_size=200, hidden_size=128, num_attention_heads=32, num_key_value_heads=1, head_dim=16,
                        intermediate_size=64), 16),
    "head_128": (_cfg(vocab_size=130, hidden_size=64, num_attention_heads=2, num_key_value_heads=2, head_dim=128,
                      intermediate_size=40), 32),
    "head_256": (_cfg(vocab_size=99, hidden_size=48, num_attention_heads=1, num_key_value_heads=1, head_dim=256,
                      intermediate_size=24, num_hidden_layers=1), 16),
    # nothing here is a multiple of 8: the plain kernels serve every product and the attention
    "odd_everything": (_cfg(vocab_size=97, hidden_size=68, num_attention_heads=4, num_key_value_heads=2, head_dim=18,
                            intermediate_size=52, tie_word_embeddings=True), 16),
    "big_pages": (_cfg(vocab_size=512, hidden_size=512, num_attention_heads=8, num_key_value_heads=4, head_dim=64,
                       intermediate_size=200, num_hidden_layers=1), 128),
}
LENGTHS = [3, 41, 90, 130]


@pytest.fixture(scope="module")
def made(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("sizes")
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            from bare_cuda_4gib_amd.weights import write_random_model
            cfg, _ = SIZES[name]
            folder = os.path.join(str(tmp), f"{name}_{dtype}")
            write_random_model(cfg, 11, folder, dtype, std=STD.get(name, 0.02))
            requests = {f"r{i}": helpers.random_ids(n, cfg["vocab_size"], 300 + i) for i, n in enumerate(LENGTHS)}
            plain = PlainLlama(folder)
            cache[(name, dtype)] = (folder, requests, {rid: plain.logits(ids).numpy() for rid, ids in requests.items()})
        return cache[(name, dtype)]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(SIZES))
def test_sizes_through_the_engine(made, name, dtype):
    from bare_cuda_4gib_amd.engine import Executor, load_model
    folder, requests, plain = made(name, dtype)
    page = SIZES[name][1]
    model, _ = load_model(folder, dtype, "cuda:0")
    steps_m, where_m, peak = helpers.trace_mixed(requests, seed=6, page_tokens=page)
    for label, (steps, where), pages in (
            ("portions", helpers.trace_portions(requests, seed=5), 4 * -(-max(LENGTHS) // page)),
            ("mixed", (steps_m, where_m), peak // page)):
        ex = Executor(model, num_pages=pages, max_requests=6, max_tokens=-(-max(LENGTHS) // page) * page,
                      page_tokens=page, poison=True)
        ex.cache.shuffle_free_pages(3)
        got = helpers.replay_in_process(ex, steps)
        helpers.compare_with_plain(got, where, plain, label=f"{label} {name} {dtype}", **TOL[dtype])
        assert ex.cache.pages_in_use() == 0


def test_sixteen_decoded_rows_at_a_width_whose_fused_norm_does_not_fit(tmp_path):
    """Hidden size 4,096: sixteen rows of it do not fit the LDS buffer of the product with the norm
    fused (eight do), so a step of sixteen decoded tokens takes the norm and the product apart --
    and gives the plain implementation's logits, like a step of eight."""
    import torch
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    from bare_cuda_4gib_amd.weights import write_random_model
    cfg = _cfg(vocab_size=72, hidden_size=4096, num_attention_heads=2, num_key_value_heads=1, head_dim=64,
               intermediate_size=48, num_hidden_layers=1)
    folder = os.path.join(str(tmp_path), "wide")
    write_random_model(cfg, 5, folder, "bfloat16", std=0.01)
    x = torch.zeros(16, 4096, device="cuda")
    w = torch.zeros(256, 4096, dtype=torch.bfloat16, device="cuda")
    assert ops.gemm_qkv_rope_supported(x[:8], 8, True, w, 64, 64) and not ops.gemm_qkv_rope_supported(x, 16, True, w, 64, 64)
    assert ops.gemm_normed_supported(x[:8], 8, w[0], w) and not ops.gemm_normed_supported(x, 16, w[0], w)
    plain = PlainLlama(folder)
    model, _ = load_model(folder, "bfloat16", "cuda:0")
    for n in (8, 16):
        ex = Executor(model, num_pages=n, max_requests=n, max_tokens=64, page_tokens=64)
        prompts = [helpers.random_ids(3 + i % 5, 72, 500 + i) for i in range(n)]
        for i, ids in enumerate(prompts):
            ex.admit(i)
            ex.step([StepEntry(i, ids[:-1], [])])
        got = ex.step([StepEntry(i, ids[-1:], [0]) for i, ids in enumerate(prompts)]).float().cpu().numpy()
        for i, ids in enumerate(prompts):
            want = plain.logits(ids).numpy()[-1]
            assert abs(got[i] - want).max() <= 6e-3 + 2e-2 * abs(want).max(), f"{n} rows, request {i}"


def test_one_layer_at_the_widths_of_an_8b_model(tmp_path):
    """One layer with the widths of a large model -- hidden 4,096, 32 query / 8 key-value heads of
    128, a feed-forward of 11,000 (no multiple of 16 x 16) -- so that every kernel meets its long
    k and its many blocks: prompts of 64 requests in batches of sixteen, then all 64 decoded together,
    then groups of 1, 8, 16, 17 and 22."""
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    from bare_cuda_4gib_amd.weights import write_random_model
    cfg = _cfg(vocab_size=1000, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=11000, num_hidden_layers=1)
    folder = os.path.join(str(tmp_path), "wide8b")
    write_random_model(cfg, 9, folder, "bfloat16", std=0.008)
    plain = PlainLlama(folder)
    model, _ = load_model(folder, "bfloat16", "cuda:0")
    n = 64
    prompts = [helpers.random_ids(4 + (7 * i) % 37, 1000, 700 + i) for i in range(n)]
    want = [plain.logits(ids).numpy() for ids in prompts]
    ex = Executor(model, num_pages=n, max_requests=n, max_tokens=64, page_tokens=64, max_batch_tokens=1024)
    for lo in range(0, n, 16):                        # prompts but for their last two tokens, sixteen requests a step
        for i in range(lo, lo + 16):
            ex.admit(i)
        ex.step([StepEntry(i, prompts[i][:-2], []) for i in range(lo, lo + 16)])

    def check(got, ids, at):
        got = got.float().cpu().numpy()
        for row, i in enumerate(ids):
            w = want[i][at]
            assert abs(got[row] - w).max() <= 6e-3 + 2e-2 * abs(w).max(), f"request {i}, token {at}, {len(ids)} rows"

    everyone = list(range(n))
    check(ex.step([StepEntry(i, prompts[i][-2:-1], [0]) for i in everyone]), everyone, -2)
    for lo, hi in ((0, 1), (1, 9), (9, 25), (25, 42), (42, 64)):
        ids = list(range(lo, hi))
        check(ex.step([StepEntry(i, prompts[i][-1:], [0]) for i in ids]), ids, -1)
