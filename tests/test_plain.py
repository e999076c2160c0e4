"""Pins the plain implementation by what fixes it beside the reference's text: special cases
that reduce to a library routine, invariants, and the constants the reference's own tests hold.
Each check is chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import helpers
import plain_llama as P

D = torch.float64


def test_rmsnorm_unit_weight_and_eps_on_the_mean():
    x = torch.tensor([[3.0, 4.0]], dtype=D)                      # mean square 12.5, sum 25
    y = P.rmsnorm(x, torch.ones(2, dtype=D), eps=1.0)
    assert torch.allclose(y, x / math.sqrt(12.5 + 1.0))          # eps on the sum would give sqrt(25/2 + 1/2)
    assert not torch.allclose(y, x / math.sqrt((25.0 + 1.0) / 2))
    w = torch.tensor([2.0, -1.0], dtype=D)
    assert torch.allclose(P.rmsnorm(x, w, 0.0), x / math.sqrt(12.5) * w)


def test_rmsnorm_matches_library_norm():
    torch.manual_seed(0)
    x, w = torch.randn(5, 300, dtype=D), torch.randn(300, dtype=D)   # reference's shape: test_rmsnorm.cu (5 x 300)
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), F.rms_norm(x, (300,), w, 1e-5))


def test_rope_position_zero_is_identity_and_norms_are_kept():
    torch.manual_seed(1)
    x = torch.randn(7, 4, 16, dtype=D)
    pos = torch.tensor([0, 1, 2, 5, 8, 13, 21])                  # reference_forward.py:163
    y = P.rope(x, pos, 10000.0)
    assert torch.equal(y[0], x[0])
    half = 8
    assert torch.allclose(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)


def test_rope_sign_and_pairing():
    # d = 4: pairs (0, 2) and (1, 3); inv_freq = [1, theta^-0.5].  A wrong sign turns the first
    # assertion's sin negative; interleaved pairing (0,1),(2,3) moves the ones elsewhere.
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]], [[0.0, 1.0, 0.0, 0.0]]], dtype=D)
    y = P.rope(x, torch.tensor([3, 3]), theta=100.0)
    assert torch.allclose(y[0, 0], torch.tensor([math.cos(3.0), 0.0, math.sin(3.0), 0.0], dtype=D))
    assert torch.allclose(y[1, 0], torch.tensor([0.0, math.cos(0.3), 0.0, math.sin(0.3)], dtype=D))


def test_rope_scores_depend_on_distance_only():
    torch.manual_seed(2)
    q, k = torch.randn(1, 1, 32, dtype=D), torch.randn(1, 1, 32, dtype=D)
    def dot(m, n):
        return float((P.rope(q, torch.tensor([m]), 500000.0) * P.rope(k, torch.tensor([n]), 500000.0)).sum())
    assert abs(dot(5, 2) - dot(105, 102)) < 1e-9
    assert abs(dot(5, 2) - dot(2, 5)) > 1e-6                     # the sign of the distance counts


def test_attention_without_groups_is_library_attention():
    torch.manual_seed(3)
    t, h, d = 9, 3, 8
    q, k, v = (torch.randn(t, h, d, dtype=D) for _ in range(3))
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(P.attention(q, k, v), ref.transpose(0, 1), atol=1e-12)


def test_attention_masks_and_special_cases():
    torch.manual_seed(4)
    t, h, kvh, d = 7, 4, 2, 8                                    # test_attention.cu: 7 tokens, 4/2 heads, d = 8
    q, k, v = torch.randn(t, h, d, dtype=D), torch.randn(t, kvh, d, dtype=D), torch.randn(t, kvh, d, dtype=D)
    s = P.attention_scores(q, k)
    assert torch.isinf(s[:, 2, 3:]).all() and torch.isfinite(s[:, 2, :3]).all()
    p = P.softmax_rows(s)
    assert torch.equal(p[:, 2, 3:], torch.zeros(h, t - 3, dtype=D))          # exactly zero where masked
    assert torch.allclose(p.sum(-1), torch.ones(h, t, dtype=D))
    out = P.attention(q, k, v)
    assert torch.allclose(out[0], v[0].repeat_interleave(2, dim=0))          # one key: that value row
    # grouped heads == ungrouped heads with keys and values repeated (consecutive query heads share)
    out_rep = P.attention(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1))
    assert torch.allclose(out, out_rep)
    # identical keys: uniform probabilities, so the output is the running mean of the values
    same = P.attention(q, k[:1].expand(t, kvh, d), v)
    assert torch.allclose(same[4, 0], v[:5, 0].mean(0))
    # scale is 1/sqrt(d), applied to the dot product
    assert torch.allclose(s[1, 5, 2], (q[5, 1] @ k[2, 0]) / math.sqrt(d))


def test_attention_window():
    torch.manual_seed(5)
    q, k = torch.randn(6, 1, 4, dtype=D), torch.randn(6, 1, 4, dtype=D)
    s = P.attention_scores(q, k, window=3)
    vis = torch.isfinite(s[0])
    assert vis[5].tolist() == [False, False, False, True, True, True]
    assert vis[1].tolist() == [True, True, False, False, False, False]


def test_swiglu_and_argmax():
    g, u = torch.tensor([0.0, 1.5, -2.0], dtype=D), torch.tensor([7.0, 2.0, 3.0], dtype=D)
    assert torch.allclose(P.swiglu(g, u), F.silu(g) * u)
    assert float(P.swiglu(g, u)[0]) == 0.0
    row = torch.tensor([1.0, 5.0, 2.0, 5.0, 5.0])
    assert P.argmax_lowest(row) == 1                              # test_elementwise.cu:56-64: lowest index wins


@pytest.fixture(scope="module")
def plain_a(tmp_path_factory):
    return P.PlainLlama(helpers.make_model_dir(tmp_path_factory.mktemp("m"), "A", "float32"))


def test_model_is_causal_and_shift_invariant(plain_a):
    ids = helpers.random_ids(20, 256, 1)
    base = plain_a.logits(ids)
    changed = list(ids)
    changed[12] = (changed[12] + 1) % 256
    other = plain_a.logits(changed)
    assert torch.equal(base[:12], other[:12]) and not torch.allclose(base[12:], other[12:])
    shifted = plain_a.logits(ids, position_offset=37)             # only distances between positions count
    assert torch.allclose(base, shifted, atol=1e-9)


def test_model_reduces_to_embedding_norm_head_without_layers_output(plain_a):
    """With the output projections zeroed the residual stream is the embedding: logits must be
    rmsnorm(E[ids]) W^T.  A norm in the wrong place, or a missing residual, fails this."""
    import copy
    m = copy.copy(plain_a)
    m.w = dict(plain_a.w)
    for i in range(m.layers):
        m.w[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(m.w[f"model.layers.{i}.self_attn.o_proj.weight"])
        m.w[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(m.w[f"model.layers.{i}.mlp.down_proj.weight"])
    ids = helpers.random_ids(6, 256, 2)
    x = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    want = F.rms_norm(x, (64,), m.w["model.norm.weight"], m.eps) @ m.w["lm_head.weight"].T
    assert torch.allclose(m.logits(ids), want, atol=1e-12)


def test_greedy_recomputes_whole_sequence(plain_a):
    ids = helpers.random_ids(5, 256, 3)
    out = plain_a.greedy(ids, 3)
    assert out[0] == P.argmax_lowest(plain_a.logits(ids)[-1])
    assert out[1] == P.argmax_lowest(plain_a.logits(ids + out[:1])[-1])


def test_sampling_distribution_vectors():
    # engine/tests/test_sampler.cu:49-61
    logits = [math.log(0.5), math.log(0.3), math.log(0.2), -1e30]
    def close(a, b):
        return all(abs(x - y) < 1e-9 for x, y in zip(a, b))
    assert close(P.sample_probabilities(logits, 1.0), [0.5, 0.3, 0.2, 0.0])
    assert close(P.sample_probabilities(logits, 0.5), [0.25 / 0.38, 0.09 / 0.38, 0.04 / 0.38, 0.0])
    assert close(P.sample_probabilities(logits, 1.0, top_k=2), [0.625, 0.375, 0.0, 0.0])
    assert close(P.sample_probabilities(logits, 1.0, top_p=0.7), [0.625, 0.375, 0.0, 0.0])
    assert close(P.sample_probabilities(logits, 1.0, top_k=2, top_p=0.6), [1.0, 0.0, 0.0, 0.0])
    assert close(P.sample_probabilities(logits, 0.0), [1.0, 0.0, 0.0, 0.0])
    assert close(P.sample_probabilities(logits, 2.0, top_k=1), [1.0, 0.0, 0.0, 0.0])
