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


# --- each branch of a layer against library routines ---------------------------------------------
# One layer of configuration B (three heads, not grouped) with norm scales drawn around 1.0, a
# different draw for each norm, and peaked attention.  With one branch's output projection zeroed
# the layer is the other branch alone, which is written here with library routines only.  Each
# check is shown to bite: the same comparison on a model whose weights are swapped the way a
# plausible mistake would swap them (the two norms' scales, gate and up, no scale at all) fails.

@pytest.fixture(scope="module")
def one_layer(tmp_path_factory):
    from bare_cuda_4gib_amd.weights import write_random_model
    cfg = dict(helpers.TINY_B, num_hidden_layers=1)
    folder = write_random_model(cfg, 7, str(tmp_path_factory.mktemp("one") / "m"), "float32", **helpers.variant_args("B", "spread"))
    return P.PlainLlama(folder)


def _with(m, **replaced):
    import copy
    out = copy.copy(m)
    out.w = dict(m.w)
    for name, t in replaced.items():
        out.w["model.layers.0." + name.replace("__", ".")] = t
    return out


def _library_attention_branch(m, x):
    """x + o_proj(SDPA(rope(q), rope(k), v)) on F.rms_norm(x, input_layernorm): heads not grouped."""
    w, t = m.w, x.shape[0]
    h = F.rms_norm(x, (m.hidden,), w["model.layers.0.input_layernorm.weight"], m.eps)
    q, k, v = (F.linear(h, w[f"model.layers.0.self_attn.{n}_proj.weight"]).view(t, m.heads, m.head_dim) for n in "qkv")
    pos = torch.arange(t)
    q, k = P.rope(q, pos, m.theta), P.rope(k, pos, m.theta)
    o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    return x + F.linear(o.transpose(0, 1).reshape(t, -1), w["model.layers.0.self_attn.o_proj.weight"])


def _library_ffn_branch(m, x):
    """x + down(F.silu(gate(h)) * up(h)) on h = F.rms_norm(x, post_attention_layernorm)."""
    w = m.w
    h = F.rms_norm(x, (m.hidden,), w["model.layers.0.post_attention_layernorm.weight"], m.eps)
    a = F.silu(F.linear(h, w["model.layers.0.mlp.gate_proj.weight"])) * F.linear(h, w["model.layers.0.mlp.up_proj.weight"])
    return x + F.linear(a, w["model.layers.0.mlp.down_proj.weight"])


def test_attention_branch_reads_its_own_norm(one_layer):
    m = one_layer
    assert m.heads == m.kv_heads and m.layers == 1
    ids = helpers.random_ids(23, m.vocab, 4)
    x = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    w1, w2 = m.w["model.layers.0.input_layernorm.weight"], m.w["model.layers.0.post_attention_layernorm.weight"]
    assert not torch.allclose(w1, w2) and float((w1 - 1).abs().max()) > 0.05
    alone = _with(m, mlp__down_proj__weight=torch.zeros_like(m.w["model.layers.0.mlp.down_proj.weight"]))
    want = _library_attention_branch(alone, x)
    assert torch.allclose(alone.hidden_states(ids), want, atol=1e-12)
    assert float((want - x).abs().max()) > 1e-3                       # the branch is really there
    # mistakes that must not pass: the other norm's scale, no scale, no norm at all
    swapped = _with(alone, input_layernorm__weight=w2, post_attention_layernorm__weight=w1)
    assert not torch.allclose(swapped.hidden_states(ids), want, atol=1e-6)
    unscaled = _with(alone, input_layernorm__weight=torch.ones_like(w1))
    assert not torch.allclose(unscaled.hidden_states(ids), want, atol=1e-6)
    qkv_of_x = [F.linear(x, m.w[f"model.layers.0.self_attn.{n}_proj.weight"]) for n in "qkv"]
    assert not torch.allclose(qkv_of_x[0], F.linear(F.rms_norm(x, (m.hidden,), w1, m.eps), m.w["model.layers.0.self_attn.q_proj.weight"]), atol=1e-3)


def test_feed_forward_branch_reads_its_own_norm_and_gates_with_gate(one_layer):
    m = one_layer
    ids = helpers.random_ids(17, m.vocab, 5)
    x = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    w1, w2 = m.w["model.layers.0.input_layernorm.weight"], m.w["model.layers.0.post_attention_layernorm.weight"]
    alone = _with(m, self_attn__o_proj__weight=torch.zeros_like(m.w["model.layers.0.self_attn.o_proj.weight"]))
    want = _library_ffn_branch(alone, x)
    assert torch.allclose(alone.hidden_states(ids), want, atol=1e-12)
    assert float((want - x).abs().max()) > 1e-3
    # mistakes that must not pass: silu on the up projection, the attention's norm, no scale
    g, u = m.w["model.layers.0.mlp.gate_proj.weight"], m.w["model.layers.0.mlp.up_proj.weight"]
    gate_up_swapped = _with(alone, mlp__gate_proj__weight=u, mlp__up_proj__weight=g)
    assert not torch.allclose(gate_up_swapped.hidden_states(ids), want, atol=1e-6)
    norms_swapped = _with(alone, input_layernorm__weight=w2, post_attention_layernorm__weight=w1)
    assert not torch.allclose(norms_swapped.hidden_states(ids), want, atol=1e-6)
    unscaled = _with(alone, post_attention_layernorm__weight=torch.ones_like(w2))
    assert not torch.allclose(unscaled.hidden_states(ids), want, atol=1e-6)


def test_both_branches_chain_through_the_residual_stream(one_layer):
    """The whole layer is the feed-forward branch applied to the attention branch's result (not to x)."""
    m = one_layer
    ids = helpers.random_ids(11, m.vocab, 6)
    x = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    want = _library_ffn_branch(m, _library_attention_branch(m, x))
    assert torch.allclose(m.hidden_states(ids), want, atol=1e-12)
    parallel = _library_attention_branch(m, x) + _library_ffn_branch(m, x) - x
    assert not torch.allclose(m.hidden_states(ids), parallel, atol=1e-6)


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
