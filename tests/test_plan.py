"""Which kernel serves a linear map at which number of rows is the weight's own plan, computed from its shape
(host-side; no GPU): the plans of the shapes the benchmark knows, of other widths and machines, and that a part
asks its weight's plan and carries no threshold of its own."""
import dataclasses

from bare_cuda_4gib_amd.csrc import ops


def test_plans_of_the_known_shapes():
    gate_up = ops.compute_plan(2 * 5632, 2048)                 # wide: tiles enough for every CU from 24 rows on
    assert gate_up.stream_rows == 23 and gate_up.streams(23) and not gate_up.streams(24)
    assert gate_up.fused_norm_rows == 8 and gate_up.parts(32) == 1
    assert [m for m in range(1, 70) if gate_up.wants_prepared(m, swiglu=True)] == [5, 6, 7, 8] + list(range(24, 65))
    out = ops.compute_plan(2048, 2048)                         # narrow and small: streamed up to 64 rows, k cut from 65
    assert out.stream_rows == 64 and out.parts(64) == 1 and out.parts(65) > 1 and out.parts(256) > 1 and out.parts(257) == 1
    assert [m for m in range(1, 70) if out.wants_prepared(m, swiglu=True)] == [5, 6, 7, 8, 64]
    assert all(out.wants_prepared(m) for m in (1, 8, 9, 64, 300))              # a q|k|v product always takes one
    big = ops.compute_plan(4096, 4096)                         # 2^24 elements: k cut from 10 rows on
    assert big.parts(9) == 1 and big.parts(10) > 1 and big.parts(64) > 1
    down = ops.compute_plan(4096, 14336)
    assert down.parts(16) in (2, 4, 8) and 14336 % (64 * down.parts(16)) == 0
    assert ops.compute_plan(2560, 2048).qkv_stream_rows == 64 and ops.compute_plan(12288, 4096).qkv_stream_rows == 47
    # the rows a fused norm stages must fit LDS: eight rows up to k = 6,136, four beyond
    assert ops.compute_plan(2048, 6136).fused_norm_rows == 8 and ops.compute_plan(2048, 6144).fused_norm_rows == 4
    assert ops.compute_plan(2048, 11008).fused_norm_rows == 4 and ops.compute_plan(4096, 14336).fused_norm_rows == 0


def test_another_width_or_machine_gets_thresholds_of_its_own():
    assert ops.compute_plan(8192, 2048).stream_rows == 23 and ops.compute_plan(8128, 2048).stream_rows == 64
    assert ops.compute_plan(8192, 2048, cus=304).stream_rows == 64             # more CUs: a wider output to fill them
    assert ops.compute_plan(4096, 2048, cus=128).stream_rows == 23
    assert ops.compute_plan(11264, 2056).stream_rows == 64                     # k no multiple of 64: the small tiles do not take it
    odd = ops.compute_plan(1000, 2056)
    assert odd.parts(100) == 1 and not odd.tiled_finishes_norm(100)


def test_a_measured_plan_takes_the_computed_one_s_place():
    n, k = 3072, 1536
    computed = ops.plan_for(n, k)
    assert computed == ops.compute_plan(n, k) and ops.streams_weights(40, n, k)
    try:
        ops.set_plan(dataclasses.replace(computed, stream_rows=16))
        assert not ops.streams_weights(40, n, k) and ops.streams_weights(16, n, k)
        assert ops.plan_for(n, k).stream_rows == 16 and ops.plan_for(n + 64, k).stream_rows == 64
    finally:
        ops.set_plan(computed)


def test_parts_ask_their_weight_s_plan():
    """No row threshold stands in the parts: what they answer follows the plan of the weight they hold."""
    import torch
    from bare_cuda_4gib_amd.parts.attention import CausalAttention
    from bare_cuda_4gib_amd.parts.feedforward import SwiGLU

    class Weight:
        def __init__(self, plan):
            self.plan, self.shape = plan, (plan.n, plan.k)

    ffn = SwiGLU(64, 176)
    ffn.interleaved, ffn.w_gu = True, Weight(ops.compute_plan(352, 64))
    assert [m for m in range(1, 70) if ffn.wants_prepared_norm(m)] == [5, 6, 7, 8, 64]
    ffn.w_gu = Weight(dataclasses.replace(ops.compute_plan(352, 64), stream_rows=11, fused_norm_rows=6))
    assert [m for m in range(1, 70) if ffn.wants_prepared_norm(m)] == [5, 6] + list(range(12, 65))
    ffn.interleaved = False
    assert not any(ffn.wants_prepared_norm(m) for m in range(1, 70))
    attn = CausalAttention(64, 4, 2, 16)
    attn.act_dtype, attn.w_qkv = torch.bfloat16, Weight(ops.compute_plan(128, 64))
    assert attn.wants_prepared_norm(1) and attn.wants_prepared_norm(64)
    attn.act_dtype = torch.float32
    assert not attn.wants_prepared_norm(8)
