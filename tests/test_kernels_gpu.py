"""Each kernel alone against a plain float64 reference, at other sizes than the engine's: ragged
widths (300, 130, 17, 61, 48 -- the reference's own test shapes), head sizes 16..256, groups of
1, 2, 3, 8 and 32 query heads, pages that are shuffled and poisoned with NaN where nobody owns
them."""
import math
import random

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from bare_cuda_4gib_amd.csrc import ops
    return ops


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64) * scale


def close(got, want, rtol, atol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert bool((err <= bound).all()), f"{what}: max error {float(err.max()):.3g} at {int(err.argmax())}, bound {float(bound.flatten()[int(err.argmax())]):.3g}"


def bf(x):
    return x.to(torch.bfloat16)


def test_embed_gather_is_exact(ops):
    table = rnd(61, 48, seed=1)
    ids = torch.tensor([0, 60, 5, 5, 17, 33, 2, 59, 1], dtype=torch.int32)
    for t in (table.float(), bf(table)):
        out = ops.embed_gather(t.to(DEV), ids.to(DEV))
        assert out.dtype == torch.float32 and torch.equal(out.cpu(), t.float()[ids.long()])


@pytest.mark.parametrize("wdt,odt", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                     (torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_rmsnorm(ops, wdt, odt):
    x, w = rnd(5, 300, seed=2), 1.0 + 0.1 * rnd(300, seed=3)
    w = w.to(wdt)
    want = P.rmsnorm(x.float().double(), w.double(), 1e-5)
    tol = dict(rtol=1e-5, atol=1e-5) if odt == torch.float32 else dict(rtol=8e-3, atol=1e-3)
    close(ops.rmsnorm(x.float().to(DEV), w.to(DEV), 1e-5, odt), want, what="rmsnorm", **tol)
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=DEV)
    close(ops.rmsnorm(x.float().to(DEV), w.to(DEV), 1e-5, odt, rows=rows), want[[4, 0, 4]], what="rmsnorm rows", **tol)
    short = torch.tensor([[3.0, 4.0]])                       # eps on the mean, not on the sum
    got = ops.rmsnorm(short.to(DEV), torch.ones(2, device=DEV), 1.0, torch.float32)
    close(got, short.double() / math.sqrt(13.5), 1e-6, 1e-6, "rmsnorm eps")


@pytest.mark.parametrize("m,n,k", [(65, 2048, 2048), (33, 4096, 5632), (128, 4096, 4096), (100, 1000, 1024), (64, 8192, 2048),
                                   (250, 2048, 5632), (10, 4096, 4096)])
def test_adding_product_in_parts_of_k_with_the_norm_after_it(ops, m, n, k):
    """A few dozen rows: the product's k cut over workgroups, the parts added to the residual in order by the kernel
    that norms it -- against the definition, and the residual against the product that adds at once."""
    assert ops.parts_of_k(m, n, k) > 1 and ops.parts_of_k(9, n, k) == 1 and ops.parts_of_k(257, n, k) == 1
    a, w = bf(rnd(m, k, seed=80)), bf(rnd(n, k, seed=81, scale=0.3))
    base, g = rnd(m, n, seed=82).float(), (1.0 + 0.1 * rnd(n, seed=83)).bfloat16()
    resid = base.clone().to(DEV)
    assert ops.gemm_parts_supported(a.to(DEV), w.to(DEV), resid, g.to(DEV))
    done = ops.gemm_parts_accumulate_norm(a.to(DEV), w.to(DEV), resid, g.to(DEV), 1e-5)
    want = base.double() + a.double() @ w.double().T
    close(resid, want, 1e-4, 1e-4 * math.sqrt(k), "residual")
    at_once = base.clone().to(DEV)
    ops.gemm_fast(a.to(DEV), w.to(DEV), accumulate_into=at_once)
    close(resid, at_once.double().cpu(), 1e-5, 1e-5 * math.sqrt(k), "residual, against the product that adds at once")
    # the norm is of the residual as the kernel holds it: the same bits as the norm kernel's of what it wrote back
    assert torch.equal(done.tensor, ops.rmsnorm(resid, g.to(DEV), 1e-5, torch.bfloat16))
    close(done.tensor, P.rmsnorm(want, g.double(), 1e-5), 8e-3, 2e-3, "norm")
    assert not ops.gemm_parts_supported(a.float().to(DEV), w.to(DEV), resid, g.to(DEV))


@pytest.mark.parametrize("m,n,k", [(17, 130, 300), (1, 130, 300), (150, 61, 48), (64, 64, 64), (3, 5, 7)])
def test_gemm_generic(ops, m, n, k):
    a, w = rnd(m, k, seed=4), rnd(n, k, seed=5)
    want = a.float().double() @ w.float().double().T
    close(ops.gemm_generic(a.float().to(DEV), w.float().to(DEV)), want, 1e-5, 1e-4, "f32")
    base = rnd(m, n, seed=6).float()
    acc = base.clone().to(DEV)
    ops.gemm_generic(a.float().to(DEV), w.float().to(DEV), accumulate_into=acc)
    close(acc, want + base.double(), 1e-5, 1e-4, "f32 accumulate")
    ab, wb = bf(a), bf(w)
    wantb = ab.double() @ wb.double().T
    close(ops.gemm_generic(ab.to(DEV), wb.to(DEV), torch.float32), wantb, 1e-5, 1e-4, "bf16 -> f32")
    close(ops.gemm_generic(ab.to(DEV), wb.to(DEV), torch.bfloat16), wantb, 8e-3, 1e-2, "bf16 -> bf16")
    close(ops.gemm_generic(ab.to(DEV), w.float().to(DEV), torch.float32), ab.double() @ w.float().double().T, 1e-5, 1e-4,
          "bf16 x f32")


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("n,k", [(130, 304), (16, 8), (2560, 2048), (301, 80)])
def test_gemm_skinny(ops, m, n, k):
    a, w = bf(rnd(m, k, seed=7)), bf(rnd(n, k, seed=8))
    want = a.double() @ w.double().T
    scale = math.sqrt(k)
    got = ops.gemm_fast(a.to(DEV), w.to(DEV), torch.float32)
    close(got, want, 1e-4, 1e-4 * scale, "skinny -> f32")
    close(ops.gemm_fast(a.to(DEV), w.to(DEV), torch.bfloat16), want, 8e-3, 1e-3 * scale, "skinny -> bf16")
    base = rnd(m, n, seed=9).float()
    acc = base.clone().to(DEV)
    assert ops.gemm_fast(a.to(DEV), w.to(DEV), accumulate_into=acc) is acc
    close(acc, want + base.double(), 1e-4, 1e-4 * scale, "skinny accumulate")
    # a row's result must not depend on the other rows of the call
    alone = ops.gemm_fast(a[:1].contiguous().to(DEV), w.to(DEV), torch.float32)
    assert torch.equal(alone[0], got[0])


def interleave8(gate, up):
    """Blocks of 16 rows: eight gate rows, then the eight up rows of the same outputs."""
    i = gate.shape[0]
    return torch.stack([gate.view(i // 8, 8, -1), up.view(i // 8, 8, -1)], dim=1).reshape(2 * i, -1).contiguous()


@pytest.mark.parametrize("m", [1, 7, 64, 100, 300])
@pytest.mark.parametrize("inter,k", [(176, 64), (112, 80), (5632, 256)])
def test_gemm_swiglu(ops, m, inter, k):
    a, w = bf(rnd(m, k, seed=10)), bf(rnd(2 * inter, k, seed=11, scale=0.3))
    gu = a.double() @ w.double().T
    want = P.swiglu(gu[:, :inter], gu[:, inter:])
    # the product is stored in bfloat16 before the activation: two roundings of 2^-9 on g and u
    close(ops.gemm_swiglu(a.to(DEV), w.to(DEV)), want, 2e-2, 3e-2, "gate rows then up rows")
    wi = interleave8(w[:inter], w[inter:])
    close(ops.gemm_swiglu(a.to(DEV), wi.to(DEV), interleaved=True), want, 8e-3, 3e-2,
          "interleaved: the activation sees the float sums")


@pytest.mark.parametrize("m,n,k", [(65, 130, 304), (70, 130, 304), (150, 257, 64), (300, 128, 2048), (128, 384, 96), (129, 61, 8),
                                   (200, 384, 96)])
def test_gemm_mfma(ops, m, n, k):
    a, w = bf(rnd(m, k, seed=12)), bf(rnd(n, k, seed=13))
    want = a.double() @ w.double().T
    scale = math.sqrt(k)
    got = ops.gemm_fast(a.to(DEV), w.to(DEV), torch.float32)
    close(got, want, 1e-4, 1e-4 * scale, "mfma -> f32")
    close(ops.gemm_fast(a.to(DEV), w.to(DEV), torch.bfloat16), want, 8e-3, 1e-3 * scale, "mfma -> bf16")
    base = rnd(m, n, seed=14).float()
    acc = base.clone().to(DEV)
    ops.gemm_fast(a.to(DEV), w.to(DEV), accumulate_into=acc)
    close(acc, want + base.double(), 1e-4, 1e-4 * scale, "mfma accumulate")
    # rows do not depend on M (while the same kind of kernel serves them: up to the plan's stream_rows the
    # weights are streamed, beyond that the output is tiled)
    part = max(m - 3, ops.SKINNY_MAX_ROWS + 1) if m > ops.SKINNY_MAX_ROWS else min(m, 40)
    fewer = ops.gemm_fast(a[:part].contiguous().to(DEV), w.to(DEV), torch.float32)
    assert torch.equal(fewer, got[:part])
    assert ops.gemm_fast(a.float().to(DEV), w.to(DEV)) is None                      # float operands: not taken


@pytest.mark.parametrize("m,n,k,tile", [(4096 - 236, 4096 - 244, 192, (256, 256)), (2048 - 20, 6144 - 12, 192, (256, 192)),
                                        (4096 - 20, 6144 - 12, 64, (256, 192)), (4096 - 20, 6144 - 12, 128, (256, 192)),
                                        (2048 - 20, 4096 - 12, 192, (256, 128)), (2048 - 20, 2048 - 12, 1024, (128, 128))])
def test_gemm_mfma_every_tile_agrees_bit_for_bit(ops, m, n, k, tile):
    """Five tiles for the operands that go straight into LDS, chosen by the output's shape.  All add over k in
    the same order: a row's result is the same bits whichever tile the number of rows selects (the first 300 rows
    alone take the smallest), with edges in both directions, for every epilogue.  The 256 x 192 tile's waves take
    turns half a step apart: one and two steps of k are its shortest walks."""
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the shapes are chosen for 256 CUs")
    assert ops.tiled_tile(m, n, k) == tile and ops.tiled_tile(300, n, k) == (64, 64)
    a, w = bf(rnd(m, k, seed=40)), bf(rnd(n, k, seed=41))
    ad, wd = a.to(DEV), w.to(DEV)
    full = ops.gemm_fast(ad, wd, torch.float32)
    close(full, a.double() @ w.double().T, 1e-4, 2e-3, f"tile {tile}")
    few = ops.gemm_fast(ad[:300].contiguous(), wd, torch.float32)
    assert torch.equal(few, full[:300])
    assert torch.equal(ops.gemm_fast(ad[:300].contiguous(), wd, torch.bfloat16), ops.gemm_fast(ad, wd, torch.bfloat16)[:300])
    acc_full, acc_few = torch.ones(m, n, device=DEV), torch.ones(300, n, device=DEV)
    ops.gemm_fast(ad, wd, accumulate_into=acc_full)
    ops.gemm_fast(ad[:300].contiguous(), wd, accumulate_into=acc_few)
    assert torch.equal(acc_few, acc_full[:300])
    close(acc_full, a.double() @ w.double().T + 1.0, 1e-4, 2e-3, f"tile {tile}, added")
    half = (n // 32) * 16                                           # gate and up rows in blocks of eight
    gate_up = interleave8(w[:half], w[half:2 * half]).to(DEV)
    assert ops.tiled_tile(m, 2 * half, k) == tile
    g = ops.gemm_swiglu(ad, gate_up, interleaved=True)
    assert torch.equal(ops.gemm_swiglu(ad[:300].contiguous(), gate_up, interleaved=True), g[:300])
    gu = a.double() @ w[:2 * half].double().T
    close(g, P.swiglu(gu[:, :half], gu[:, half:]), 8e-3, 3e-2, f"tile {tile}, SwiGLU")


def test_gemm_mfma_both_forms_agree_bit_for_bit(ops):
    """A k that is no multiple of 64 goes through registers, in 128 x 128 tiles; the same operands padded with
    zeros to whole steps go straight into LDS.  Zeros add nothing, and both add over k in the same order: the
    same bits, for every epilogue."""
    m, n, k = 700, 2060, 200
    a, w = bf(rnd(m, k, seed=42)), bf(rnd(n, k, seed=43))
    pad = lambda t: torch.cat([t, torch.zeros(t.shape[0], 256 - k, dtype=t.dtype)], dim=1).contiguous()
    ad, wd, ap, wp = a.to(DEV), w.to(DEV), pad(a).to(DEV), pad(w).to(DEV)
    staged = ops.gemm_fast(ad, wd, torch.float32)
    close(staged, a.double() @ w.double().T, 1e-4, 2e-3, "through registers")
    assert torch.equal(staged, ops.gemm_fast(ap, wp, torch.float32))
    assert torch.equal(ops.gemm_fast(ad, wd, torch.bfloat16), ops.gemm_fast(ap, wp, torch.bfloat16))
    acc_staged, acc_direct = torch.ones(m, n, device=DEV), torch.ones(m, n, device=DEV)
    ops.gemm_fast(ad, wd, accumulate_into=acc_staged)
    ops.gemm_fast(ap, wp, accumulate_into=acc_direct)
    assert torch.equal(acc_staged, acc_direct)
    gate_up = interleave8(w[:1024], w[1024:2048])
    assert torch.equal(ops.gemm_swiglu(ad, gate_up.to(DEV), interleaved=True),
                       ops.gemm_swiglu(ap, pad(gate_up).to(DEV), interleaved=True))
    # the form through registers with many tiles (20 x 17) and an operand that does not start on 16 bytes
    big = bf(rnd(2500, k, seed=44))
    close(ops.gemm_fast(big.to(DEV), wd, torch.float32), big.double() @ w.double().T, 1e-4, 2e-3, "many tiles")
    shifted = torch.zeros(m * 256 + 4, dtype=torch.bfloat16, device=DEV)[4:].view(m, 256)     # 8 bytes off
    shifted.copy_(ap)
    assert torch.equal(ops.gemm_fast(shifted, wp, torch.float32), staged)


@pytest.mark.parametrize("m,n", [(1024, 1024), (2304, 640), (1280 + 5, 384), (4352, 256)])
def test_gemm_mfma_tile_numbering_covers_every_tile(ops, m, n):
    """Tiles are dealt to the XCDs and walked in bands of eight rows of tiles: every tile is computed
    once, whether the rows of tiles are a multiple of the band or not and whether the tile count is a multiple of
    the XCDs or not; with operands straight into LDS (k = 64) and through registers (k = 72)."""
    for k in (64, 72):
        a, w = bf(rnd(m, k, seed=15)), bf(rnd(n, k, seed=16))
        close(ops.gemm_fast(a.to(DEV), w.to(DEV), torch.float32), a.double() @ w.double().T, 1e-4, 1e-3, f"numbering, k={k}")


def test_gemm_mfma_xcd_numbering_covers_every_tile(ops):
    a, w = bf(rnd(1024, 64, seed=15)), bf(rnd(1024, 64, seed=16))                    # 8 x 8 tiles: remapped ids
    close(ops.gemm_fast(a.to(DEV), w.to(DEV), torch.float32), a.double() @ w.double().T, 1e-4, 1e-3, "xcd")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_swiglu(ops, dt):
    gu = rnd(9, 2 * 176, seed=17).to(dt)
    want = P.swiglu(gu.double()[:, :176], gu.double()[:, 176:])
    close(ops.swiglu(gu.to(DEV)), want, 1e-5 if dt == torch.float32 else 8e-3, 1e-6 if dt == torch.float32 else 1e-3)


def block_pair_order(d):
    """Dimensions of a head in blocks of 16: eight dimensions, then their rotation partners."""
    return [8 * b + t + (d // 2 if half else 0) for b in range(d // 16) for half in (0, 1) for t in range(8)]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,rotate", [(16, True), (48, True), (64, True), (32, False)])
def test_rope_kv_write_blocks_with_table(ops, dt, d, rotate):
    """The block-order kernel with a table of angles: rows in block order in, rotated pairs out,
    compared in the natural order with the plain rotation."""
    nh, nkv, page, pages = 3, 2, 16, 5
    positions = [0, 1, 2, 5, 8, 13, 21, 34, 3]
    t = len(positions)
    natural = rnd(t, nh + 2 * nkv, d, seed=60)
    order = block_pair_order(d)
    qkv = natural[:, :, order].reshape(t, -1).to(dt)
    slots = [3 * page + i for i in range(4)] + [0, page + 15, 4 * page + 7, 2 * page + 1, 2 * page + 2]
    kc = torch.full((pages, nkv, page, d), -7.5, dtype=dt, device=DEV)
    vc = torch.full((pages, nkv, d, page), -7.5, dtype=dt, device=DEV)
    pos_dev = torch.tensor(positions, dtype=torch.int32, device=DEV)
    table = ops.rope_table(pos_dev, d, 10000.0) if rotate else None
    if rotate:                                                           # the table itself: cos and sin of the angles
        ang = torch.tensor(positions, dtype=torch.float64)[:, None] / 10000.0 ** (torch.arange(d // 2, dtype=torch.float64) * 2 / d)
        close(table[..., 0], torch.cos(ang), 0, 5e-6, "cos")             # (float angles: 34 * 2^-24 off at most)
        close(table[..., 1], torch.sin(ang), 0, 5e-6, "sin")
    buf = qkv.clone().to(DEV)
    ops.rope_kv_write_blocks(buf, table, torch.tensor(slots, dtype=torch.int32, device=DEV), kc, vc, nh, nkv, d)
    x = qkv.double().view(t, nh + 2 * nkv, d)                            # (rounded as the kernel's input is)
    inverse = torch.argsort(torch.tensor(order))
    x_nat = x[:, :, inverse]
    pos = torch.tensor(positions)
    q_want = P.rope(x_nat[:, :nh], pos, 10000.0, d) if rotate else x_nat[:, :nh]
    k_want = P.rope(x_nat[:, nh:nh + nkv], pos, 10000.0, d) if rotate else x_nat[:, nh:nh + nkv]
    tol = dict(rtol=1e-5, atol=1e-5) if dt == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    out = buf.cpu().double().view(t, nh + 2 * nkv, d)
    close(out[:, :nh][:, :, inverse], q_want, what="q", **tol)
    kc_c, vc_c = (c.cpu().double() for c in ops.cache_to_plain(kc, vc))   # by token and dimension
    touched = torch.zeros(pages, page, dtype=torch.bool)
    for i, sl in enumerate(slots):
        pg, off = divmod(sl, page)
        close(kc_c[pg, :, off, :][:, inverse], k_want[i], what=f"k row {i}", **tol)
        close(vc_c[pg, :, :, off][:, inverse], x_nat[i, nh + nkv:], what=f"v row {i}", **tol)
        touched[pg, off] = True
    assert bool((kc_c.permute(0, 2, 1, 3)[~touched] == -7.5).all()) and bool((vc_c.permute(0, 3, 1, 2)[~touched] == -7.5).all())


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rotary_dim", [16, 8, 0])
def test_rope_kv_write(ops, dt, rotary_dim):
    nh, nkv, d, page, pages = 4, 2, 16, 4, 9
    positions = [0, 1, 2, 5, 8, 13, 21]                                 # reference_forward.py:163
    t = len(positions)
    qkv = rnd(t, (nh + 2 * nkv) * d, seed=18).to(dt)
    slots = [5 * page + 1, 5 * page + 2, 2 * page + 0, 0, 8 * page + 3, 7 * page + 2, 3 * page + 1]
    sentinel = -7.5                                                       # test_kv_cache_write.cu:25-41
    kc = torch.full((pages, nkv, page, d), sentinel, dtype=dt, device=DEV)
    vc = torch.full((pages, nkv, d, page), sentinel, dtype=dt, device=DEV)
    buf = qkv.clone().to(DEV)
    ops.rope_kv_write(buf, torch.tensor(positions, dtype=torch.int32, device=DEV),
                      torch.tensor(slots, dtype=torch.int32, device=DEV), kc, vc, nh, nkv, d, rotary_dim, 10000.0)
    x = qkv.double().view(t, nh + 2 * nkv, d)
    pos = torch.tensor(positions)
    q_want = P.rope(x[:, :nh], pos, 10000.0, rotary_dim) if rotary_dim else x[:, :nh]
    k_want = P.rope(x[:, nh:nh + nkv], pos, 10000.0, rotary_dim) if rotary_dim else x[:, nh:nh + nkv]
    v_want = x[:, nh + nkv:]
    tol = dict(rtol=1e-5, atol=1e-5) if dt == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    out = buf.cpu().double().view(t, nh + 2 * nkv, d)
    close(out[:, :nh], q_want, what="q", **tol)
    assert torch.equal(out[:, nh:], x[:, nh:]) or rotary_dim       # k, v in the buffer are not the product
    kc_c, vc_c = (c.cpu().double() for c in ops.cache_to_plain(kc, vc))   # by token and dimension
    touched_k = torch.zeros_like(kc_c, dtype=torch.bool)
    touched_v = torch.zeros_like(vc_c, dtype=torch.bool)
    for i, s in enumerate(slots):
        pg, off = divmod(s, page)
        close(kc_c[pg, :, off, :], k_want[i], what=f"k row {i}", **tol)
        close(vc_c[pg, :, :, off], v_want[i], what=f"v row {i}", **tol)
        touched_k[pg, :, off, :] = True
        touched_v[pg, :, :, off] = True
    assert bool((kc_c[~touched_k] == sentinel).all()) and bool((vc_c[~touched_v] == sentinel).all()), "spill"


# --- attention --------------------------------------------------------------------

def paged_case(seqs, nh, nkv, d, page, dt, seed, poison=True, far=None):
    """seqs: [(cached tokens, new tokens)].  Builds q for the new tokens, keys and values for all,
    puts them into shuffled pages (NaN elsewhere) and returns what the kernels need plus the
    plain result."""
    rng = random.Random(seed)
    total_pages = sum(-(-(c + n) // page) for c, n in seqs) + 3
    free = list(range(total_pages))
    rng.shuffle(free)
    fill = float("nan") if poison else 0.0
    kc = torch.full((total_pages, nkv, page, d), fill, dtype=torch.float64)
    vc = torch.full((total_pages, nkv, d, page), fill, dtype=torch.float64)
    width = max(-(-(c + n) // page) for c, n in seqs) + 1
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    rows_q, row_seq, positions, seq_start, seq_ctx, wants = [], [], [], [0], [], []
    for s, (c, n) in enumerate(seqs):
        L = c + n
        k = rnd(L, nkv, d, seed=seed * 100 + 2 * s)
        v = rnd(L, nkv, d, seed=seed * 100 + 2 * s + 1)
        q = rnd(L, nh, d, seed=seed * 100 + 50 + s)
        if far is not None and L > far[1]:
            # one query (the last) and one far key made to stand out: a kernel that skips that
            # key, or reads its neighbour, is off by far more than rounding
            h, j = far
            q[L - 1, h] = 0.0
            q[L - 1, h, 0] = 16.0
            k[:, h // (nh // nkv), 0] = 0.0
            k[j, h // (nh // nkv), 0] = 16.0
        k, v, q = k.to(dt).double(), v.to(dt).double(), q.to(dt).double()
        for pidx in range(-(-L // page)):
            pg = free.pop()
            table[s, pidx] = pg
            lo, hi = pidx * page, min(L, (pidx + 1) * page)
            kc[pg, :, :hi - lo, :] = k[lo:hi].transpose(0, 1)
            vc[pg, :, :, :hi - lo] = v[lo:hi].permute(1, 2, 0)
        rows_q.append(q[c:])
        row_seq += [s] * n
        positions += list(range(c, L))
        seq_start.append(seq_start[-1] + n)
        seq_ctx.append(c)
        wants.append((q, k, v, c))
    qkv = torch.zeros(seq_start[-1], nh + 2 * nkv, d, dtype=torch.float64)
    qkv[:, :nh] = torch.cat(rows_q)
    return dict(qkv=qkv.view(seq_start[-1], -1).to(dt).to(DEV), kc=kc.to(dt).to(DEV), vc=vc.to(dt).to(DEV),
                table=table.to(DEV), row_seq=torch.tensor(row_seq, dtype=torch.int32, device=DEV),
                positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
                seq_start=seq_start, seq_ctx=seq_ctx, wants=wants, nh=nh, nkv=nkv, d=d)


def plain_result(case, window=0):
    outs = []
    for q, k, v, c in case["wants"]:
        outs.append(P.attention(q, k, v, window)[c:].reshape(q.shape[0] - c, -1))
    return torch.cat(outs)


SHAPES = [  # nh, nkv, d, page
    (4, 2, 16, 16), (3, 3, 32, 16), (6, 2, 48, 32), (32, 4, 64, 64), (8, 1, 128, 16), (32, 1, 16, 16), (2, 1, 256, 16),
]
SEQS = [(0, 33), (40, 1), (17, 2), (0, 1), (64, 70), (129, 1)]


@pytest.mark.parametrize("nh,nkv,d,page", SHAPES)
@pytest.mark.parametrize("window", [0, 20])
def test_attention_generic(ops, nh, nkv, d, page, window):
    for dt, tol in ((torch.float32, dict(rtol=1e-4, atol=1e-5)), (torch.bfloat16, dict(rtol=2e-2, atol=2e-2))):
        case = paged_case(SEQS, nh, nkv, d, page, dt, seed=3)
        got = ops.attention_generic(case["qkv"], case["kc"], case["vc"], case["table"], case["row_seq"],
                                    case["positions"], nh, nkv, d, window)
        close(got, plain_result(case, window), what=f"generic {dt}", **tol)


def run_mfma(ops, case, window, n_splits, q_tiles=1, shared=False, staged=False):
    nh, nkv, d = case["nh"], case["nkv"], case["d"]
    tpt = ops.attention_tile_tokens(nh, nkv) * q_tiles * (ops.ATTENTION_STAGED_WAVES if staged else 1)
    starts = [0]
    for s in range(len(case["seq_ctx"])):
        starts.append(starts[-1] + -(-(case["seq_start"][s + 1] - case["seq_start"][s]) // tpt))
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    kc, vc = ops.cache_from_plain(case["kc"], case["vc"])      # the layout the writers leave for these sizes
    return ops.attention_mfma(case["qkv"], kc, vc, case["table"], dev(case["seq_start"]),
                              dev(case["seq_ctx"]), dev(starts), starts[-1], nh, nkv, d, window,
                              1.0 / math.sqrt(d), n_splits, q_tiles, 2 if staged else int(shared))


@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 16), (32, 4, 64, 64), (8, 1, 128, 16)])
@pytest.mark.parametrize("window", [0, 40])
@pytest.mark.parametrize("slots,least", [(512, 1000), (512, 1), (100000, 2)])
def test_attention_mfma_from_a_work_list(ops, nh, nkv, d, page, window, slots, least, monkeypatch):
    """The prompt form from a work list: every piece's walk cut into as many parts as the host says (none with a
    least walk beyond these contexts of 1 to 134 tokens; up to five otherwise, by an even share of 512 or of very
    many places for workgroups), items in the host's order, rows with one part written at once and left alone by the
    merge.  The partial outputs are allocated where a tensor of NaNs has just been freed: a merge that read a
    part that no workgroup wrote would show."""
    import types
    monkeypatch.setattr(ops, "ATTENTION_SLOTS", slots)
    monkeypatch.setattr(ops, "ATTENTION_MIN_WALK", least)
    case = paged_case(SEQS, nh, nkv, d, page, torch.bfloat16, seed=5)
    want = plain_result(case, window)
    t = case["qkv"].shape[0]
    qt = ops.attention_q_tiles(d)
    piece = ops.attention_tile_tokens(nh, nkv) * qt * ops.ATTENTION_STAGED_WAVES
    starts = [0]
    for s in range(len(case["seq_ctx"])):
        starts.append(starts[-1] + -(-(case["seq_start"][s + 1] - case["seq_start"][s]) // piece))
    batch = types.SimpleNamespace(n_seqs=len(case["seq_ctx"]), n_tokens=t, seq_start=case["seq_start"], seq_ctx=case["seq_ctx"])
    items, row_parts, most = ops.prompt_work_list(batch, starts, piece, nkv * -(-(nh // nkv) // 16), window)
    assert sorted(i & 0xfffff for i in items if (i >> 20) & 15 == 0) == list(range(starts[-1])), "every piece once"
    assert all(sum(1 for i in items if i & 0xfffff == p) == next(i >> 24 for i in items if i & 0xfffff == p) for p in range(starts[-1]))
    assert (most > 1) == (least < 1000) and max(row_parts) == most
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    kc, vc = ops.cache_from_plain(case["kc"], case["vc"])
    junk = torch.full((most, t, nh, d), float("nan"), dtype=torch.float32, device=DEV)
    del junk
    got = ops.attention_mfma(case["qkv"], kc, vc, case["table"], dev(case["seq_start"]), dev(case["seq_ctx"]), dev(starts),
                             starts[-1], nh, nkv, d, window, 1.0 / math.sqrt(d), most, qt, 2, items=dev(items),
                             n_items=len(items), row_parts=dev(row_parts))
    close(got, want, rtol=2e-2, atol=2e-2, what=f"work list, {len(items)} items, up to {most} parts")
    if most == 1:        # nothing cut: the same keys in the same order as the grid's own order gives
        assert torch.equal(got, run_mfma(ops, case, window, 1, qt, staged=True))


@pytest.mark.parametrize("nh,nkv,d,page", SHAPES)
@pytest.mark.parametrize("window", [0, 20])
@pytest.mark.parametrize("n_splits", [1, 3, 16, 64])
def test_attention_mfma(ops, nh, nkv, d, page, window, n_splits):
    case = paged_case(SEQS, nh, nkv, d, page, torch.bfloat16, seed=4)
    assert ops.attention_mfma_supported(case["qkv"], case["kc"], d)
    got = run_mfma(ops, case, window, n_splits)
    close(got, plain_result(case, window), rtol=2e-2, atol=2e-2, what="mfma")
    many = ops.attention_q_tiles(d)                       # several query tiles per wave: the same result
    if many > 1:
        again = run_mfma(ops, case, window, n_splits, many)
        close(again, plain_result(case, window), rtol=2e-2, atol=2e-2, what="mfma, several tiles a wave")
        if n_splits == 1:   # (with split keys the parts are cut elsewhere: equal up to rounding only)
            assert torch.equal(again, got), "a row's result must not depend on how rows are grouped into waves"
    # four waves of a workgroup walking their keys together through LDS (the form prompts use)
    for qt in sorted({1, many}):
        staged = run_mfma(ops, case, window, n_splits, qt, staged=True)
        close(staged, plain_result(case, window), rtol=2e-2, atol=2e-2, what=f"mfma, key tiles staged in LDS, {qt} tiles a wave")
        if n_splits == 1:   # the same keys in the same order for every row: the same bits
            assert torch.equal(staged, got), "a row's result must not depend on which waves share its keys"
    # a workgroup's waves sharing one tile's keys (the form decoded tokens use)
    close(run_mfma(ops, case, window, n_splits, shared=True), plain_result(case, window), rtol=2e-2, atol=2e-2,
          what="mfma, keys shared between a workgroup's waves")


@pytest.mark.parametrize("n_splits", [1, 3])
def test_attention_of_a_decode_step_without_looking_requests_up(ops, n_splits):
    """Every request brings exactly one row: told so, the kernel takes request s for tile s and row s
    and asks for nothing before the block table and the query -- the same bits as with the lookup, for
    few requests and for more than a wave's lanes hold (70)."""
    for n_req in (5, 70):
        seqs = [(3 + 17 * i % 190, 1) for i in range(n_req)]
        case = paged_case(seqs, 8, 2, 32, 16, torch.bfloat16, seed=12)
        kc, vc = ops.cache_from_plain(case["kc"], case["vc"])
        dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
        args = (case["qkv"], kc, vc, case["table"], dev(case["seq_start"]), dev(case["seq_ctx"]),
                dev(list(range(n_req + 1))), n_req, 8, 2, 32, 0, 1.0 / math.sqrt(32), n_splits, 1, 1)
        looked_up = ops.attention_mfma(*args)
        told = ops.attention_mfma(*args, single_rows=True)
        assert torch.equal(told, looked_up)
        close(told, plain_result(case), rtol=2e-2, atol=2e-2, what=f"{n_req} single rows")
    with pytest.raises(Exception, match="single rows"):
        two = paged_case([(4, 2), (9, 1)], 8, 2, 32, 16, torch.bfloat16, seed=13)
        kc, vc = ops.cache_from_plain(two["kc"], two["vc"])
        ops.attention_mfma(two["qkv"], kc, vc, two["table"], dev(two["seq_start"]), dev(two["seq_ctx"]), dev([0, 1, 2]), 2,
                           8, 2, 32, 0, 1.0 / math.sqrt(32), 1, 1, 1, single_rows=True)


@pytest.mark.parametrize("n_splits", [1, 5])
def test_attention_far_key_among_hundreds(ops, n_splits):
    """The last query of each request looks at one key far back (position 3 of 400+): softmax puts
    nearly all weight there, so skipping it or reading a neighbour shows at once."""
    seqs = [(0, 420), (418, 2), (431, 1)]
    for dt, fn in ((torch.bfloat16, "mfma"), (torch.float32, "generic")):
        case = paged_case(seqs, 4, 2, 64, 16, dt, seed=5, far=(1, 3))
        want = plain_result(case)
        if fn == "mfma":
            got = run_mfma(ops, case, 0, n_splits)
            close(run_mfma(ops, case, 0, n_splits, 4, staged=True), want, rtol=2e-2, atol=2e-2, what="mfma, staged keys")
            shared = run_mfma(ops, case, 0, n_splits, shared=True)
            close(shared, want, rtol=2e-2, atol=2e-2, what="mfma, shared keys")
            assert float((shared[419].double().cpu().view(4, 64)[1] - case["wants"][0][2][3, 0]).abs().max()) < 0.05
        else:
            got = ops.attention_generic(case["qkv"], case["kc"], case["vc"], case["table"], case["row_seq"],
                                        case["positions"], 4, 2, 64, 0)
        close(got, want, rtol=2e-2, atol=2e-2, what=fn)
        v_far = case["wants"][0][2][3, 0]                          # the value row the far key carries
        last = got[419].double().cpu().view(4, 64)[1]
        assert float((last - v_far).abs().max()) < 0.05, "the far key's value must dominate"


@pytest.mark.parametrize("nh,nkv,d,page", [(8, 2, 128, 64), (16, 2, 64, 16)])
def test_attention_long_context(ops, nh, nkv, d, page):
    """A whole prompt of 2,200 tokens, a portion of 40 after 2,100 cached ones, single tokens after
    2,177 and 1,030: hundreds of key tiles a row, the block table beyond one register a lane for the
    small pages, a window that ends inside the cached part; every form and several ways to cut the keys."""
    seqs = [(0, 2200), (2100, 40), (2177, 1), (1030, 1)]
    case = paged_case(seqs, nh, nkv, d, page, torch.bfloat16, seed=12, poison=False)
    qt = ops.attention_q_tiles(d)
    for window in (0, 700):
        want = plain_result(case, window)
        for n_splits in (1, 8):
            close(run_mfma(ops, case, window, n_splits, qt, staged=True), want, rtol=2e-2, atol=2e-2,
                  what=f"staged, window {window}, {n_splits} parts")
            close(run_mfma(ops, case, window, n_splits, qt), want, rtol=2e-2, atol=2e-2,
                  what=f"independent waves, window {window}, {n_splits} parts")
    # (4,300 tokens in pages of 16 are 269 pages: more than the 256 table entries a wave keeps in its lanes)
    more = [(2199, 1)] + ([(4300, 2)] if page == 16 else [])
    decode = paged_case(seqs[2:] + more, nh, nkv, d, page, torch.bfloat16, seed=13, poison=False)
    for window in (0, 700):
        for n_splits in (1, 5, 64):
            close(run_mfma(ops, decode, window, n_splits, shared=True), plain_result(decode, window), rtol=2e-2, atol=2e-2,
                  what=f"shared keys, window {window}, {n_splits} parts")


def test_attention_walk_over_more_pages_than_the_table_copy_holds(ops):
    """The prompt form keeps a copy of its walk's part of the block table in LDS, 1,024 entries; a portion of 40 tokens
    after 16,500 cached ones in pages of 16 walks 1,034 pages, the last of them looked up in memory -- with the keys in
    one part and cut, and with a window that begins far into the walk."""
    case = paged_case([(16500, 40), (3, 20)], 4, 1, 32, 16, torch.bfloat16, seed=15, poison=False)
    qt = ops.attention_q_tiles(32)
    for window in (0, 900):
        want = plain_result(case, window)
        for n_splits in (1, 3):
            close(run_mfma(ops, case, window, n_splits, qt, staged=True), want, rtol=2e-2, atol=2e-2,
                  what=f"staged, window {window}, {n_splits} parts")


def test_attention_window_edge(ops):
    """Keys exactly at the window's edge: position p sees p - window + 1 but not p - window."""
    case = paged_case([(0, 50)], 2, 1, 32, 16, torch.bfloat16, seed=6, poison=False)
    for window in (1, 16, 17, 31, 32, 33):
        close(run_mfma(ops, case, window, 1), plain_result(case, window), rtol=2e-2, atol=2e-2, what=f"window {window}")
        close(run_mfma(ops, case, window, 1, shared=True), plain_result(case, window), rtol=2e-2, atol=2e-2,
              what=f"window {window}, shared keys")
        close(run_mfma(ops, case, window, 1, ops.attention_q_tiles(32), staged=True), plain_result(case, window), rtol=2e-2, atol=2e-2,
              what=f"window {window}, staged keys")


def test_argmax_ties_and_sampling(ops):
    logits = torch.full((3, 1000), -1.0)
    logits[0, 7] = logits[0, 500] = logits[0, 999] = 5.0             # tie: lowest index
    logits[1, 999] = 2.0                                              # maximum in the last place
    logits[2] = torch.linspace(0, 1, 1000)
    assert ops.argmax(logits.to(DEV)).tolist() == [7, 999, 999]
    from bare_cuda_4gib_amd.sampling import MT19937_64, SamplingParams, sample_token
    row = rnd(1, 32000, seed=20, scale=2.0).float()
    us = [MT19937_64(s).uniform() for s in range(64)]
    temps = [0.0 if i % 8 == 0 else 0.5 + 0.05 * i for i in range(64)]
    got = ops.sample(row.expand(64, -1).contiguous().to(DEV), torch.tensor(temps, device=DEV),
                     torch.tensor(us, dtype=torch.float64, device=DEV)).tolist()

    class Fixed:
        def __init__(self, u): self.u = u
        def uniform(self): return self.u
    for i in range(64):
        want = sample_token(row[0].numpy(), SamplingParams(temperature=temps[i]), Fixed(us[i]))
        if got[i] != want:   # float sums in another order may move a boundary by one token at most
            w = np.exp((row[0].numpy() - row[0].numpy().max()) / temps[i])
            cum = np.cumsum(w.astype(np.float64))
            edge = abs(us[i] * cum[-1] - cum[min(got[i], want)])
            assert abs(got[i] - want) == 1 and edge < 1e-3 * cum[-1], (i, got[i], want)


@pytest.mark.parametrize("vocab", [97, 1000, 1028, 128256, 300001, 2100003])
def test_sampling_follows_the_law_at_other_vocabularies(ops, vocab):
    """The device's draw against the host's walk through the vocabulary for the same uniform numbers:
    vocabularies that are no multiple of the 512-token groups (with and without a row start on 16 bytes: the
    kernel reads by four where it can), one as large as Llama 3's, and one beyond 2,097,152 tokens (a lane
    then takes more than eight tokens of a group); u near 0 and near 1 reach the ends."""
    from bare_cuda_4gib_amd.sampling import SamplingParams, sample_token
    row = rnd(1, vocab, seed=21, scale=2.0).float()
    us = [0.0, 1e-12, 0.25, 0.5, 0.731, 0.999999, 0.9999999999]
    temps = [1.0, 0.7, 1.3, 0.2, 2.0, 1.0, 1.0]
    got = ops.sample(row.expand(len(us), -1).contiguous().to(DEV), torch.tensor(temps, device=DEV),
                     torch.tensor(us, dtype=torch.float64, device=DEV)).tolist()

    class Fixed:
        def __init__(self, u): self.u = u
        def uniform(self): return self.u
    for i, (uu, t) in enumerate(zip(us, temps)):
        want = sample_token(row[0].numpy(), SamplingParams(temperature=t), Fixed(uu))
        if got[i] != want:   # sums in another order may move a boundary by one token at most
            w = np.exp((row[0].numpy() - row[0].numpy().max()) / t)
            cum = np.cumsum(w.astype(np.float64))
            edge = abs(uu * cum[-1] - cum[min(got[i], want)])
            assert abs(got[i] - want) == 1 and edge < 1e-6 * cum[-1], (vocab, i, got[i], want)


FILTERED_ROWS = {
    "normal": lambda g, n, v: g.normal(0, 2.0, (n, v)),
    "ties": lambda g, n, v: np.round(g.normal(0, 1.5, (n, v)) * 2) / 2,          # many tokens share a weight
    "equal": lambda g, n, v: np.full((n, v), 0.25),                             # all of them do
    "peaked": lambda g, n, v: g.normal(0, 1.0, (n, v)) + 12.0 * (g.random((n, v)) < 3.0 / v),   # as a model's rows are
    "wide": lambda g, n, v: g.normal(0, 30.0, (n, v)),                          # weights down to zero
}


@pytest.mark.parametrize("kind", sorted(FILTERED_ROWS))
@pytest.mark.parametrize("vocab", [7, 1000, 18433, 36864, 36865, 128256])
def test_filtered_sampling_follows_the_law(ops, vocab, kind):
    """Top-k, top-p and both on the device against the host's sorted walk (sampling/host.py, the reference's law)
    for the same uniform numbers, into chosen places of the output: rows whose candidates fit the kernel's list
    (peaked) and rows whose do not (flat: their patterns in LDS up to 36,864 tokens, worked out again beyond), rows
    where many or all tokens share a weight (the order of the ids decides), k beyond what one bucket holds, a
    nucleus of one token, u at both ends.  The same call twice gives the same ids (the sums are integer adds)."""
    from bare_cuda_4gib_amd.sampling import SamplingParams, sample_token
    gen = np.random.default_rng(vocab * 7 + len(kind))
    n = 30
    logits = FILTERED_ROWS[kind](gen, n + 2, vocab).astype(np.float32)
    us = gen.random(n)
    us[0], us[1], us[-1] = 0.0, 1e-12, 1.0 - 2.0 ** -53
    temps = np.array([(0.7, 1.0, 1.6, 0.05)[i % 4] for i in range(n)], np.float32)
    ks = np.array([(0, 1 + vocab // 50, 5, 2, 40, vocab - 1, 3)[i % 7] for i in range(n)], np.int32)
    ps = np.array([(0.9, 0.5, 0.99, 0.1, 1e-6)[(i // 2) % 5] if not 0 < ks[i] < vocab or i % 3 else 1.0 for i in range(n)], np.float64)
    # (a row with neither limit is not the kernel's: the law without filters walks in the order of the ids)
    rows = np.array([(i * 7) % (n + 2) for i in range(n)], np.int32)            # some logits rows, in another order
    assert len(set(rows.tolist())) == n
    dev = lambda a: torch.from_numpy(a).to(DEV)
    out = torch.full((n + 2,), -7, dtype=torch.int32, device=DEV)
    ops.sample_filtered(dev(logits), out, dev(rows), dev(temps), dev(us), dev(ks), dev(ps))
    again = torch.full((n + 2,), -7, dtype=torch.int32, device=DEV)
    ops.sample_filtered(dev(logits), again, dev(rows), dev(temps), dev(us), dev(ks), dev(ps))
    got = out.cpu().numpy()
    assert np.array_equal(got, again.cpu().numpy())
    assert sorted(np.nonzero(got == -7)[0].tolist()) == sorted(set(range(n + 2)) - set(rows.tolist()))   # the others untouched

    class Fixed:
        def __init__(self, u): self.u = u
        def uniform(self): return self.u
    for i in range(n):
        row = logits[rows[i]]
        params = SamplingParams(temperature=float(temps[i]), top_p=float(ps[i]), top_k=int(ks[i]))
        want = sample_token(row, params, Fixed(float(us[i])))
        if got[rows[i]] != want:      # sums in another order may move an edge by one place of the sorted walk
            w = np.exp((row - row.max()) * (np.float32(1.0) / temps[i])).astype(np.float32).astype(np.float64)
            order = np.lexsort((np.arange(vocab), -w))
            at = {int(t): j for j, t in enumerate(order[:max(int(ks[i]), 64) if ks[i] else vocab])}
            assert int(got[rows[i]]) in at and abs(at[int(got[rows[i]])] - at[want]) == 1, (vocab, kind, i, got[rows[i]], want)
            cum = np.cumsum(w[order])
            edge = min(abs(us[i] * c - cum[min(at[int(got[rows[i]])], at[want])]) for c in (cum[-1], cum[len(at) - 1]))
            assert edge < 1e-9 * cum[-1], (vocab, kind, i, got[rows[i]], want, edge)


def test_filtered_sampling_beyond_half_a_million_tokens(ops):
    """Beyond 2^19 tokens a bucket's count no longer fits beside its mantissa sum in one word: the kernel keeps the
    two apart there.  Rows whose candidates fit the list and rows whose do not."""
    from bare_cuda_4gib_amd.sampling import SamplingParams, sample_token
    vocab, n = 600001, 6
    gen = np.random.default_rng(5)
    logits = np.concatenate([FILTERED_ROWS["peaked"](gen, n // 2, vocab), FILTERED_ROWS["ties"](gen, n // 2, vocab)]).astype(np.float32)
    us = np.array([0.0, 0.37, 0.93, 0.5, 0.11, 1.0 - 2.0 ** -53])
    temps = np.array([1.0, 0.7, 1.3, 1.0, 0.7, 1.3], np.float32)
    ks = np.array([40, 0, 5, 0, 3000, 40], np.int32)
    ps = np.array([0.9, 0.5, 1.0, 0.9, 0.99, 0.3], np.float64)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    out = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    ops.sample_filtered(dev(logits), out, torch.arange(n, dtype=torch.int32, device=DEV), dev(temps), dev(us), dev(ks), dev(ps))

    class Fixed:
        def __init__(self, u): self.u = u
        def uniform(self): return self.u
    want = [sample_token(logits[i], SamplingParams(temperature=float(temps[i]), top_p=float(ps[i]), top_k=int(ks[i])),
                         Fixed(float(us[i]))) for i in range(n)]
    assert out.tolist() == want


def test_filtered_sampling_refuses_what_it_cannot_read(ops):
    logits = torch.zeros(2, 50, device=DEV)
    good = dict(out=torch.zeros(2, dtype=torch.int32, device=DEV), rows=torch.zeros(1, dtype=torch.int32, device=DEV),
                temperature=torch.ones(1, device=DEV), u=torch.zeros(1, dtype=torch.float64, device=DEV),
                top_k=torch.ones(1, dtype=torch.int32, device=DEV), top_p=torch.ones(1, dtype=torch.float64, device=DEV))
    ops.sample_filtered(logits, **good)
    for name, bad in (("out", torch.zeros(3, dtype=torch.int32, device=DEV)), ("u", torch.zeros(1, device=DEV)),
                      ("top_p", torch.ones(2, dtype=torch.float64, device=DEV)), ("top_k", torch.ones(1, device=DEV))):
        with pytest.raises(Exception, match="sample_filtered"):
            ops.sample_filtered(logits, **dict(good, **{name: bad}))
    with pytest.raises(Exception, match="sample_filtered"):
        ops.sample_filtered(logits.to(torch.bfloat16), **good)


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("n,k", [(130, 304), (2560, 2048), (301, 80)])
@pytest.mark.parametrize("gdt", [torch.bfloat16, torch.float32])
def test_gemm_with_fused_rmsnorm(ops, m, n, k, gdt):
    x = rnd(m + 3, k, seed=21, scale=3.0).float()
    g = (1.0 + 0.2 * rnd(k, seed=22)).to(gdt)
    w = bf(rnd(n, k, seed=23))
    rows = torch.tensor(list(range(m + 2, 2, -1)), dtype=torch.int32)          # a gather, in another order
    xs = x[rows.long()]
    # rounded where the kernel rounds: bf16(x * g) into the matrix cores, the row's scale afterwards
    hb = (xs * g.float()).to(torch.bfloat16).double()
    scale = 1.0 / torch.sqrt((xs.double() ** 2).mean(-1, keepdim=True) + 1e-5)
    exact = scale * (hb @ w.double().T)
    ideal = P.rmsnorm(xs.double(), g.double(), 1e-5) @ w.double().T
    mag = math.sqrt(k)
    got = ops.gemm_normed(x.to(DEV), rows.to(DEV), m, g.to(DEV), 1e-5, w.to(DEV), ops.EPI_STORE_F32)
    close(got, exact, 1e-4, 1e-4 * mag, "fused norm, same rounding")
    close(got, ideal, 2e-2, 1e-2 * mag, "fused norm, ideal")
    whole = ops.gemm_normed(x[:m].contiguous().to(DEV), None, m, g.to(DEV), 1e-5, w.to(DEV), ops.EPI_STORE_BF16)
    close(whole, P.rmsnorm(x.double()[:m], g.double(), 1e-5) @ w.double().T, 2e-2, 1e-2 * mag, "fused norm bf16")
    if n % 16 == 0:
        got = ops.gemm_normed(x.to(DEV), rows.to(DEV), m, g.to(DEV), 1e-5, w.to(DEV), ops.EPI_SWIGLU)
        blocks = exact.view(m, n // 16, 2, 8)                    # w read as interleaved gate/up blocks
        want = P.swiglu(blocks[:, :, 0, :], blocks[:, :, 1, :]).reshape(m, n // 2)
        close(got, want, 1e-2, 1e-2 * mag, "fused norm + swiglu")


def block_order(d):
    half = d // 2
    return [8 * b + t if t < 8 else half + 8 * b + (t - 8) for b in range(d // 16) for t in range(16)]


@pytest.mark.parametrize("nh,nkv,d", [(4, 2, 16), (3, 3, 32), (6, 2, 48), (32, 4, 64)])
@pytest.mark.parametrize("m,normed", [(1, True), (9, True), (16, False), (40, False)])
@pytest.mark.parametrize("rotate", [True, False])
def test_qkv_product_with_rotation_and_cache_write(ops, nh, nkv, d, m, normed, rotate):
    """The fused decode kernel against: plain product, plain rotation, rows written where the slot
    map says -- all in the reordered head layout -- and against the unfused kernels bit for bit in
    what they share (the cache contents for the same inputs)."""
    k, page, pages, theta = 80, 16, 7, 500.0
    order = block_order(d)
    w = bf(rnd((nh + 2 * nkv) * d, k, seed=30, scale=0.3))
    wp = w.view(nh + 2 * nkv, d, k)[:, order, :].reshape(-1, k).contiguous()        # reordered rows
    positions = [3 + 5 * i for i in range(m)]
    slots = random.Random(1).sample(range(pages * page), m)
    g = (1.0 + 0.1 * rnd(k, seed=31)).bfloat16()
    if normed:
        x = rnd(m, k, seed=32, scale=2.0).float()
        hb = (x * g.float()).to(torch.bfloat16).double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5)
        xin, gin = x.to(DEV), g.to(DEV)
    else:
        hb = bf(rnd(m, k, seed=32)).double()
        xin, gin = hb.to(torch.bfloat16).to(DEV), None
    qkv = (hb @ w.double().T).view(m, nh + 2 * nkv, d)
    pos = torch.tensor(positions)
    rd = d if rotate else 0
    q_want = P.rope(qkv[:, :nh], pos, theta) if rotate else qkv[:, :nh]
    k_want = P.rope(qkv[:, nh:nh + nkv], pos, theta) if rotate else qkv[:, nh:nh + nkv]
    v_want = qkv[:, nh + nkv:]
    kc = torch.full((pages, nkv, page, d), -7.5, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((pages, nkv, d, page), -7.5, dtype=torch.bfloat16, device=DEV)
    q = ops.gemm_qkv_rope(xin, gin, 1e-5, wp.to(DEV), torch.tensor(positions, dtype=torch.int32, device=DEV),
                          torch.tensor(slots, dtype=torch.int32, device=DEV), kc, vc, nh, nkv, d, rd, theta)
    tol = dict(rtol=2e-2, atol=3e-2)
    close(q.view(m, nh, d), q_want[:, :, order], what="q", **tol)
    kc_c, vc_c = (c.cpu().double() for c in ops.cache_to_plain(kc, vc))   # by token and dimension
    seen_k, seen_v = torch.zeros_like(kc_c, dtype=torch.bool), torch.zeros_like(vc_c, dtype=torch.bool)
    for i, s in enumerate(slots):
        pg, off = divmod(s, page)
        close(kc_c[pg, :, off, :], k_want[i][:, order], what=f"k row {i}", **tol)
        close(vc_c[pg, :, :, off], v_want[i][:, order], what=f"v row {i}", **tol)
        seen_k[pg, :, off, :] = True
        seen_v[pg, :, :, off] = True
    assert bool((kc_c[~seen_k] == -7.5).all()) and bool((vc_c[~seen_v] == -7.5).all()), "spill"
    if not normed:   # the unfused pair of kernels on the same reordered weights writes the same cache
        kc2, vc2 = torch.full_like(kc, -7.5), torch.full_like(vc, -7.5)
        buf = ops.gemm_fast(xin, wp.to(DEV), torch.bfloat16)
        ops.rope_kv_write(buf, torch.tensor(positions, dtype=torch.int32, device=DEV),
                          torch.tensor(slots, dtype=torch.int32, device=DEV), kc2, vc2, nh, nkv, d, rd, theta,
                          block_pairs=True)
        kc2, vc2 = ops.cache_to_plain(kc2, vc2)
        close(kc2, kc_c, 1e-2, 2e-2, "unfused keys")
        close(vc2, vc_c, 1e-2, 2e-2, "unfused values")
        close(buf.view(m, nh + 2 * nkv, d)[:, :nh], q.view(m, nh, d), 1e-2, 2e-2, "unfused queries")


@pytest.mark.parametrize("nh,nkv,d,m,k,page", [(4, 2, 16, 200, 64, 16), (6, 2, 48, 333, 128, 16), (32, 4, 64, 2048 - 20, 192, 64),
                                               (24, 8, 128, 2048 - 20, 192, 32), (32, 8, 128, 4096 - 236, 192, 64),
                                               (16, 8, 128, 4096 - 236, 192, 64), (16, 8, 128, 2048 - 20, 192, 64),
                                               (8, 4, 128, 2048 - 20, 1024, 64), (32, 4, 64, 2048 - 20, 1024, 64),
                                               (64, 32, 64, 56, 192, 64)])
@pytest.mark.parametrize("rotate", [True, False])
def test_tiled_qkv_product_with_rotation_and_cache_write(ops, nh, nkv, d, m, k, page, rotate):
    """The same for the many rows of a prompt portion, in the tiled kernel's epilogue (every tile, 64 x 64 up to
    256 x 256, by the shapes; the last five 256 x 256, 256 x 128, 128 x 128, 128 x 64 and a wide output of few rows): queries rotated, keys rotated into the pages the slot map names, values into theirs, nothing else
    touched -- against the plain product and rotation, and against the unfused pair of kernels."""
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the shapes are chosen for 256 CUs")
    theta = 500.0
    order = block_order(d)
    pages = -(-m // page) + 3                                     # (room for the rows in a row from the second page on)
    w = bf(rnd((nh + 2 * nkv) * d, k, seed=33, scale=0.3))
    wp = w.view(nh + 2 * nkv, d, k)[:, order, :].reshape(-1, k).contiguous()        # reordered rows
    positions = [3 + 5 * i for i in range(m)]
    slots = random.Random(2).sample(range(pages * page), m)
    x = bf(rnd(m, k, seed=34))
    xin = x.to(DEV)
    assert ops.gemm_qkv_rope_tiled_supported(xin, wp.to(DEV), d, d if rotate else 0)
    qkv = (x.double() @ w.double().T).view(m, nh + 2 * nkv, d)
    pos = torch.tensor(positions)
    q_want = P.rope(qkv[:, :nh], pos, theta) if rotate else qkv[:, :nh]
    k_want = P.rope(qkv[:, nh:nh + nkv], pos, theta) if rotate else qkv[:, nh:nh + nkv]
    v_want = qkv[:, nh + nkv:]
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    kc = torch.full((pages, nkv, page, d), -7.5, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((pages, nkv, d, page), -7.5, dtype=torch.bfloat16, device=DEV)
    table = ops.rope_table(dev(positions), d, theta) if rotate else None
    q = ops.gemm_qkv_rope_tiled(xin, wp.to(DEV), table, dev(slots), kc, vc, nh, nkv, d)
    assert tuple(q.shape) == (m, nh * d)
    tol = dict(rtol=2e-2, atol=3e-2)
    close(q.view(m, nh, d), q_want[:, :, order], what="q", **tol)
    kc_c, vc_c = (c.cpu().double() for c in ops.cache_to_plain(kc, vc))   # by token and dimension
    at = torch.tensor(slots)
    close(kc_c[at // page, :, at % page, :], k_want[:, :, order], what="keys", **tol)
    close(vc_c[at // page, :, :, at % page], v_want[:, :, order], what="values", **tol)
    seen = torch.zeros(pages, page, dtype=torch.bool)
    seen[at // page, at % page] = True
    assert bool((kc_c.permute(0, 2, 1, 3)[~seen] == -7.5).all()) and bool((vc_c.permute(0, 3, 1, 2)[~seen] == -7.5).all()), "spill"
    # the unfused pair: the product rounded to bfloat16 before it is rotated (either half of a pair is off by up to
    # 2^-9 of itself there, and the rotation mixes the two), then rounded once more
    kc2, vc2 = torch.full_like(kc, -7.5), torch.full_like(vc, -7.5)
    buf = ops.gemm_fast(xin, wp.to(DEV), torch.bfloat16)
    ops.rope_kv_write_blocks(buf, table, dev(slots), kc2, vc2, nh, nkv, d)
    kc2, vc2 = ops.cache_to_plain(kc2, vc2)
    twice = 2.0 ** -7 * float(qkv.abs().max())
    close(kc2, kc_c, 1e-2, twice, "unfused keys")
    close(vc2, vc_c, 1e-2, twice, "unfused values")
    close(buf.view(m, nh + 2 * nkv, d)[:, :nh], q.view(m, nh, d), 1e-2, twice, "unfused queries")
    # without the cache (a layer that reads another layer's): queries only
    q_only = ops.gemm_qkv_rope_tiled(xin, wp.to(DEV), table, None, None, None, nh, nkv, d, write_kv=False)
    assert torch.equal(q_only, q)
    # a prompt portion's tokens lie one after the other in their pages (four tokens of a value dimension are then
    # stored at once, where the four begin at a multiple of four): from the first place of a page, and from its fourth
    for first in (page, page + 3):
        run = [first + i for i in range(m)]
        kc3, vc3 = torch.full_like(kc, -7.5), torch.full_like(vc, -7.5)
        assert torch.equal(ops.gemm_qkv_rope_tiled(xin, wp.to(DEV), table, dev(run), kc3, vc3, nh, nkv, d), q)
        kc3, vc3 = (c.cpu().double() for c in ops.cache_to_plain(kc3, vc3))
        to = torch.tensor(run)
        assert torch.equal(kc3[to // page, :, to % page, :], kc_c[at // page, :, at % page, :]), "the same keys, elsewhere"
        assert torch.equal(vc3[to // page, :, :, to % page], vc_c[at // page, :, :, at % page]), "the same values, elsewhere"
        free = torch.ones(pages, page, dtype=torch.bool)
        free[to // page, to % page] = False
        assert bool((kc3.permute(0, 2, 1, 3)[free] == -7.5).all()) and bool((vc3.permute(0, 3, 1, 2)[free] == -7.5).all()), "spill"


@pytest.mark.parametrize("m,width,n2", [(24, 128, 8192), (37, 320, 8208), (64, 2048, 11264), (50, 192, 9008)])
def test_tiled_swiglu_finishes_a_prepared_norm(ops, m, width, n2):
    """A wide gate-up product of 24 to 64 rows goes to the tiled kernel, which takes what the adding product before it
    left (bfloat16(residual * g) and the parts of the rows' sums of squares) and puts every row's factor into its
    epilogue: equal to SwiGLU of rmsnorm(residual) w^T up to rounding, and to what the weight-streaming kernel makes
    of the same operands (rows whose sizes differ a hundredfold show a factor taken from the wrong row), in
    tiles that hang over the rows and the columns, and with other things having been in the parts' memory."""
    k = 64
    a, w = bf(rnd(m, k, seed=80)), bf(rnd(width, k, seed=81, scale=0.3))
    g = bf(1.0 + 0.2 * rnd(width, seed=82))
    base = rnd(m, width, seed=83, scale=2.0).float()
    base *= torch.tensor([100.0 if r % 3 == 1 else (0.01 if r % 3 == 2 else 1.0) for r in range(m)]).unsqueeze(1)
    res = base.clone().to(DEV)
    torch.full((4096,), 1e30, device=DEV)                     # (freed at once: what the next allocations may find)
    pre = ops.gemm_accumulate_emit(a.to(DEV), w.to(DEV), res, g.to(DEV), 1e-5)
    r = res.cpu()
    hb = pre.xb.cpu().double() / torch.sqrt((r.double() ** 2).mean(-1, keepdim=True) + 1e-5)
    w2 = bf(rnd(n2, width, seed=84, scale=0.3))
    wi = interleave8(w2[:n2 // 2], w2[n2 // 2:]).to(DEV)
    assert not ops.streams_weights(m, n2, width) and ops.gemm_prenormed_supported(pre, wi, ops.EPI_SWIGLU)
    assert not ops.gemm_prenormed_supported(pre, wi, ops.EPI_STORE_BF16)
    got = ops.gemm_prenormed(pre, wi, ops.EPI_SWIGLU)
    gu = hb @ w2.double().T
    close(got, P.swiglu(gu[:, :n2 // 2], gu[:, n2 // 2:]), 8e-3, 3e-2, "prenormed, SwiGLU, tiled")
    # the weight-streaming kernel on the first 23 rows of the same operands: the same factor from the same parts
    few = ops.Prenormed(pre.xb[:23].contiguous(), pre.parts[:, :23].contiguous(), pre.eps)
    assert ops.streams_weights(23, n2, width)
    close(got[:23], ops.gemm_prenormed(few, wi, ops.EPI_SWIGLU), 8e-3, 1e-3, "against the weight-streaming kernel")


@pytest.mark.parametrize("m", [1, 5, 8, 9, 16, 33, 64])
@pytest.mark.parametrize("width,k,gdt", [(96, 40, torch.bfloat16), (2048, 256, torch.bfloat16), (200, 72, torch.float32)])
def test_adding_product_prepares_the_next_norm(ops, m, width, k, gdt):
    """The product that adds into the residual stream also leaves bfloat16(new residual * g) and, per
    block of 16 columns, every row's part of its sum of squares; the product after it takes both
    instead of a norm.  The residual is the same bits as without the extra outputs; what is left is
    exactly what the definition says; and the next product equals rmsnorm(residual) w^T computed from
    the residual it saw -- with every epilogue, the q|k|v one with rotation and cache write included."""
    a, w = bf(rnd(m, k, seed=70)), bf(rnd(width, k, seed=71, scale=0.3))
    g = (1.0 + 0.2 * rnd(width, seed=72)).to(gdt)
    base = rnd(m, width, seed=73, scale=2.0).float()
    res, res_plain = base.clone().to(DEV), base.clone().to(DEV)
    assert ops.gemm_emit_supported(a.to(DEV), w.to(DEV), res, g.to(DEV))
    pre = ops.gemm_accumulate_emit(a.to(DEV), w.to(DEV), res, g.to(DEV), 1e-5)
    ops.gemm_fast(a.to(DEV), w.to(DEV), accumulate_into=res_plain)
    assert torch.equal(res, res_plain)
    r = res.cpu()
    assert torch.equal(pre.xb.cpu(), (r * g.float()).to(torch.bfloat16))
    assert tuple(pre.parts.shape) == (-(-width // 16), m)
    pad = torch.zeros(m, 16 * pre.parts.shape[0])
    pad[:, :width] = r
    close(pre.parts.cpu().T, (pad.double() ** 2).view(m, -1, 16).sum(-1), 1e-5, 1e-6, "parts of the sums of squares")
    # the product after it
    hb = pre.xb.cpu().double() / torch.sqrt((r.double() ** 2).mean(-1, keepdim=True) + 1e-5)
    n2 = 176
    w2 = bf(rnd(n2, width, seed=74, scale=0.3))
    scale = math.sqrt(width)
    close(ops.gemm_prenormed(pre, w2.to(DEV), ops.EPI_STORE_F32), hb @ w2.double().T, 1e-4, 1e-4 * scale, "prenormed -> f32")
    close(ops.gemm_prenormed(pre, w2.to(DEV), ops.EPI_STORE_BF16), hb @ w2.double().T, 8e-3, 1e-3 * scale, "prenormed -> bf16")
    gu = hb @ w2.double().T
    wi = interleave8(w2[:n2 // 2], w2[n2 // 2:])
    close(ops.gemm_prenormed(pre, wi.to(DEV), ops.EPI_SWIGLU), P.swiglu(gu[:, :n2 // 2], gu[:, n2 // 2:]), 8e-3, 3e-2,
          "prenormed, SwiGLU")
    if m <= 8 and width % 8 == 0:   # the norm fused into the product instead: the same up to rounding
        fused = ops.gemm_normed(res, None, m, g.to(DEV), 1e-5, w2.to(DEV), ops.EPI_STORE_F32)
        close(ops.gemm_prenormed(pre, w2.to(DEV), ops.EPI_STORE_F32), fused, 1e-4, 1e-4 * scale, "against the fused norm")
    if m <= 64:
        nh, nkv, d, page, pages, theta = 3, 1, 32, 16, 8, 10000.0
        order = block_order(d)
        wq = bf(rnd((nh + 2 * nkv) * d, width, seed=75, scale=0.3))
        wp = wq.view(nh + 2 * nkv, d, width)[:, order, :].reshape(-1, width).contiguous()
        positions = [2 + 3 * i for i in range(m)]
        slots = random.Random(2).sample(range(pages * page), m)
        kc = torch.full((pages, nkv, page, d), -7.5, dtype=torch.bfloat16, device=DEV)
        vc = torch.full((pages, nkv, d, page), -7.5, dtype=torch.bfloat16, device=DEV)
        q = ops.gemm_qkv_rope(pre.xb, None, 0.0, wp.to(DEV), torch.tensor(positions, dtype=torch.int32, device=DEV),
                              torch.tensor(slots, dtype=torch.int32, device=DEV), kc, vc, nh, nkv, d, d, theta, pre=pre)
        qkv = (hb @ wq.double().T).view(m, nh + 2 * nkv, d)
        pos = torch.tensor(positions)
        tol = dict(rtol=2e-2, atol=3e-2)
        close(q.view(m, nh, d), P.rope(qkv[:, :nh], pos, theta)[:, :, order], what="q after a prepared norm", **tol)
        kc_c, vc_c = (c.cpu().double() for c in ops.cache_to_plain(kc, vc))
        k_want = P.rope(qkv[:, nh:nh + nkv], pos, theta)
        for i, sl in enumerate(slots):
            pg, off = divmod(sl, page)
            close(kc_c[pg, :, off, :], k_want[i][:, order], what=f"k row {i} after a prepared norm", **tol)
            close(vc_c[pg, :, :, off], qkv[i, nh + nkv:][:, order], what=f"v row {i} after a prepared norm", **tol)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (7, 100, 200), (33, 272, 1000), (64, 16, 8)])
def test_streamed_weight_packing(ops, m, n, k):
    """The packed copy holds the same matrix: the weight-streaming kernel gives, bit for bit, what
    it gives for a copy packed on the host by the layout's definition, and that is x w^T."""
    torch.manual_seed(m + n + k)
    w = (torch.randn(n, k) * 0.1).bfloat16()
    x = torch.randn(m, k).bfloat16()
    nb, ks = -(-n // 16), -(-k // 32)
    host = torch.zeros(nb, ks, 64, 8, dtype=torch.bfloat16)
    for row in range(n):
        for kk in range(0, k, 8):
            lane = ((kk % 32) // 8) * 16 + row % 16
            host[row // 16, kk // 32, lane] = w[row, kk:kk + 8]
    held = ops.StreamedWeight(w.cuda())
    assert torch.equal(held.packed.cpu(), host.view(-1))
    out = ops.gemm_fast(x.cuda(), held, torch.float32)
    want = x.double() @ w.double().T
    torch.testing.assert_close(out.cpu().double(), want, rtol=2e-3, atol=2e-3)
    assert torch.equal(out, ops.gemm_fast(x.cuda(), w.cuda(), torch.float32))


def test_products_at_random_sizes(ops):
    """Forty seeded draws of (rows, outputs, k): every row count from 1 to 140 crosses the kernels'
    borders (16 rows a tile, 64 a pass, 128 rows to the tiled kernel), outputs are multiples of
    nothing, k any multiple of 8 -- each against the product in double precision, stored as bfloat16,
    as float, and added into a float matrix."""
    rng = random.Random(2024)
    for case in range(40):
        m = rng.choice([1, 2, 7, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 140])
        n = rng.choice([1, 5, 16, 17, 40, 129, 250, 511])
        k = 8 * rng.choice([1, 2, 3, 5, 8, 13, 32, 33, 64, 100, 129])
        a, w = bf(rnd(m, k, seed=100 + case)), bf(rnd(n, k, seed=200 + case))
        want = a.double() @ w.double().T
        scale = math.sqrt(k)
        ad, wd = a.to(DEV), ops.StreamedWeight(w.to(DEV))
        close(ops.gemm_fast(ad, wd, torch.float32), want, 1e-4, 1e-4 * scale, f"case {case}: {m}x{n}x{k} -> f32")
        close(ops.gemm_fast(ad, wd, torch.bfloat16), want, 8e-3, 1e-3 * scale, f"case {case}: {m}x{n}x{k} -> bf16")
        base = rnd(m, n, seed=300 + case).float()
        acc = base.clone().to(DEV)
        ops.gemm_fast(ad, wd, accumulate_into=acc)
        close(acc, want + base.double(), 1e-4, 1e-4 * scale, f"case {case}: {m}x{n}x{k} accumulate")


def test_attention_at_random_batches(ops):
    """Twelve seeded batches of up to five requests -- cached lengths and new tokens at random, pages
    of 16 or 32 tokens, with and without a window -- through the three forms of the matrix-core
    kernel with random cuts of the keys, each against the plain result."""
    rng = random.Random(77)
    for case in range(12):
        nh, nkv, d, page = rng.choice([(4, 2, 16, 16), (6, 2, 48, 32), (8, 2, 64, 16), (4, 4, 128, 32), (16, 1, 32, 16)])
        seqs = [(rng.choice([0, 1, 15, 16, 17, 63, 64, 200]), rng.choice([1, 1, 2, 3, 16, 33, 70])) for _ in range(rng.randint(1, 5))]
        window = rng.choice([0, 0, 24, 65])
        data = paged_case(seqs, nh, nkv, d, page, torch.bfloat16, seed=500 + case)
        want = plain_result(data, window)
        what = f"case {case}: heads {nh}/{nkv} d={d} page={page} window={window} {seqs}"
        qt = ops.attention_q_tiles(d)
        for n_splits in (1, rng.choice([2, 3, 7])):
            close(run_mfma(ops, data, window, n_splits, qt, staged=True), want, rtol=2e-2, atol=2e-2, what=what + " staged")
            close(run_mfma(ops, data, window, n_splits, qt), want, rtol=2e-2, atol=2e-2, what=what + " independent")
            close(run_mfma(ops, data, window, n_splits, shared=True), want, rtol=2e-2, atol=2e-2, what=what + " shared")


@pytest.mark.parametrize("m,n,k", [(2048, 11264, 2048), (300, 2048, 5632), (2048, 2560, 2048), (96, 2048, 2048), (70, 200, 192),
                                   (1000, 4096, 4096), (130, 32000, 2048)])
def test_the_tiled_kernel_reads_the_packed_weight(ops, m, n, k):
    """A bound weight whose k is whole steps of 64 is held once, packed for the weight-streaming kernel; the tiled
    kernel reads that copy and gives the bits it gives from the rows -- for every tile form these shapes select, for
    the store, accumulate and SwiGLU epilogues and with k cut over workgroups -- and the rows are not kept."""
    torch.manual_seed(n + k)
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    a = torch.randn(m, k, device=DEV).bfloat16()
    held = ops.StreamedWeight(w)
    assert held.packed is not None and not held.holds_rows
    assert not ops.streams_weights(m, n, k)
    for dtype in (torch.bfloat16, torch.float32):
        assert torch.equal(ops.gemm_fast(a, held, dtype), ops.gemm_fast(a, w, dtype))
    base = torch.randn(m, n, device=DEV)
    one, two = base.clone(), base.clone()
    ops.gemm_fast(a, held, accumulate_into=one)
    ops.gemm_fast(a, w, accumulate_into=two)
    assert torch.equal(one, two)
    if n % 16 == 0:
        assert torch.equal(ops.gemm_swiglu(a, held, True), ops.gemm_swiglu(a, w, True))
    g = torch.ones(n, device=DEV, dtype=torch.bfloat16)
    if ops.gemm_parts_supported(a, w, base, g):
        one, two = base.clone(), base.clone()
        f1 = ops.gemm_parts_accumulate_norm(a, held, one, g, 1e-5)
        f2 = ops.gemm_parts_accumulate_norm(a, w, two, g, 1e-5)
        assert torch.equal(one, two) and torch.equal(f1.tensor, f2.tensor)
    assert not held.holds_rows
    assert torch.equal(held.rows, w) and held.holds_rows                 # made from the packed copy when someone asks


def test_a_weight_the_tiled_kernel_cannot_read_packed_keeps_its_rows(ops):
    w = (torch.randn(48, 176, device=DEV) * 0.05).bfloat16()            # k no multiple of 64
    held = ops.StreamedWeight(w)
    assert held.packed is not None and held.holds_rows
    a = torch.randn(100, 176, device=DEV).bfloat16()
    assert torch.equal(ops.gemm_fast(a, held, torch.float32), ops.gemm_fast(a, w, torch.float32))
    f32 = ops.StreamedWeight(w.float())
    assert f32.packed is None and f32.holds_rows


@pytest.mark.parametrize("dtypes", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16)])
def test_the_plain_product_s_two_tiles_give_the_same_bits(ops, dtypes):
    """Up to 16 rows the plain float product runs in tiles of 16 x 16 (sixteen times the blocks, for a decode step of
    the 32-bit path), beyond that in tiles of 64 x 64; every output element is the same sum over k in ascending order
    in one thread either way, so a row's bits do not depend on how many rows came with it."""
    ta, tw = dtypes
    for m, n, k in ((16, 301, 176), (3, 64, 2048), (9, 1000, 88)):
        torch.manual_seed(m + n + k)
        a = torch.randn(40, k, device=DEV).to(ta)
        w = (torch.randn(n, k, device=DEV) * 0.1).to(tw)
        many = ops.gemm_generic(a, w, torch.float32)                       # 40 rows: the large tile
        few = ops.gemm_generic(a[:m].contiguous(), w, torch.float32)       # the small one
        assert torch.equal(few, many[:m])
        want = a[:m].double() @ w.double().T
        torch.testing.assert_close(few.double(), want, rtol=1e-4, atol=1e-4 * math.sqrt(k))
        base = torch.randn(40, n, device=DEV)
        one, two = base.clone(), base[:m].clone()
        ops.gemm_generic(a, w, accumulate_into=one)
        ops.gemm_generic(a[:m].contiguous(), w, accumulate_into=two)
        assert torch.equal(two, one[:m])
