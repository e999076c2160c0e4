"""That the framework's parts are general: a toy architecture, defined here and registered from
here without a change to the framework's files, with
  - a mixer with state of its own (a running mean over the request's tokens, kept in a state slot),
  - attention with a window (its cache group gives pages back as the window moves on),
  - a layer that runs twice (own cache each time) and a layer that reads another layer's cache,
  - attention without any position encoding,
  - (a second toy) a feed-forward with routing and a position encoding of another pairing,
is built, loaded from a random model folder, and stepped whole, in portions, and mixed with few
pages -- against a plain implementation of the same toy model written with the plain functions.
Each part of a layer is also run alone against its plain function."""
import dataclasses
import json
import os

import numpy as np
import pytest
import torch

import helpers
import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

H, NH, NKV, D, INTER, VOCAB, WINDOW = 48, 4, 2, 16, 80, 97, 24


def register_toy():
    from bare_cuda_4gib_amd.cache import FixedState
    from bare_cuda_4gib_amd.config import Architecture, ModelConfig, field_from_json, register_architecture
    from bare_cuda_4gib_amd.config.registry import unregister_architecture
    from bare_cuda_4gib_amd.engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from bare_cuda_4gib_amd.parts import Part, register_part
    from bare_cuda_4gib_amd.weights import WeightSpec

    class RunningMean(Part):
        """out[t] = W * mean(h[0..t]) over the request's tokens so far; state = [sum of h, count]."""
        category = "mixer"

        def __init__(self, hidden_size):
            self.hidden = hidden_size

        def cache_spec(self):
            return FixedState((self.hidden + 1,), "float32")

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.hidden, self.hidden))}

        def bind(self, tensors, rt):
            self.w = tensors["mix.weight"].float()

        def forward(self, h, ctx, cache, residual, writes=True):
            h = h.float()
            for s in range(ctx.n_seqs):
                a, b = ctx.seq_start[s], ctx.seq_start[s + 1]
                state = cache.state[ctx.seq_slots[s]]
                sums = torch.cumsum(h[a:b], dim=0) + state[:self.hidden]
                counts = torch.arange(1, b - a + 1, device=h.device, dtype=torch.float32) + state[self.hidden]
                residual[a:b] += (sums / counts[:, None]) @ self.w.T
                if writes:
                    state[:self.hidden] = sums[-1]
                    state[self.hidden] = counts[-1]

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        vocab_size: int = field_from_json("vocab_size")
        hidden_size: int = field_from_json("hidden_size")
        window: int = field_from_json("window")
        eps: float = field_from_json("eps")

    def describe(cfg):
        norm = dict(size=cfg.hidden_size, eps=cfg.eps)
        def attn(prefix, window, position):
            return PartSpec("attention", dict(hidden_size=cfg.hidden_size, num_heads=NH, num_kv_heads=NKV, head_dim=D,
                                              window=window, position=position), prefix=prefix)
        rot = PartSpec("rotary", dict(theta=100.0, dim=8))              # rotary on half of the head only
        def layer(i, mixer):
            p = f"blocks.{i}."
            return LayerSpec("prenorm", mixer, PartSpec("swiglu", dict(hidden_size=cfg.hidden_size, intermediate_size=INTER),
                                                        prefix=p + "ffn."),
                             PartSpec("rmsnorm", dict(norm), prefix=p + "norm1."), PartSpec("rmsnorm", dict(norm), prefix=p + "norm2."))
        layers = [layer(0, attn("blocks.0.attn.", cfg.window, rot)),
                  layer(1, PartSpec("toy_running_mean", dict(hidden_size=cfg.hidden_size), prefix="blocks.1.")),
                  layer(2, attn("blocks.2.attn.", 0, PartSpec("none", {}))),
                  layer(3, attn("blocks.3.attn.", 0, rot))]
        schedule = [ScheduleEntry(0, "win"), ScheduleEntry(1, "mean"), ScheduleEntry(2, "full-a"),
                    ScheduleEntry(2, "full-b"),                           # the same layer again, a cache of its own
                    ScheduleEntry(3, "full-a", writes=False)]             # reads what layer 2's first run cached
        return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, max_seq_len=4096,
                         embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="embed."),
                         layers=layers, schedule=schedule, final_norm=PartSpec("rmsnorm", dict(norm), prefix="final_norm."),
                         head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, tied_to="embed.weight"),
                                       prefix="head."))

    try:
        register_part("mixer", "toy_running_mean", RunningMean)
    except Exception:
        pass
    unregister_architecture("ToyHybridForTests")
    register_architecture(Architecture("ToyHybridForTests", "toy_hybrid_for_tests", ToyConfig, describe))


TOY_CONFIG = dict(architectures=["ToyHybridForTests"], vocab_size=VOCAB, hidden_size=H, window=WINDOW, eps=1e-4)


def plain_toy_logits(folder, ids):
    """The toy model, whole sequence, float64, from the plain functions."""
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        w = {n: f.get_tensor(n).double() for n in f.keys()}
    t = len(ids)
    pos = torch.arange(t)
    x = w["embed.weight"][torch.tensor(ids)]

    def qkv(p, h):
        q = (h @ w[p + "q_proj.weight"].T).view(t, NH, D)
        k = (h @ w[p + "k_proj.weight"].T).view(t, NKV, D)
        v = (h @ w[p + "v_proj.weight"].T).view(t, NKV, D)
        return q, k, v

    def ffn(i, x):
        p = f"blocks.{i}."
        h = P.rmsnorm(x, w[p + "norm2.weight"], 1e-4)
        return x + P.swiglu(h @ w[p + "ffn.gate_proj.weight"].T, h @ w[p + "ffn.up_proj.weight"].T) @ w[p + "ffn.down_proj.weight"].T

    # layer 0: windowed attention with partial rotary
    h = P.rmsnorm(x, w["blocks.0.norm1.weight"], 1e-4)
    q, k, v = qkv("blocks.0.attn.", h)
    o = P.attention(P.rope(q, pos, 100.0, 8), P.rope(k, pos, 100.0, 8), v, window=WINDOW)
    x = ffn(0, x + o.reshape(t, -1) @ w["blocks.0.attn.o_proj.weight"].T)
    # layer 1: running mean
    h = P.rmsnorm(x, w["blocks.1.norm1.weight"], 1e-4)
    mean = torch.cumsum(h, 0) / torch.arange(1, t + 1, dtype=torch.float64)[:, None]
    x = ffn(1, x + mean @ w["blocks.1.mix.weight"].T)
    # layer 2, twice; the first run's keys and values are kept for layer 3
    kept = None
    for run in range(2):
        h = P.rmsnorm(x, w["blocks.2.norm1.weight"], 1e-4)
        q, k, v = qkv("blocks.2.attn.", h)
        if run == 0:
            kept = (k, v)
        x = ffn(2, x + P.attention(q, k, v).reshape(t, -1) @ w["blocks.2.attn.o_proj.weight"].T)
    # layer 3: its own queries (rotated) on layer 2's cached keys (not rotated) and values
    h = P.rmsnorm(x, w["blocks.3.norm1.weight"], 1e-4)
    q, _, _ = qkv("blocks.3.attn.", h)
    x = ffn(3, x + P.attention(P.rope(q, pos, 100.0, 8), kept[0], kept[1]).reshape(t, -1) @ w["blocks.3.attn.o_proj.weight"].T)
    return P.rmsnorm(x, w["final_norm.weight"], 1e-4) @ w["embed.weight"].T


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_toy()
    from bare_cuda_4gib_amd.weights import write_random_model
    tmp = tmp_path_factory.mktemp("toy")
    out = {}
    for dtype in ("float32", "bfloat16"):
        folder = write_random_model(TOY_CONFIG, 9, str(tmp / dtype), dtype, std=0.08)
        requests = {f"r{i}": helpers.random_ids(n, VOCAB, 300 + i) for i, n in enumerate([3, 50, 131, 90, 64])}
        out[dtype] = (folder, requests, {r: plain_toy_logits(folder, ids).numpy() for r, ids in requests.items()})
    return out


TOL = {"float32": dict(rtol=2e-4, atol=2e-5), "bfloat16": dict(rtol=3e-2, atol=3e-2)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_whole_portions_and_mixed(toy, dtype):
    from bare_cuda_4gib_amd.cache import FixedState, PagedKV
    from bare_cuda_4gib_amd.engine import Executor, load_model
    folder, requests, plain = toy[dtype]
    model, cfg = load_model(folder, dtype)
    streams = model.cache_streams()
    assert streams["win"] == PagedKV(NKV, D, WINDOW) and streams["full-a"] == PagedKV(NKV, D, 0)
    assert streams["mean"] == FixedState((H + 1,), "float32") and set(streams) == {"win", "mean", "full-a", "full-b"}
    page = 16
    for label, (steps, where), pages in (
            ("whole", helpers.trace_whole(requests), 12),
            ("tail", helpers.trace_tail_one_by_one(requests, 32), 12),
            ("portions", helpers.trace_portions(requests, seed=8), 12)):
        ex = Executor(model, num_pages=pages, max_requests=4, max_tokens=160, page_tokens=page, poison=True)
        assert not ex.use_graphs                                      # the toy mixer is not graph-safe
        ex.cache.shuffle_free_pages(1)
        got = helpers.replay_in_process(ex, steps)
        helpers.compare_with_plain(got, where, plain, label=f"toy {label} {dtype}", **TOL[dtype])
        assert ex.cache.pages_in_use() == 0
    steps, where, peak = helpers.trace_mixed(requests, seed=2, max_live=4, page_tokens=page)
    ex = Executor(model, num_pages=peak // page, max_requests=4, max_tokens=160, page_tokens=page, poison=True)
    ex.cache.shuffle_free_pages(2)
    got = helpers.replay_in_process(ex, steps)
    helpers.compare_with_plain(got, where, plain, label=f"toy mixed {dtype}", **TOL[dtype])
    full, win = ex.cache.groups[("window", 0)].pool, ex.cache.groups[("window", WINDOW)].pool
    assert full.high_water_mark == full.num_pages                    # the pool of the full group was used up
    assert win.high_water_mark < full.high_water_mark, "the windowed group must have given pages back early"


def test_unknown_part_and_bad_schedule_are_refused(toy):
    from bare_cuda_4gib_amd.engine import Model
    from bare_cuda_4gib_amd.engine.spec import PartSpec, ScheduleEntry
    from bare_cuda_4gib_amd.config import architecture_for
    from bare_cuda_4gib_amd.errors import ConfigError
    arch = architecture_for(TOY_CONFIG)
    spec = arch.describe(arch.config_class.from_dict(TOY_CONFIG))
    spec.schedule.append(ScheduleEntry(3, "nobody-writes-this", writes=False))
    with pytest.raises(ConfigError):
        Model(spec).cache_streams()
    spec = arch.describe(arch.config_class.from_dict(TOY_CONFIG))
    spec.layers[0].ffn = PartSpec("no_such_feedforward", {})
    with pytest.raises(ConfigError) as e:
        Model(spec)
    assert "swiglu" in str(e.value)


# --- each part of a layer alone -------------------------------------------------------

def _bind(part, tensors, dtype):
    from bare_cuda_4gib_amd.engine import Runtime
    rt = Runtime(torch.device(DEV), dtype)
    part.bind({k: rt.place_weight(v) for k, v in tensors.items()}, rt)
    return part


def _ctx_for(model_like_executor, entries):
    return model_like_executor.build_context(entries)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_parts_alone(dtype):
    """Norm, feed-forward, embedding and head, each built from its sizes alone and compared with
    its plain function; attention (with rotary, cache write and block table) through a one-layer
    context is covered by the kernel tests and the toy model above."""
    from bare_cuda_4gib_amd.parts import build_part
    from bare_cuda_4gib_amd.engine.spec import PartSpec
    g = torch.Generator().manual_seed(0)
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    wdt = dtype
    x = torch.randn(70, 48, generator=g)                                  # 70 rows: beyond the skinny kernels
    xs = x[:5].contiguous()
    # norm
    nw = (1 + 0.1 * torch.randn(48, generator=g)).to(wdt)
    norm = _bind(build_part("norm", PartSpec("rmsnorm", dict(size=48, eps=1e-3))), {"weight": nw}, dtype)
    for inp in (x, xs):
        got = norm.forward(inp.to(DEV)).float().cpu()
        want = P.rmsnorm(inp.double(), nw.double(), 1e-3)
        assert torch.allclose(got.double(), want, **tol)
    # feed-forward: adds into the residual stream
    wg, wu, wd = (torch.randn(s, generator=g).mul(0.2).to(wdt) for s in ((80, 48), (80, 48), (48, 80)))
    ffn = _bind(build_part("feedforward", PartSpec("swiglu", dict(hidden_size=48, intermediate_size=80))),
                {"gate_proj.weight": wg, "up_proj.weight": wu, "down_proj.weight": wd}, dtype)
    for inp in (x, xs):
        h = inp.to(dtype)
        res = torch.ones(inp.shape[0], 48, device=DEV)
        ffn.forward(h.to(DEV), None, res)
        want = 1.0 + P.swiglu(h.double() @ wg.double().T, h.double() @ wu.double().T) @ wd.double().T
        assert torch.allclose(res.cpu().double(), want, **tol)
    # embedding and head
    table = torch.randn(61, 48, generator=g).to(wdt)
    emb = _bind(build_part("embedding", PartSpec("embedding", dict(vocab_size=61, hidden_size=48))), {"weight": table}, dtype)

    class Ids:
        token_ids = torch.tensor([3, 60, 0, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(Ids).cpu(), table.float()[[3, 60, 0, 3]])
    head = _bind(build_part("head", PartSpec("lm_head", dict(vocab_size=61, hidden_size=48))), {"weight": table}, dtype)
    hrows = x[:9].to(dtype)
    got = head.forward(hrows.to(DEV).contiguous())
    assert got.dtype == torch.float32
    assert torch.allclose(got.cpu().double(), hrows.double() @ table.double().T, **tol)


# --- a second toy: a feed-forward with routing, and another position encoding ---------------
# Both are defined here and never leave the tests.  The feed-forward picks, per token, the
# likeliest of three small experts (router logits in float32) and scales the expert's output by
# the router's softmax weight; the position encoding rotates neighbouring pairs (2i, 2i + 1) --
# a pairing the framework's fused kernels do not have, so it goes through the ``apply`` interface.
# Routing is a discontinuous choice, so this model is stepped in float32 only, and the plain
# implementation asserts that no router decision was a near-tie.

E_EXPERTS, E_INTER = 3, 40


def register_routed_toy():
    from bare_cuda_4gib_amd.config import Architecture, ModelConfig, field_from_json, register_architecture
    from bare_cuda_4gib_amd.config.registry import unregister_architecture
    from bare_cuda_4gib_amd.engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from bare_cuda_4gib_amd.parts import Part, register_part
    from bare_cuda_4gib_amd.weights import WeightSpec

    class TopOneExperts(Part):
        category = "feedforward"

        def __init__(self, hidden_size, intermediate_size, experts):
            self.h, self.i, self.e = hidden_size, intermediate_size, experts

        def weight_specs(self):
            specs = {"router.weight": WeightSpec((self.e, self.h))}
            for e in range(self.e):
                specs[f"experts.{e}.w1.weight"] = WeightSpec((self.i, self.h))
                specs[f"experts.{e}.w2.weight"] = WeightSpec((self.h, self.i))
            return specs

        def bind(self, tensors, rt):
            self.router = tensors["router.weight"].float()
            self.w1 = [tensors[f"experts.{e}.w1.weight"].float() for e in range(self.e)]
            self.w2 = [tensors[f"experts.{e}.w2.weight"].float() for e in range(self.e)]

        def forward(self, h, ctx, residual):
            h = h.float()
            logits = h @ self.router.T
            weight, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            for e in range(self.e):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    out = torch.relu(h[rows] @ self.w1[e].T) @ self.w2[e].T
                    residual[rows] += out * weight[rows, None]

    class NeighbourRotary(Part):
        category = "position"

        def __init__(self, theta):
            self.theta = float(theta)

        def fused(self):
            return None                                   # no kernel of the framework's rotates this pairing

        def apply(self, qkv, ctx, n_heads, n_kv_heads, head_dim):
            t = qkv.shape[0]
            x = qkv.view(t, n_heads + 2 * n_kv_heads, head_dim)[:, :n_heads + n_kv_heads].float()
            inv = self.theta ** (-torch.arange(0, head_dim, 2, device=qkv.device, dtype=torch.float32) / head_dim)
            ang = ctx.positions.float()[:, None] * inv
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            even, odd = x[..., 0::2], x[..., 1::2]
            rot = torch.stack([even * cos - odd * sin, odd * cos + even * sin], dim=-1).flatten(-2)
            qkv.view(t, n_heads + 2 * n_kv_heads, head_dim)[:, :n_heads + n_kv_heads] = rot.to(qkv.dtype)

    @dataclasses.dataclass
    class RoutedConfig(ModelConfig):
        vocab_size: int = field_from_json("vocab_size")
        hidden_size: int = field_from_json("hidden_size")
        experts: int = field_from_json("experts")

    def describe(cfg):
        norm = dict(size=cfg.hidden_size, eps=1e-5)
        def layer(i, position):
            p = f"blocks.{i}."
            attn = PartSpec("attention", dict(hidden_size=cfg.hidden_size, num_heads=NH, num_kv_heads=NKV, head_dim=D,
                                              window=0, position=position), prefix=p + "attn.")
            ffn = PartSpec("toy_top_one_experts", dict(hidden_size=cfg.hidden_size, intermediate_size=E_INTER,
                                                       experts=cfg.experts), prefix=p + "moe.")
            return LayerSpec("prenorm", attn, ffn, PartSpec("rmsnorm", dict(norm), prefix=p + "norm1."),
                             PartSpec("rmsnorm", dict(norm), prefix=p + "norm2."))
        layers = [layer(0, PartSpec("toy_neighbour_rotary", dict(theta=50.0))),
                  layer(1, PartSpec("rotary", dict(theta=10000.0, dim=D)))]
        return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, max_seq_len=4096,
                         embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="embed."),
                         layers=layers, schedule=[ScheduleEntry(0, "kv0"), ScheduleEntry(1, "kv1")],
                         final_norm=PartSpec("rmsnorm", dict(norm), prefix="final_norm."),
                         head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="head."))

    for category, kind, cls in (("feedforward", "toy_top_one_experts", TopOneExperts),
                                ("position", "toy_neighbour_rotary", NeighbourRotary)):
        try:
            register_part(category, kind, cls)
        except Exception:
            pass
    unregister_architecture("ToyRoutedForTests")
    register_architecture(Architecture("ToyRoutedForTests", "toy_routed_for_tests", RoutedConfig, describe))


ROUTED_CONFIG = dict(architectures=["ToyRoutedForTests"], vocab_size=VOCAB, hidden_size=H, experts=E_EXPERTS)


def plain_routed_logits(folder, ids):
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        w = {n: f.get_tensor(n).double() for n in f.keys()}
    t = len(ids)
    pos = torch.arange(t)
    x = w["embed.weight"][torch.tensor(ids)]
    smallest_margin = float("inf")
    for i in range(2):
        p = f"blocks.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], 1e-5)
        q = (h @ w[p + "attn.q_proj.weight"].T).view(t, NH, D)
        k = (h @ w[p + "attn.k_proj.weight"].T).view(t, NKV, D)
        v = (h @ w[p + "attn.v_proj.weight"].T).view(t, NKV, D)
        if i == 0:      # neighbouring pairs: the rotate-half rotation of the de-interleaved head, interleaved again
            def rot(z):
                split = torch.cat([z[..., 0::2], z[..., 1::2]], dim=-1)
                r = P.rope(split, pos, 50.0)
                return torch.stack([r[..., :D // 2], r[..., D // 2:]], dim=-1).flatten(-2)
            q, k = rot(q), rot(k)
        else:
            q, k = P.rope(q, pos, 10000.0), P.rope(k, pos, 10000.0)
        x = x + P.attention(q, k, v).reshape(t, -1) @ w[p + "attn.o_proj.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], 1e-5)
        logits = h @ w[p + "moe.router.weight"].T
        top2 = torch.topk(logits, 2, dim=-1).values
        smallest_margin = min(smallest_margin, float((top2[:, 0] - top2[:, 1]).min()))
        prob = torch.softmax(logits, dim=-1)
        choice = logits.argmax(dim=-1)
        out = torch.zeros_like(x)
        for r in range(t):
            e = int(choice[r])
            out[r] = torch.relu(h[r] @ w[p + f"moe.experts.{e}.w1.weight"].T) @ w[p + f"moe.experts.{e}.w2.weight"].T * prob[r, e]
        x = x + out
    assert smallest_margin > 1e-4, "a router decision is a near-tie: pick other seeds"
    return P.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["head.weight"].T


def test_routed_feed_forward_and_another_position_encoding(tmp_path):
    register_routed_toy()
    from bare_cuda_4gib_amd.engine import Executor, load_model
    from bare_cuda_4gib_amd.weights import write_random_model
    folder = write_random_model(ROUTED_CONFIG, 21, str(tmp_path / "routed"), "float32", std=0.1)
    requests = {f"r{i}": helpers.random_ids(n, VOCAB, 500 + i) for i, n in enumerate([4, 37, 90, 65])}
    plain = {r: plain_routed_logits(folder, ids).numpy() for r, ids in requests.items()}
    model, _ = load_model(folder, "float32")
    page = 16
    steps, where, peak = helpers.trace_mixed(requests, seed=4, max_live=3, page_tokens=page)
    for label, (st, wh), pages in (("whole", helpers.trace_whole(requests), 16),
                                   ("portions", helpers.trace_portions(requests, seed=3), 16),
                                   ("mixed", (steps, where), peak // page)):
        ex = Executor(model, num_pages=pages, max_requests=4, max_tokens=96, page_tokens=page, poison=True)
        assert not ex.use_graphs                                      # the toy parts are not graph-safe
        got = helpers.replay_in_process(ex, st)
        helpers.compare_with_plain(got, wh, plain, label=f"routed toy {label}", rtol=2e-4, atol=2e-5)
        assert ex.cache.pages_in_use() == 0


# --- a third toy: a mixer with a cache layout and a launch geometry of its own, inside captured graphs ---
# Defined here and never leaving the tests.  It keeps, per token, the vector it was given (a cache spec
# of its own: one float tensor per page, no keys or values) and gives every row the mean of its
# request's vectors so far, times a matrix.  It walks the cache in chunks of 64 positions, as many as
# the longest context needs -- a launch geometry of its own, which a captured step has to fix for the
# graph's whole context bucket -- and it divides by counts that the host works out for every step and
# sends up with the batch.  All of it through the part hooks; nothing under engine/ or cache/ knows it.

G_CHUNK = 64


def register_geometry_toy():
    from bare_cuda_4gib_amd.config import Architecture, ModelConfig, field_from_json, register_architecture
    from bare_cuda_4gib_amd.config.registry import unregister_architecture
    from bare_cuda_4gib_amd.engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from bare_cuda_4gib_amd.parts import Part, register_part
    from bare_cuda_4gib_amd.weights import WeightSpec

    @dataclasses.dataclass(frozen=True)
    class PagedVectors:
        """One float vector per token, in pages: a cache spec the framework has never heard of."""
        width: int
        window: int = 0
        per_token = True

        def page_tensors(self, page_tokens):
            return {"h": ((page_tokens, self.width), "float32")}

    class CausalMean(Part):
        category = "mixer"
        graph_safe = True                 # torch kernels on the current stream only, nothing read back
        calls = {"forward": 0, "prepare_step": 0, "prepare_capture": []}

        def __init__(self, hidden_size):
            self.hidden = hidden_size
            self.frozen_chunks = {}

        def cache_spec(self):
            return PagedVectors(self.hidden)

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.hidden, self.hidden))}

        def bind(self, tensors, rt):
            self.w = tensors["mix.weight"].float()

        def prepare_step(self, batch):
            CausalMean.calls["prepare_step"] += 1
            counts = []
            for s in range(batch.n_seqs):
                n = int(batch.seq_start[s + 1] - batch.seq_start[s])
                counts.extend(range(int(batch.seq_ctx[s]) + 1, int(batch.seq_ctx[s]) + n + 1))
            return {"counts": counts}, dict(chunks=-(-batch.max_kv_len // G_CHUNK))

        def prepare_capture(self, n_seqs, max_context):
            CausalMean.calls["prepare_capture"].append((n_seqs, max_context))
            self.frozen_chunks[n_seqs] = -(-max_context // G_CHUNK)

        def forward(self, h, ctx, cache, residual, writes=True):
            CausalMean.calls["forward"] += 1
            arrays, notes = ctx.step_data[id(self)]
            chunks = notes["chunks"]
            if ctx.captured:                                    # the geometry fixed for the bucket, not this step's
                assert chunks == self.frozen_chunks[ctx.n_seqs] == -(-ctx.max_kv_len // G_CHUNK)
            P_, H_ = cache.page_tokens, self.hidden
            store = cache.h.view(-1, H_)
            if writes:
                store[ctx.slot_maps[cache.group].long()] = h.float()
            table = ctx.block_tables[cache.group][ctx.row_seq.long()].long()           # [T, pages]
            positions = ctx.positions.long()
            total = torch.zeros(ctx.n_tokens, H_, device=h.device)
            for c in range(chunks):
                pos = c * G_CHUNK + torch.arange(G_CHUNK, device=h.device)
                seen = pos[None, :] <= positions[:, None]                                # [T, chunk]
                page = torch.gather(table, 1, (pos // P_).clamp(max=table.shape[1] - 1)[None, :].expand(ctx.n_tokens, -1))
                index = torch.where(seen, page * P_ + pos % P_, torch.zeros_like(page))
                rows = store[index.clamp(min=0)]                                         # [T, chunk, H]
                total += torch.where(seen[:, :, None], rows, torch.zeros_like(rows)).sum(dim=1)
            mean = total / arrays["counts"].float()[:, None]
            residual += mean @ self.w.T

    @dataclasses.dataclass
    class GeometryConfig(ModelConfig):
        vocab_size: int = field_from_json("vocab_size")
        hidden_size: int = field_from_json("hidden_size")

    def describe(cfg):
        norm = dict(size=cfg.hidden_size, eps=1e-5)
        def layer(i, mixer):
            p = f"blocks.{i}."
            return LayerSpec("prenorm", mixer, PartSpec("swiglu", dict(hidden_size=cfg.hidden_size, intermediate_size=INTER),
                                                        prefix=p + "ffn."),
                             PartSpec("rmsnorm", dict(norm), prefix=p + "norm1."), PartSpec("rmsnorm", dict(norm), prefix=p + "norm2."))
        layers = [layer(0, PartSpec("toy_causal_mean", dict(hidden_size=cfg.hidden_size), prefix="blocks.0.")),
                  layer(1, PartSpec("attention", dict(hidden_size=cfg.hidden_size, num_heads=NH, num_kv_heads=NKV, head_dim=D,
                                                      window=0, position=PartSpec("rotary", dict(theta=1000.0, dim=D))),
                                    prefix="blocks.1.attn."))]
        return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, max_seq_len=4096,
                         embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="embed."),
                         layers=layers, schedule=[ScheduleEntry(0, "vectors"), ScheduleEntry(1, "kv")],
                         final_norm=PartSpec("rmsnorm", dict(norm), prefix="final_norm."),
                         head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="head."))

    register_part("mixer", "toy_causal_mean", CausalMean, replace=True)
    unregister_architecture("ToyGeometryForTests")
    register_architecture(Architecture("ToyGeometryForTests", "toy_geometry_for_tests", GeometryConfig, describe))
    return CausalMean


GEOMETRY_CONFIG = dict(architectures=["ToyGeometryForTests"], vocab_size=VOCAB, hidden_size=H)


def plain_geometry_logits(folder, ids):
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        w = {n: f.get_tensor(n).double() for n in f.keys()}
    t = len(ids)
    pos = torch.arange(t)
    x = w["embed.weight"][torch.tensor(ids)]

    def ffn(i, x):
        p = f"blocks.{i}."
        h = P.rmsnorm(x, w[p + "norm2.weight"], 1e-5)
        return x + P.swiglu(h @ w[p + "ffn.gate_proj.weight"].T, h @ w[p + "ffn.up_proj.weight"].T) @ w[p + "ffn.down_proj.weight"].T
    h = P.rmsnorm(x, w["blocks.0.norm1.weight"], 1e-5)
    mean = torch.cumsum(h, 0) / torch.arange(1, t + 1, dtype=torch.float64)[:, None]
    x = ffn(0, x + mean @ w["blocks.0.mix.weight"].T)
    h = P.rmsnorm(x, w["blocks.1.norm1.weight"], 1e-5)
    q = (h @ w["blocks.1.attn.q_proj.weight"].T).view(t, NH, D)
    k = (h @ w["blocks.1.attn.k_proj.weight"].T).view(t, NKV, D)
    v = (h @ w["blocks.1.attn.v_proj.weight"].T).view(t, NKV, D)
    o = P.attention(P.rope(q, pos, 1000.0), P.rope(k, pos, 1000.0), v)
    x = ffn(1, x + o.reshape(t, -1) @ w["blocks.1.attn.o_proj.weight"].T)
    return P.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_its_own_cache_layout_and_step_geometry_runs_in_captured_graphs(tmp_path, dtype):
    CausalMean = register_geometry_toy()
    from bare_cuda_4gib_amd.cache import bytes_per_page
    from bare_cuda_4gib_amd.engine import Executor, StepEntry, load_model
    from bare_cuda_4gib_amd.weights import write_random_model
    folder = write_random_model(GEOMETRY_CONFIG, 33, str(tmp_path / "geometry"), dtype, std=0.08, norm_std=0.1)
    requests = {f"r{i}": helpers.random_ids(n, VOCAB, 700 + i) for i, n in enumerate([270, 90, 41])}
    plain = {r: plain_geometry_logits(folder, ids).numpy() for r, ids in requests.items()}
    model, _ = load_model(folder, dtype)
    page = 16
    streams = model.cache_streams()
    elem = 4 if dtype == "float32" else 2
    assert bytes_per_page(streams.values(), page, model.rt.act_dtype) == page * H * 4 + 2 * NKV * D * page * elem
    tol = TOL[dtype]
    # whole, portions, and mixed with few pages: the general path
    steps_m, where_m, peak = helpers.trace_mixed(requests, seed=3, max_live=3, page_tokens=page)
    for label, (steps, where), pages in (("whole", helpers.trace_whole(requests), 20),
                                         ("portions", helpers.trace_portions(requests, seed=2), 20),
                                         ("mixed", (steps_m, where_m), peak // page)):
        ex = Executor(model, num_pages=pages, max_requests=3, max_tokens=304, page_tokens=page, poison=True)
        assert ex.use_graphs                                          # every part here says it may be captured
        ex.cache.shuffle_free_pages(6)
        got = helpers.replay_in_process(ex, steps)
        helpers.compare_with_plain(got, where, plain, label=f"geometry toy {label} {dtype}", **tol)
    # decoding: three requests' last tokens one by one, all three in every step -- replayed from graphs
    ex = Executor(model, num_pages=40, max_requests=3, max_tokens=304, page_tokens=page, poison=True)
    ex.cache.shuffle_free_pages(8)
    tail = 30
    for r, ids in requests.items():
        ex.admit(r)
        ex.step([StepEntry(r, ids[:-tail], [])])
    before = dict(CausalMean.calls, prepare_capture=list(CausalMean.calls["prepare_capture"]))
    for i in range(tail):
        rows = ex.step([StepEntry(r, [ids[len(ids) - tail + i]], [0]) for r, ids in requests.items()]).float().cpu().numpy()
        for row, (r, ids) in zip(rows, requests.items()):
            want = plain[r][len(ids) - tail + i]
            assert np.all(np.abs(row - want) <= tol["atol"] + tol["rtol"] * np.abs(want)), f"decode step {i}, request {r}"
    # the longest request crosses from the 256-token bucket into the 512-token one: two graphs, each captured once
    # after the hook was told its request count and context bound; forward ran for the captures only (twice each),
    # the step preparation for every step
    assert sorted(ex._graphs) == [(3, 256), (3, 512)]
    assert CausalMean.calls["prepare_capture"][len(before["prepare_capture"]):] == [(3, 256), (3, 512)]
    assert CausalMean.calls["forward"] - before["forward"] == 4
    assert CausalMean.calls["prepare_step"] - before["prepare_step"] >= tail


# --- through the scheduler: a model whose every stream has a window, and one that keeps nothing per token ---
# The scheduler asks the cache manager what a request may need at most (by each stream's own rule), not how
# long the request is: the first toy runs requests much longer than its pool, the second with no pages at all.

def register_stack_toy():
    register_toy()                       # (the running-mean mixer)
    from bare_cuda_4gib_amd.config import Architecture, ModelConfig, field_from_json, register_architecture
    from bare_cuda_4gib_amd.config.registry import unregister_architecture
    from bare_cuda_4gib_amd.engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    @dataclasses.dataclass
    class StackConfig(ModelConfig):
        vocab_size: int = field_from_json("vocab_size")
        hidden_size: int = field_from_json("hidden_size")
        kinds: str = field_from_json("kinds")          # one letter a layer: w = windowed attention, m = running mean
        window: int = field_from_json("window")

    def describe(cfg):
        norm = dict(size=cfg.hidden_size, eps=1e-5)
        layers = []
        for i, kind in enumerate(cfg.kinds):
            p = f"blocks.{i}."
            if kind == "w":
                mixer = PartSpec("attention", dict(hidden_size=cfg.hidden_size, num_heads=NH, num_kv_heads=NKV, head_dim=D,
                                                   window=cfg.window, position=PartSpec("rotary", dict(theta=100.0, dim=D))),
                                 prefix=p + "attn.")
            else:
                mixer = PartSpec("toy_running_mean", dict(hidden_size=cfg.hidden_size), prefix=p)
            layers.append(LayerSpec("prenorm", mixer, PartSpec("swiglu", dict(hidden_size=cfg.hidden_size, intermediate_size=INTER),
                                                               prefix=p + "ffn."),
                                    PartSpec("rmsnorm", dict(norm), prefix=p + "norm1."), PartSpec("rmsnorm", dict(norm), prefix=p + "norm2.")))
        return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, max_seq_len=4096,
                         embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="embed."),
                         layers=layers, schedule=[ScheduleEntry(i, f"c{i}") for i in range(len(layers))],
                         final_norm=PartSpec("rmsnorm", dict(norm), prefix="final_norm."),
                         head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size), prefix="head."))

    unregister_architecture("ToyStackForTests")
    register_architecture(Architecture("ToyStackForTests", "toy_stack_for_tests", StackConfig, describe))


def plain_stack_logits(folder, ids, kinds, window):
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        w = {n: f.get_tensor(n).double() for n in f.keys()}
    t = len(ids)
    pos = torch.arange(t)
    x = w["embed.weight"][torch.tensor(ids)]
    for i, kind in enumerate(kinds):
        p = f"blocks.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], 1e-5)
        if kind == "w":
            q = (h @ w[p + "attn.q_proj.weight"].T).view(t, NH, D)
            k = (h @ w[p + "attn.k_proj.weight"].T).view(t, NKV, D)
            v = (h @ w[p + "attn.v_proj.weight"].T).view(t, NKV, D)
            o = P.attention(P.rope(q, pos, 100.0), P.rope(k, pos, 100.0), v, window=window)
            x = x + o.reshape(t, -1) @ w[p + "attn.o_proj.weight"].T
        else:
            mean = torch.cumsum(h, 0) / torch.arange(1, t + 1, dtype=torch.float64)[:, None]
            x = x + mean @ w[p + "mix.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], 1e-5)
        x = x + P.swiglu(h @ w[p + "ffn.gate_proj.weight"].T, h @ w[p + "ffn.up_proj.weight"].T) @ w[p + "ffn.down_proj.weight"].T
    return P.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["head.weight"].T


@pytest.mark.parametrize("kinds,pages", [("ww", 8), ("mm", 0)])
def test_the_scheduler_asks_the_cache_what_a_request_needs(tmp_path, kinds, pages):
    """Requests of 40 to 150 tokens plus 12 generated, in portions of 32, with three live at a time.  The windowed
    model (window 24, pages of 16) holds at most five pages a request and runs in a pool of eight, fewer than the
    eleven that the longest request's tokens alone would take; the model of running means has no pages.  Greedy tokens against the plain
    implementation of the same toy, followed along the engine's own tokens."""
    register_stack_toy()
    from bare_cuda_4gib_amd.engine import Executor, load_model
    from bare_cuda_4gib_amd.engine.scheduler import Request, Scheduler
    from bare_cuda_4gib_amd.sampling.device import DevicePicker
    from bare_cuda_4gib_amd.weights import write_random_model
    config = dict(architectures=["ToyStackForTests"], vocab_size=VOCAB, hidden_size=H, kinds=kinds, window=WINDOW)
    folder = write_random_model(config, 33, str(tmp_path / kinds), "float32", std=0.08)
    model, _ = load_model(folder, "float32")
    ex = Executor(model, num_pages=pages, max_requests=3, max_tokens=176, page_tokens=16, poison=True)
    sched = Scheduler(ex, DevicePicker(), max_batch_tokens=64, prefill_chunk=32)
    if kinds == "ww":
        assert ex.cache.peak_pages(161, 32) == {("window", WINDOW): 5} and sched.limits.kv_pages == 8
    else:
        assert ex.cache.groups == {} and sched.limits.kv_pages == 0
    prompts = {i: helpers.random_ids(n, VOCAB, 700 + i) for i, n in enumerate([150, 40, 97, 64, 121])}
    for i, ids in prompts.items():
        assert sched.check(Request(id=i, prompt=ids, max_new_tokens=12)) == ""
        sched.submit(Request(id=i, prompt=ids, max_new_tokens=12))
    out = {i: [] for i in prompts}
    for _ in range(400):
        if sched.idle():
            break
        for e in sched.step():
            if e.token >= 0:
                out[e.id].append(e.token)
    assert sched.idle() and ex.cache.pages_in_use() == 0 and ex.cache.free_slots == 3
    assert sched.stats().prefill_tokens >= sum(len(ids) for ids in prompts.values())
    for i, ids in prompts.items():
        assert len(out[i]) == 12
        full = plain_stack_logits(folder, ids + out[i], kinds, WINDOW)
        for j, tok in enumerate(out[i]):
            row = full[len(ids) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-4, f"request {i}, token {j}: {tok} is not the plain best {int(row.argmax())}"
