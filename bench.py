"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--dtype bf16]

The default run has the layer sizes of TinyLlama-1.1B (22 layers, hidden 2048, 32 query heads /
4 key-value heads, head size 64, feed-forward 5632, vocabulary 32000, context 2048) with random
weights, a batch of 8 requests with 512-token prompts, and times K decode steps (each step: one
token for every request through the engine's step function, greedy choice on the device, the
chosen ids read back while the next step runs).  It prints ONE JSON line: decoded tokens a second, the prefill of one
2,048-token prompt, the decode step against the HBM roofline, and decoding at batch 1 and 64.

The prefill figure is the best of three runs, the decode figure the mean of K steps; both are also stated
against what this device was measured to deliver (`--only peaks`: a kernel that only reads; nothing but
matrix-core instructions, on normally distributed operands like the benchmark's -- the chip's clock follows the
power that toggling operands draw -- and on ones).

Beside the headline: `--shape` runs the same measurements at the sizes of Llama-2-7B or Llama-3-8B;
`--only decode|prefill` runs one part and prints a short line of its own (what the profiles use);
`--only serve` submits `--requests` requests of mixed lengths to the scheduler and times the whole
run, prompts in portions of `--chunk` tokens beside the others' decoded tokens (`--new-tokens-spread`:
the requests end one after the other instead of all together; `--top-k`, `--top-p`: they sample with these).
`--only chat` is a closed loop of `--requests` requests with short prompts and long answers that come and go all the
time (`--gather-ms`: the scheduler gathers those who came for so long before it admits them).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                       # MI355X: 8 TB/s
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
TINYLLAMA = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=32000, hidden_size=2048,
                 num_hidden_layers=22, num_attention_heads=32, num_key_value_heads=4, head_dim=64,
                 intermediate_size=5632, rope_theta=10000.0, rms_norm_eps=1e-5,
                 max_position_embeddings=2048, tie_word_embeddings=False)
# Other shapes of the same architecture, for measurements beside the headline (--shape).
SHAPES = {
    "tinyllama-1.1b": TINYLLAMA,
    "llama-2-7b": dict(TINYLLAMA, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
                       num_key_value_heads=32, head_dim=128, intermediate_size=11008, max_position_embeddings=4096),
    "llama-3-8b": dict(TINYLLAMA, vocab_size=128256, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
                       num_key_value_heads=8, head_dim=128, intermediate_size=14336, rope_theta=500000.0,
                       max_position_embeddings=8192),
}
BASELINE_DECODE_B1 = 77.3                   # the reference's only FP16 decode number (batch 1, RTX 3050)


def build_model(layers, dtype, seed=0, shape=TINYLLAMA):
    import torch
    from bare_cuda_4gib_amd.config import architecture_for
    from bare_cuda_4gib_amd.engine import Model, Runtime, parse_dtype
    from bare_cuda_4gib_amd.weights.random_device import random_tensors_on_device
    raw = dict(shape, num_hidden_layers=layers)
    arch = architecture_for(raw)
    cfg = arch.config_class.from_dict(raw)
    model = Model(arch.describe(cfg))
    tdtype = parse_dtype(dtype)
    tensors = random_tensors_on_device(model.expected_weights(), seed, tdtype, "cuda:0")
    model.bind(tensors, Runtime(torch.device("cuda:0"), tdtype))
    return model, cfg


def decode_bytes(model, elem, contexts):
    """Bytes one decode step has to read: every weight it uses once (linear maps, norms, the
    embedding rows of the batch) and the cached keys and values of the live requests -- as the model's
    parts state them (Model.step_work), so another architecture's bytes need no formula here."""
    from bare_cuda_4gib_amd.engine.batch import HostBatch
    n = len(contexts)
    batch = HostBatch(n_tokens=n, n_seqs=n, seq_start=list(range(n + 1)), seq_ctx=[c - 1 for c in contexts],
                      seq_slots=list(range(n)), max_q_len=1, max_kv_len=max(contexts))
    return model.step_work(batch, n, elem)[1]


def prefill_flops(model, t):
    """Operations of one prompt of t tokens with logits at its last place only (Model.step_work)."""
    from bare_cuda_4gib_amd.engine.batch import HostBatch
    batch = HostBatch(n_tokens=t, n_seqs=1, seq_start=[0, t], seq_ctx=[0], seq_slots=[0], max_q_len=t, max_kv_len=t)
    return model.step_work(batch, 1, 2)[0]


def run_decode(model, cfg, batch, prompt_len, steps, warmup, seed=1):
    """(seconds for `steps` decode steps, context lengths at the middle of the timed region)."""
    import torch
    from bare_cuda_4gib_amd.csrc import ops
    from bare_cuda_4gib_amd.engine import Executor, StepEntry
    total = prompt_len + warmup + steps + 1
    page = 64
    pages_each = -(-total // page)
    ex = Executor(model, num_pages=pages_each * batch, max_requests=batch, max_tokens=pages_each * page,
                  page_tokens=page)
    gen = torch.Generator().manual_seed(seed)
    last = []
    for b in range(batch):
        ex.admit(b)
        prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=gen).tolist()
        logits = ex.step([StepEntry(b, prompt, [prompt_len - 1])])
        last.append(int(ops.argmax(logits)[0]))

    # Every step's tokens are the ids the step before chose, taken on the device; the host reads a
    # step's ids (through pinned memory) while the next step runs, so describing a step to the
    # device costs the GPU no time.
    entries = [StepEntry(b, [0], [0]) for b in range(batch)]
    stage = [torch.empty(batch, dtype=torch.int32).pin_memory() for _ in range(2)]
    copied = [torch.cuda.Event() for _ in range(2)]
    read = []

    def launch(ids, i):
        chosen = ops.argmax(ex.step(entries, device_tokens=ids))
        stage[i % 2].copy_(chosen, non_blocking=True)
        copied[i % 2].record()
        return chosen

    def run(n, ids):
        for i in range(n):
            ids = launch(ids, i)
            if i > 0:                                    # the ids of the step before, now that this one is under way
                copied[(i - 1) % 2].synchronize()
                read.append(stage[(i - 1) % 2].tolist())
        copied[(n - 1) % 2].synchronize()
        read.append(stage[(n - 1) % 2].tolist())
        return ids

    ids = run(warmup, torch.tensor(last, dtype=torch.int32, device="cuda:0"))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ids = run(steps, ids)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(read) == warmup + steps and all(len(r) == batch for r in read)
    mid = prompt_len + warmup + steps // 2
    for b in range(batch):
        ex.release(b)
    del ex
    torch.cuda.empty_cache()
    return dt, [mid] * batch


def run_prefill(model, cfg, tokens, runs=3, seed=2):
    import torch
    from bare_cuda_4gib_amd.engine import Executor, StepEntry
    page = 64
    ex = Executor(model, num_pages=-(-tokens // page), max_requests=1, max_tokens=-(-tokens // page) * page,
                  page_tokens=page)
    gen = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=gen).tolist()
    best = float("inf")
    for i in range(runs + 1):
        ex.admit("p")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ex.step([StepEntry("p", prompt, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ex.release("p")
        if i > 0:
            best = min(best, dt)
    del ex
    torch.cuda.empty_cache()
    return best


def run_gemm(m, n, k, runs=20):
    """One product of the linear maps' kernels alone (operands drawn as the model's are)."""
    import torch
    from bare_cuda_4gib_amd.csrc import ops
    gen = torch.Generator(device="cuda").manual_seed(4)
    a = torch.randn(m, k, device="cuda", generator=gen).bfloat16()
    w = ops.StreamedWeight((torch.randn(n, k, device="cuda", generator=gen) * 0.02).bfloat16())   # as a model holds it
    for _ in range(3):
        ops.gemm_fast(a, w, torch.bfloat16)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(runs):
        ops.gemm_fast(a, w, torch.bfloat16)
    end.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(end) / runs * 1e3
    return {"only": "gemm", "m": m, "n": n, "k": k, "us": round(us, 1), "tflops": round(2.0 * m * n * k / us / 1e6, 1),
            "frac": round(2.0 * m * n * k / us / 1e6 / PEAK_TFLOPS["bf16"], 4)}


def run_serve(model, cfg, n_requests, new_tokens, chunk, seed=3, spread=0, top_k=0, top_p=1.0):
    """A mixed batch through the scheduler: n_requests submitted at once, prompt lengths uniform in
    [128, max context - new_tokens], prompts cut into portions of `chunk` tokens beside the decoded
    tokens of the others, temperature 1.0 (with ``top_k`` / ``top_p`` if given).  ``spread``: the requests' numbers of new tokens are spaced
    evenly from new_tokens down to new_tokens - spread, so that they end one after the other and the
    number of decoding requests takes every value on its way down (0: all generate new_tokens and end
    together).  Returns (seconds, scheduler statistics with the decode graphs captured in the timed run)."""
    import torch
    from bare_cuda_4gib_amd.engine import Executor
    from bare_cuda_4gib_amd.engine.scheduler import Request, Scheduler
    from bare_cuda_4gib_amd.sampling.device import DevicePicker
    from bare_cuda_4gib_amd.sampling.params import SamplingParams
    page = 64
    longest = min(cfg.max_seq_len - new_tokens, 4096)
    gen = torch.Generator().manual_seed(seed)
    lengths = torch.randint(128, longest + 1, (n_requests,), generator=gen).tolist()
    pages = sum(-(-(n + new_tokens) // page) for n in lengths)
    ex = Executor(model, num_pages=pages, max_requests=n_requests, max_tokens=cfg.max_seq_len, page_tokens=page,
                  max_batch_tokens=2048)
    sched = Scheduler(ex, DevicePicker(), max_batch_tokens=2048, prefill_chunk=chunk, run_ahead=True)   # as Engine does

    spread = max(0, min(spread, new_tokens - 1))
    new = [new_tokens - (i * spread) // max(1, n_requests - 1) for i in range(n_requests)]

    def submit_all(tag):
        for i, n in enumerate(lengths):
            prompt = torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
            sched.submit(Request(id=tag * n_requests + i, prompt=prompt, max_new_tokens=new[i],
                                 sampling=SamplingParams(temperature=1.0, top_p=top_p, top_k=top_k, seed=i)))

    def drain():
        made = 0
        while not sched.idle():
            made += sum(1 for e in sched.step() if e.token >= 0)
        return made

    submit_all(0)                     # once untimed: graphs are captured, buffers made
    drain()
    before, captured = sched.stats(), ex.captures
    submit_all(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    made = drain()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    after = sched.stats()
    return dt, dict(requests=n_requests, generated=made, prompt_tokens=sum(lengths), new_tokens_spread=spread,
                    top_k=top_k, top_p=top_p,
                    steps=after.steps - before.steps, preemptions=after.preemptions - before.preemptions,
                    graphs=len(ex._graphs), graphs_captured_in_the_timed_run=ex.captures - captured)


def run_chat(model, cfg, concurrency, gather_ms, finished=384, seed=5):
    """Requests that come and go all the time: `concurrency` requests in flight, each with a prompt of 16 to 64
    tokens and 64 to 192 new ones at temperature 1.0; whenever one ends the next is submitted (a closed loop), so
    that new prompts arrive every few steps beside the others' decoded tokens.  ``gather_ms``: the scheduler's
    wait before it admits those who came (Scheduler(gather_ms=...)).  Times the steps in which `finished` requests
    end, after as many to warm up.  Returns (seconds, figures)."""
    import random
    import torch
    from bare_cuda_4gib_amd.engine import Executor
    from bare_cuda_4gib_amd.engine.scheduler import Request, Scheduler
    from bare_cuda_4gib_amd.sampling.device import DevicePicker
    from bare_cuda_4gib_amd.sampling.params import SamplingParams
    ex = Executor(model, num_pages=concurrency * 4, max_requests=concurrency, max_tokens=256, page_tokens=64,
                  max_batch_tokens=2048)
    sched = Scheduler(ex, DevicePicker(), max_batch_tokens=2048, prefill_chunk=512, run_ahead=True, gather_ms=gather_ms)
    rnd = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    ids = iter(range(1 << 30))

    def arrive():
        n = rnd.randint(16, 64)
        i = next(ids)
        sched.submit(Request(id=i, prompt=torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist(),
                             max_new_tokens=rnd.randint(64, 192), sampling=SamplingParams(temperature=1.0, seed=i)))

    def run(until):
        made = ended = 0
        while ended < until:
            for e in sched.step():
                made += e.token >= 0
                if e.finish:
                    ended += 1
                    arrive()
        return made

    for _ in range(concurrency):
        arrive()
    run(finished)
    torch.cuda.synchronize()
    before = sched.stats()
    t0 = time.perf_counter()
    made = run(finished)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    after = sched.stats()
    steps = after.steps - before.steps
    return dt, dict(concurrency=concurrency, gather_ms=gather_ms, requests_ended=finished, generated=made, steps=steps,
                    ms_per_step=round(dt / steps * 1e3, 3), preemptions=after.preemptions - before.preemptions)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="tinyllama-1.1b",
                    help="layer sizes; the headline is measured on the default")
    ap.add_argument("--layers", type=int, default=None, help="fewer than the shape has only where time needs it")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip decoding at batch 1 and 64")
    ap.add_argument("--requests", type=int, default=64, help="--only serve: requests submitted at once")
    ap.add_argument("--new-tokens", type=int, default=256, help="--only serve: tokens generated per request")
    ap.add_argument("--chunk", type=int, default=512, help="--only serve: prompt portion size")
    ap.add_argument("--new-tokens-spread", type=int, default=0,
                    help="--only serve: the requests generate from --new-tokens down to --new-tokens minus this, evenly "
                         "spaced, so they end one after the other (0: all end together)")
    ap.add_argument("--top-k", type=int, default=0, help="--only serve: the requests sample with this top-k (0: none)")
    ap.add_argument("--top-p", type=float, default=1.0, help="--only serve: ... and this top-p (1: none)")
    ap.add_argument("--gather-ms", type=float, default=0.0,
                    help="--only chat: the scheduler waits this long before it admits those who came while others decode")
    ap.add_argument("--only", choices=["decode", "prefill", "serve", "chat", "gemm", "peaks"], default=None,
                    help="run one part only and print its own short line (for profiling); peaks: what a kernel that only "
                         "reads, and one of nothing but matrix-core instructions, reach on this device")
    ap.add_argument("--mnk", default="2048,11264,2048",
                    help="--only gemm: rows, outputs and k of one bfloat16 product x w^T (the tiled matrix-core kernel)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from bare_cuda_4gib_amd.csrc import library
    library.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.only == "gemm":
        print(json.dumps(run_gemm(*(int(v) for v in args.mnk.split(",")))), flush=True)
        return 0
    from bare_cuda_4gib_amd.csrc.peaks import measured_peaks
    measured = measured_peaks()
    if args.only == "peaks":
        print(json.dumps({"only": "peaks", "hbm_gbs": measured["hbm_gbs"], "hbm_frac_of_published": round(measured["hbm_gbs"] / HBM_PEAK_GBS, 4),
                          "bf16_tflops": measured["bf16_tflops"], "bf16_tflops_ones": measured["bf16_tflops_ones"],
                          "bf16_frac_of_published": round(measured["bf16_tflops"] / PEAK_TFLOPS["bf16"], 4)}), flush=True)
        return 0
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    elem = 2 if args.dtype == "bf16" else 4
    shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    model, cfg = build_model(args.layers, dtype, shape=shape)

    if args.only == "decode":
        dt, contexts = run_decode(model, cfg, args.batch, args.prompt_len, args.steps, args.warmup)
        gbs = decode_bytes(model, elem, contexts) / (dt / args.steps) / 1e9
        print(json.dumps({"only": "decode", "shape": args.shape, "batch": args.batch, "context": contexts[0],
                          "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "hbm_frac_of_measured": round(gbs / measured["hbm_gbs"], 4),
                          "ms_per_step": round(dt / args.steps * 1e3, 4),
                          "tokens_per_s": round(args.batch * args.steps / dt, 1)}), flush=True)
        return 0
    if args.only == "prefill":
        pre_s = run_prefill(model, cfg, args.prefill_tokens)
        frac = prefill_flops(model, args.prefill_tokens) / pre_s / (PEAK_TFLOPS[args.dtype] * 1e12)
        print(json.dumps({"only": "prefill", "shape": args.shape, "tokens": args.prefill_tokens, "of": "best of 3",
                          "ms": round(pre_s * 1e3, 3), "frac": round(frac, 4),
                          "frac_of_measured": round(frac * PEAK_TFLOPS[args.dtype] / measured["bf16_tflops"], 4) if args.dtype == "bf16" else None,
                          "tokens_per_s": round(args.prefill_tokens / pre_s, 1)}), flush=True)
        return 0

    if args.only == "chat":
        dt, st = run_chat(model, cfg, args.requests, args.gather_ms, finished=6 * args.requests)
        print(json.dumps(dict(only="chat", shape=args.shape, **st, seconds=round(dt, 3),
                              generated_per_s=round(st["generated"] / dt, 1))), flush=True)
        return 0

    if args.only == "serve":
        dt, st = run_serve(model, cfg, args.requests, args.new_tokens, args.chunk, spread=args.new_tokens_spread,
                           top_k=args.top_k, top_p=args.top_p)
        print(json.dumps(dict(only="serve", shape=args.shape, **st, seconds=round(dt, 3),
                              generated_per_s=round(st["generated"] / dt, 1),
                              all_tokens_per_s=round((st["generated"] + st["prompt_tokens"]) / dt, 1))), flush=True)
        return 0

    dt, contexts = run_decode(model, cfg, args.batch, args.prompt_len, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = decode_bytes(model, elem, contexts) / (dt / args.steps) / 1e9

    pre_s = run_prefill(model, cfg, args.prefill_tokens)
    pre_frac = prefill_flops(model, args.prefill_tokens) / pre_s / (PEAK_TFLOPS[args.dtype] * 1e12)

    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps_b = max(16, args.steps // 2)
            dtb, _ = run_decode(model, cfg, b, args.prompt_len, steps_b, max(4, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * steps_b / dtb, 1)

    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(points.get("decode_b1", 0.0) / BASELINE_DECODE_B1, 2) if points else None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {"model": "TinyLlama-1.1B shape" if args.shape == "tinyllama-1.1b" else args.shape + " shape",
                   "layers": args.layers, "layers_full": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "global_batch": args.batch, "seq_len": cfg.max_seq_len, "prompt_len": args.prompt_len,
                   "page_tokens": 64, "parallelism": "single GPU",
                   "vs_baseline_is": "decode_b1 / 77.3 tok/s (reference, FP16, batch 1, RTX 3050)"},
        "prefill": {"value": round(args.prefill_tokens / pre_s, 1), "tokens": args.prefill_tokens,
                    "ms": round(pre_s * 1e3, 3), "frac": round(pre_frac, 4), "of": "best of 3",
                    "frac_of_measured": round(pre_frac * PEAK_TFLOPS[args.dtype] / measured["bf16_tflops"], 4) if args.dtype == "bf16" else None,
                    "measured_peak_tflops": measured["bf16_tflops"], "measured_peak_tflops_ones": measured["bf16_tflops_ones"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "measured_peak": measured["hbm_gbs"],
                     "frac_of_measured": round(achieved / measured["hbm_gbs"], 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
