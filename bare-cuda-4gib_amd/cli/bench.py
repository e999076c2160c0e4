"""``llm-bench``: latency and throughput of requests through the engine, with the options of the
reference's program of the same name (bench/src/bench_main.cc:63-78): ``--model (--prompt
id,id,... | --prompt-len N) [--tokens N] [--runs N] [--warmup N] [--batch N] [--kernels]``.

A request is one prompt, or with ``--batch N`` N copies of it decoded together, through the Python
entry point (the scheduler included).  Every token's arrival at the host is stamped; from the stamps:
TTFT, the gaps between tokens (TPOT: all, each sequence's first and last), E2E, decode tokens/s
``(tokens - 1) / (E2E - TTFT)``, and for a batch ``N (tokens - 1) / (last token - last first
token)`` (bench_main.cc:141-176, 366-374), each as mean, nearest-rank p50/p90/p99, min and max
(:108-125).  ``--kernels`` adds a per-kernel table of one more request, run with the profiler on
and without captured graphs: calls, device time, and the stated work against the peaks of the
MI355X (:208-254).  Added here: ``--dtype``, ``--page-tokens``, and ``--random-weights CONFIG_JSON``
to write the model folder first."""
from __future__ import annotations

import argparse
import math
import sys
import time
from typing import Dict, List, Sequence

from .infer import parse_ids

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}


def synthetic_prompt(length: int, vocab: int) -> List[int]:
    """Id 1 followed by a fixed spread of ids: latency depends on the length, not the content
    (bench_main.cc:96-106; ids kept inside small vocabularies here)."""
    low = 100 if vocab > 200 else 0
    return [1 % vocab] + [low + (i * 7919) % (vocab - low) for i in range(1, length)]


def percentile(samples: Sequence[float], p: float) -> float:
    """Nearest rank: the smallest sample with at least p % of the samples at or below it."""
    ordered = sorted(samples)
    rank = math.ceil(p / 100.0 * len(ordered))
    return ordered[max(rank, 1) - 1]


def row(name: str, unit: str, samples: Sequence[float]) -> str:
    mean = sum(samples) / len(samples)
    return (f"  {name:<15s} {unit:<5s} {mean:10.2f} {percentile(samples, 50):10.2f} {percentile(samples, 90):10.2f} "
            f"{percentile(samples, 99):10.2f} {min(samples):10.2f} {max(samples):10.2f}")


def run_request(engine, prompt: Sequence[int], tokens: int, copies: int) -> Dict[int, List[float]]:
    """Submits `copies` copies of the prompt and returns, per sequence, the times (ms from the
    start) at which its tokens reached the host."""
    stamps: Dict[int, List[float]] = {i: [] for i in range(copies)}
    start = time.perf_counter()
    for i in range(copies):
        status, message = engine.submit(i, prompt, tokens)
        if status != "ok":
            raise RuntimeError(f"request refused ({status}): {message}")
    left = copies
    while left:
        events = engine.poll()
        now = (time.perf_counter() - start) * 1e3
        if not events:
            raise RuntimeError("the engine went idle before every request had finished: " + engine.failure)
        for rid, token, _, finish in events:
            if token >= 0:
                stamps[rid].append(now)
            if finish:
                if finish != "length":
                    raise RuntimeError(f"request {rid} ended with {finish!r}")
                left -= 1
    return stamps


def kernel_report(engine, run, dtype: str) -> str:
    from ..csrc.profile import profiler
    prof = profiler()
    graphs = engine.executor.use_graphs
    engine.executor.use_graphs = False           # a graph replays its kernels unseen by the profiler
    prof.reset()
    prof.enable(True)
    start = time.perf_counter()
    try:
        stamps = run()
    finally:
        prof.enable(False)
        engine.executor.use_graphs = graphs
    stats = prof.stats()
    wall = (time.perf_counter() - start) * 1e3
    total = sum(s.ms for s in stats) or 1e-9
    peak_tf = PEAK_TFLOPS[dtype]
    from ..csrc.peaks import measured_peaks
    measured = measured_peaks()
    lines = [f"\nper-kernel breakdown of one profiled request ({wall:.1f} ms wall, {total:.1f} ms on device; "
             "steps launched kernel by kernel, no captured graphs)",
             f"device peaks: {HBM_PEAK_GBS:.0f} GB/s memory, {peak_tf:.1f} TFLOP/s dense {dtype} (MI355X, published); measured "
             f"on this device: {measured['hbm_gbs']:.0f} GB/s by a kernel that only reads, {measured['bf16_tflops']:.0f} TFLOP/s of "
             "nothing but bfloat16 MFMAs\n",
             f"  {'kernel':<24s} {'calls':>7s} {'ms':>9s} {'%':>6s} {'TFLOP/s':>9s} {'%peak':>6s} {'GB/s':>9s} {'%peak':>6s} "
             f"{'%meas':>6s} {'req GB/s':>9s} {'re-read':>8s}"]
    for s in stats:
        sec = s.ms / 1e3
        tf = s.flops / sec / 1e12 if sec > 0 else 0.0
        gbs = s.bytes / sec / 1e9 if sec > 0 else 0.0
        req = s.moved / sec / 1e9 if sec > 0 else 0.0
        lines.append(f"  {s.name:<24s} {s.calls:7d} {s.ms:9.2f} {100 * s.ms / total:6.1f} {tf:9.2f} {100 * tf / peak_tf:6.1f} "
                     f"{gbs:9.1f} {100 * gbs / HBM_PEAK_GBS:6.1f} {100 * gbs / measured['hbm_gbs']:6.1f} {req:9.1f} "
                     f"{(s.moved / s.bytes if s.bytes > 0 else 0.0):8.1f}")
    slowest = max(stamps.values(), key=lambda t: t[-1])
    lines += [f"\n  {'host + gaps':<24s} {wall - total:9.2f} ms ({100 * (wall - total) / wall:.1f}% of wall) -- launches, "
              "token copies, the profiler's events",
              f"  profiled TTFT {slowest[0]:.2f} ms, E2E {slowest[-1]:.2f} ms (compare with the table above, which ran "
              "without the profiler)",
              "\n  ms       device time between the events around every launch, summed",
              "  TFLOP/s  floating-point work the result needs / device time",
              "  GB/s     bytes that have to be moved at least (every operand once) / device time; %peak of the published",
              "           bandwidth, %meas of what a kernel that only reads reaches on this device",
              "  req      bytes the kernel's workgroups ask for in all / device time (what L2 has to deliver)",
              "  re-read  asked for / moved at least: 1.0 means every byte is read once; the weight-streaming product reads",
              "           all its rows of x in every block of 16 columns, prompt attention walks the keys once per piece of rows"]
    return "\n".join(lines)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="llm-bench", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="model folder (config.json + model.safetensors)")
    ap.add_argument("--prompt", default="", help="comma-separated token ids")
    ap.add_argument("--prompt-len", type=int, default=0, help="use a synthetic prompt of N ids instead")
    ap.add_argument("--tokens", type=int, default=32, help="tokens to generate per request (default 32)")
    ap.add_argument("--runs", type=int, default=20, help="measured requests (default 20)")
    ap.add_argument("--warmup", type=int, default=2, help="unmeasured requests first (default 2)")
    ap.add_argument("--batch", type=int, default=0, help="decode N copies of the prompt together")
    ap.add_argument("--kernels", action="store_true", help="add a per-kernel breakdown of one profiled request")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-tokens", type=int, default=64)
    ap.add_argument("--random-weights", metavar="CONFIG_JSON", default=None,
                    help="first write --model from this config.json with random weights")
    ap.add_argument("--weights-seed", type=int, default=0)
    args = ap.parse_args(argv)
    prompt = parse_ids(args.prompt)
    if bool(prompt) == (args.prompt_len > 0) or args.tokens < 2 or args.runs < 1 or args.warmup < 0 or args.batch < 0:
        # exactly one prompt source; at least two tokens so that TPOT has a sample
        ap.print_usage(sys.stderr)
        return 1
    if args.random_weights:
        from ..config.base import read_config_json
        from ..weights import write_random_model
        write_random_model(read_config_json(args.random_weights), args.weights_seed, args.model, args.dtype)

    import torch
    from ..engine.engine import Engine
    from ..errors import EngineError
    n_prompt = len(prompt) or args.prompt_len
    copies = max(args.batch, 1)
    free_before, _ = torch.cuda.mem_get_info()
    load_start = time.perf_counter()
    try:
        engine = Engine(args.model, max_tokens=n_prompt + args.tokens, max_seqs=copies, dtype=args.dtype,
                        page_tokens=args.page_tokens, max_batch_tokens=max(2048, copies))
    except EngineError as e:
        print(f"[llm] {e}", file=sys.stderr)
        return 1
    torch.cuda.synchronize()
    load_ms = (time.perf_counter() - load_start) * 1e3
    free_after, _ = torch.cuda.mem_get_info()
    if not prompt:
        prompt = synthetic_prompt(args.prompt_len, engine.vocab_size)
    mib = 2.0 ** 20
    print(f"model      {args.model}")
    print(f"request    prompt {n_prompt} tokens, generate {args.tokens} tokens"
          + (f", {args.batch} sequences decoded together" if args.batch else "")
          + f" | {args.warmup} warmup + {args.runs} measured runs")
    print(f"load       {load_ms:.0f} ms (file read, upload, weight layouts; excluded below)")
    print(f"memory     {(free_before - free_after) / mib:.1f} MiB taken on the device | {engine.model.weight_bytes / mib:.1f} "
          f"weights ({engine.model.device_weight_bytes / mib:.1f} on the device, as the kernels read them) + "
          f"{engine.executor.cache.storage_bytes() / mib:.1f} cache accounted, dtype {args.dtype}")
    print(f"kv pool    {engine.kv_pages} pages of {args.page_tokens} tokens | max batch {engine.max_seqs} at "
          f"{engine.max_tokens} tokens per sequence\n")

    request = lambda: run_request(engine, prompt, args.tokens, copies)
    for _ in range(args.warmup):
        request()
    ttft, e2e, tps_decode, tps_e2e, tpot_all, tpot_first, tpot_last, batch_decode, batch_e2e = ([] for _ in range(9))
    for _ in range(args.runs):
        stamps = request()
        for t in stamps.values():
            gaps = [b - a for a, b in zip(t, t[1:])]
            ttft.append(t[0])
            e2e.append(t[-1])
            tps_decode.append((args.tokens - 1) / ((t[-1] - t[0]) / 1e3))
            tps_e2e.append(args.tokens / (t[-1] / 1e3))
            tpot_all.extend(gaps)
            tpot_first.append(gaps[0])
            tpot_last.append(gaps[-1])
        if args.batch:
            last_first = max(t[0] for t in stamps.values())
            last = max(t[-1] for t in stamps.values())
            batch_decode.append(args.batch * (args.tokens - 1) / ((last - last_first) / 1e3))
            batch_e2e.append(args.batch * args.tokens / (last / 1e3))
    print(f"  {'metric':<15s} {'unit':<5s} {'mean':>10s} {'p50':>10s} {'p90':>10s} {'p99':>10s} {'min':>10s} {'max':>10s}")
    print(row("TTFT", "ms", ttft))
    print(row("TPOT (all)", "ms", tpot_all))
    print(row("TPOT (1st)", "ms", tpot_first))
    print(row("TPOT (last)", "ms", tpot_last))
    print(row("E2E latency", "ms", e2e))
    print(row("TPS (decode)", "tok/s", tps_decode))
    print(row("TPS (e2e)", "tok/s", tps_e2e))
    if args.batch:
        print(row("TPS batch (dec)", "tok/s", batch_decode))
        print(row("TPS batch (e2e)", "tok/s", batch_e2e))
        print("\n  rows above the batch rows are per sequence; batch rows are whole-batch rates")
    if args.kernels:
        print(kernel_report(engine, request, args.dtype))
    if args.runs < 100:
        print(f"\n  note: p99 over {args.runs} runs is the max sample; use --runs 100+ for a real tail")
    return 0


if __name__ == "__main__":
    sys.exit(main())
