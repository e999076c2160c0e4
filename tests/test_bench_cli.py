"""The llm-bench program: its statistics and the kernel profiler's accounting on the host; the
program itself on the GPU."""
import os
import subprocess
import sys

import pytest

import helpers
from bare_cuda_4gib_amd.cli.bench import percentile, synthetic_prompt
from bare_cuda_4gib_amd.csrc.profile import KernelProfiler


def test_nearest_rank_percentiles():
    """The smallest sample with at least p % of the samples at or below it: always a value that
    was seen (reference: bench/src/bench_main.cc:108-112)."""
    s = [5.0, 1.0, 4.0, 2.0, 3.0]
    assert [percentile(s, p) for p in (0, 1, 20, 21, 50, 90, 99, 100)] == [1.0, 1.0, 1.0, 2.0, 3.0, 5.0, 5.0, 5.0]
    assert percentile([7.0], 99) == 7.0
    twenty = [float(i) for i in range(1, 21)]
    assert percentile(twenty, 99) == 20.0 and percentile(twenty, 90) == 18.0 and percentile(twenty, 50) == 10.0


def test_synthetic_prompt_stays_in_the_vocabulary():
    for vocab in (50, 256, 32000):
        ids = synthetic_prompt(300, vocab)
        assert len(ids) == 300 and all(0 <= t < vocab for t in ids) and ids == synthetic_prompt(300, vocab)


class FakeEvent:
    """Stands for a device event: `record` takes the next tick of a shared clock."""
    clock = [0.0]

    def record(self):
        FakeEvent.clock[0] += 1.5
        self.at = FakeEvent.clock[0]

    def synchronize(self):
        pass

    def elapsed_time(self, other):
        return other.at - self.at


def test_profiler_accounting():
    """Per name: calls, the time between the two events of every launch, and the work the caller
    stated, asked for only while the profiler is on; events are reused after a flush."""
    made = []

    def new_event():
        made.append(FakeEvent())
        return made[-1]
    prof = KernelProfiler(new_event)
    asked = []

    def cost(flops, nbytes):
        def f():
            asked.append(flops)
            return flops, nbytes
        return f
    prof.enable(True)
    for name, flops, nbytes in (("gemm", 100.0, 10.0), ("norm", 0.0, 4.0), ("gemm", 300.0, 30.0)):
        mark = prof.begin(name, cost(flops, nbytes))
        prof.end(mark)
    mark = prof.begin("bare", None)
    prof.end(mark)
    mark = prof.begin("reread", lambda: (8.0, 10.0, 25.0))        # operations, bytes at least, bytes asked for in all
    prof.end(mark)
    stats = {s.name: s for s in prof.stats()}
    assert stats["reread"].bytes == 10.0 and stats["reread"].moved == 25.0
    assert stats["gemm"].moved == 40.0                              # nothing said: every byte once
    assert stats["gemm"].calls == 2 and stats["gemm"].flops == 400.0 and stats["gemm"].bytes == 40.0
    assert stats["gemm"].ms == pytest.approx(3.0) and stats["norm"].ms == pytest.approx(1.5)
    assert stats["bare"].calls == 1 and stats["bare"].flops == 0.0
    assert [s.name for s in prof.stats()][0] == "gemm" and asked == [100.0, 0.0, 300.0]
    n_events = len(made)
    prof.end(prof.begin("norm", cost(1.0, 1.0)))
    prof.flush()
    assert len(made) == n_events, "events come from the pool after a flush"
    prof.reset()
    assert prof.stats() == []


@pytest.mark.gpu
def test_llm_bench_program(tmp_path):
    """One sequence, then three together with the kernel table: the rows are there, the table's
    shares add up, and the kernels of a decode step and of a prefill are in it."""
    folder = helpers.make_model_dir(tmp_path, "A", "bfloat16")
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "llm-bench")
    run = lambda *a: subprocess.run([sys.executable, exe, "--model", folder, *a], capture_output=True, text=True, timeout=300)
    one = run("--prompt", "5,17,3,9,200", "--tokens", "6", "--runs", "3", "--warmup", "1")
    assert one.returncode == 0, one.stderr[-2000:]
    for name in ("TTFT", "TPOT (all)", "TPOT (1st)", "TPOT (last)", "E2E latency", "TPS (decode)", "TPS (e2e)"):
        assert any(line.strip().startswith(name) for line in one.stdout.splitlines()), name
    assert "TPS batch" not in one.stdout and "prompt 5 tokens, generate 6 tokens" in one.stdout
    # (three prompts of 20 tokens are 60 rows a step: up to 64 the weight-streaming product takes them)
    many = run("--prompt-len", "20", "--tokens", "5", "--runs", "2", "--warmup", "1", "--batch", "3", "--kernels")
    assert many.returncode == 0, many.stderr[-2000:]
    assert "TPS batch (dec)" in many.stdout and "3 sequences decoded together" in many.stdout
    table = many.stdout.split("per-kernel breakdown")[1]
    rows = [l.split() for l in table.splitlines() if l.startswith("  ") and len(l.split()) == 11 and l.split()[1].isdigit()]
    names = {r[0] for r in rows}
    assert {"gemm_skinny_qkv", "attention_mfma", "gemm_skinny", "argmax", "embed_gather"} <= names, names
    assert abs(sum(float(r[3]) for r in rows) - 100.0) < 1.0
    assert "host + gaps" in table and "measured on this device" in table
    by_name = {r[0]: r for r in rows}
    assert float(by_name["gemm_skinny"][10]) > 1.5, "the weight-streaming product reads x once per block of columns"
    assert float(by_name["argmax"][10]) == 1.0
    assert run("--prompt", "1,2", "--prompt-len", "4").returncode == 1          # two prompt sources
    assert run("--prompt-len", "4", "--tokens", "1").returncode == 1            # TPOT needs two tokens


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_llm_batch_check_program(tmp_path, dtype):
    """The program itself on a tiny model with random prompts: eight prompts (the longest the model's positions hold),
    four decoding at once; in 32-bit every request's ids are identical alone and batched, in bfloat16 a split may only
    be a near-tie."""
    import helpers
    folder = helpers.make_model_dir(tmp_path, "C", dtype, variant="spread")
    prog = os.path.join(helpers.ROOT, "bin", "llm-batch-check")
    proc = subprocess.run([sys.executable, prog, "--model", folder, "--tokens", "24", "--batch", "4", "--dtype", dtype,
                           "--page-tokens", "16"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    assert lines[-1] == "PASS: batched decode agrees with decoding alone"
    assert "8 prompts of 6-301 tokens, 24 new tokens each, 4 decoding at once" in lines[1]
    verdicts = [l for l in lines if l.startswith("prompt ")]
    assert len(verdicts) == 8
    if dtype == "float32":
        assert all("match, 24 ids identical" in l for l in verdicts), proc.stdout
    bad = subprocess.run([sys.executable, prog, "--model", str(tmp_path / "none")], capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "config.json" in bad.stderr
