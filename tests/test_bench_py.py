"""bench.py keeps its contract: one JSON line with the keys the record wants, a refusal of more than one GPU, and
every `--only` part runs.  (Two layers of the shape instead of all: the contract's words, not the speed, are what
is tested here; `config` then names both numbers.)"""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def bench(*args, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    done = bench("--gpus", "2")
    assert done.returncode == 2 and len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout


@pytest.mark.gpu
def test_the_headline_line():
    done = bench("--layers", "2", "--steps", "6", "--warmup", "2")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 6 and line["warmup"] == 2 and line["dtype"] == "bf16"
    assert line["higher_is_better"] is True and line["unit"] == "tokens/s" and "synthetic" in line["data"]
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())       # flat
    assert config["layers"] == 2 and config["layers_full"] == 22 and config["global_batch"] == 8 and config["seq_len"] == 2048
    for key in ("hidden", "heads", "kv_heads", "head_dim", "intermediate", "vocab"):
        assert isinstance(config[key], int)
    assert set(line["prefill"]) >= {"value", "tokens", "ms", "frac"} and line["prefill"]["tokens"] == 2048
    assert 0.0 < line["prefill"]["frac"] < 1.0
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0.0 < roof["frac"] < 1.0
    assert set(line["points"]) == {"decode_b1", "decode_b64"} and all(v > 0 for v in line["points"].values())
    assert abs(line["value"] - 8 * 1e3 / line["ms_per_step"]) < 0.01 * line["value"]                 # batch 8 a step


@pytest.mark.gpu
@pytest.mark.parametrize("part", [["decode", "--batch", "4", "--steps", "4", "--warmup", "1"], ["prefill", "--prefill-tokens", "300"],
                                  ["serve", "--requests", "6", "--new-tokens", "8", "--top-k", "5", "--top-p", "0.9"],
                                  ["chat", "--requests", "4", "--gather-ms", "2"], ["gemm", "--mnk", "64,256,128"]])
def test_every_part_alone(part):
    done = bench("--layers", "2", "--only", *part)
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads([l for l in done.stdout.splitlines() if l.startswith("{")][-1])
    assert line["only"] == part[0]
