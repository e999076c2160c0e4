"""Shared by the tests: tiny configurations, model folders, traces and replay."""
from __future__ import annotations

import json
import os
import random
import subprocess
import sys
from typing import Dict, List, Sequence, Tuple

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Tiny configurations of the architecture that differ in every size and option:
# layers, width, head counts and grouping (4/2 grouped, 3/3 not grouped, 6/2 with a group of
# three), head size (16, 32, 48), feed-forward width (176 is no multiple of 64), vocabulary
# (301 is odd), rope_theta, rms_norm_eps, max positions, tied or untied output head, and a
# width that is not heads * head_dim (C).
TINY_A = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, intermediate_size=176,
              rope_theta=10000.0, rms_norm_eps=1e-5, max_position_embeddings=128,
              tie_word_embeddings=False)
TINY_B = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=384, hidden_size=96,
              num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=3, intermediate_size=256,
              rope_theta=500000.0, rms_norm_eps=1e-6, max_position_embeddings=256,
              tie_word_embeddings=True)
TINY_C = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=301, hidden_size=80,
              num_hidden_layers=1, num_attention_heads=6, num_key_value_heads=2, head_dim=48,
              intermediate_size=112, rope_theta=1000.0, rms_norm_eps=1e-3,
              max_position_embeddings=512, tie_word_embeddings=False)
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 2), "C": (TINY_C, 5)}   # name -> (config, weight seed)


# How a model folder's weights are drawn.  "ones": every matrix N(0, 0.02), every norm scale exactly
# 1.0 (what the benchmark's configurations say).  "spread": every norm scale 1 + 0.1 * randn, a draw of
# its own for each norm (the reference's fixture draws 1 + 0.05 * randn,
# tools/references/reference_forward.py:306-318) -- a scale handed to the wrong norm, or dropped,
# then changes the logits -- and query and key weights several times as large, so that the scores
# have a spread of about one to two and attention is peaked rather than near-uniform: a wrong key or a
# wrong score shows.  (Configuration B, with three layers, gets the smaller factor: peaked attention
# multiplies whatever error the layers before have left in its input -- the plain implementation itself,
# with its activations rounded to bfloat16 where the engine rounds them, is off by more than the
# bfloat16 tolerance at a factor of eight there, and by half of it at five.)
QK_FACTOR = {"A": 8.0, "B": 5.0, "C": 8.0}


def variant_args(name: str, variant: str) -> dict:
    if variant == "ones":
        return {}
    assert variant == "spread"
    f = QK_FACTOR[name]
    return dict(norm_std=0.1, scales={"*.q_proj.weight": f, "*.k_proj.weight": f})


def make_model_dir(tmp_path, name: str, dtype: str = "float32", std: float = 0.02, variant: str = "ones") -> str:
    """A model folder with random weights, written by the framework's own random-weights mode."""
    from bare_cuda_4gib_amd.weights import write_random_model
    cfg, seed = TINY[name]
    out = os.path.join(str(tmp_path), f"tiny_{name}_{dtype}_{variant}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        write_random_model(cfg, seed, out, dtype, std=std, **variant_args(name, variant))
    return out


def random_ids(n: int, vocab: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(x) for x in rng.integers(0, vocab, size=n)]


# --- traces -------------------------------------------------------------------
# A trace is a list of steps {"step", "entries": [{"id", "tokens", "want"}], "end"}; alongside it,
# `where` maps (step, row in that step's output) -> (request, absolute position).

def _finish(steps):
    where = {}
    for s in steps:
        r = 0
        for e in s["entries"]:
            for w in e["want"]:
                where[(s["step"], r)] = (e["id"], e["_start"] + w)
                r += 1
    clean = [{"step": s["step"], "entries": [{k: v for k, v in e.items() if k != "_start"} for e in s["entries"]],
              "end": s["end"]} for s in steps]
    return clean, where


def trace_whole(requests: Dict[str, List[int]]):
    """Each request alone and whole, logits at every position."""
    steps = []
    for i, (rid, ids) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids))), "_start": 0}],
                      "end": [rid]})
    return _finish(steps)


def trace_tail_one_by_one(requests: Dict[str, List[int]], tail: int = 32):
    """Most of each request in one step, its last `tail` tokens one by one."""
    steps, n = [], 0
    for rid, ids in requests.items():
        head = max(1, len(ids) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[:head], "want": [head - 1], "_start": 0}], "end": []})
        n += 1
        for p in range(head, len(ids)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [ids[p]], "want": [0], "_start": p}],
                          "end": [rid] if p == len(ids) - 1 else []})
            n += 1
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return _finish(steps)


def trace_portions(requests: Dict[str, List[int]], seed: int, sizes: Sequence[int] = (17, 2, 5, 64, 3, 2, 31, 9)):
    """Each request in portions of changing size, down to two tokens; logits at every position."""
    rng = random.Random(seed)
    steps, n = [], 0
    for rid, ids in requests.items():
        p, k = 0, rng.randrange(len(sizes))
        while p < len(ids):
            size = min(sizes[k % len(sizes)], len(ids) - p)
            if len(ids) - p - size == 1:      # never leave a single token: portions go down to two
                size += 1
            k += 1
            last = p + size == len(ids)
            steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[p:p + size], "want": list(range(size)),
                                                  "_start": p}], "end": [rid] if last else []})
            n += 1
            p += size
    return _finish(steps)


def trace_mixed(requests: Dict[str, List[int]], seed: int, max_live: int = 4, tail: int = 12,
                page_tokens: int = 64):
    """Up to `max_live` live requests; portions of some beside single decoded tokens of others;
    requests left out of a step now and then; a finished request's place goes to the next one.
    Returns (steps, where, max_tokens): max_tokens is the peak of the live requests' token counts,
    each rounded up to whole pages, so a pool of that size makes pages go round."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: List[Tuple[str, List[int]]] = []
    done_upto: Dict[str, int] = {}
    steps, n, peak = [], 0, 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, ids = waiting.pop(0)
            live.append((rid, ids))
            done_upto[rid] = 0
        entries, ends = [], []
        order = list(live)
        rng.shuffle(order)                      # batch order is not admission order
        for rid, ids in order:
            if len(order) > 1 and rng.random() < 0.2:
                continue                        # left out of this step, goes on later
            p = done_upto[rid]
            remaining = len(ids) - p
            if remaining <= tail:
                size = 1                        # decoding: one token a step
            else:
                size = min(rng.choice([2, 3, 7, 16, 29, 40, 64]), remaining - tail)
                if size < 2:
                    size = remaining - tail if remaining - tail >= 2 else 1
            want = sorted(set([0, size - 1] + [rng.randrange(size) for _ in range(2)]))
            entries.append({"id": rid, "tokens": ids[p:p + size], "want": want, "_start": p})
            done_upto[rid] = p + size
            if p + size == len(ids):
                ends.append(rid)
        held = sum(-(-done_upto[rid] // page_tokens) * page_tokens for rid, _ in live)
        peak = max(peak, held)
        if entries:
            steps.append({"step": n, "entries": entries, "end": ends})
            n += 1
        live = [(rid, ids) for rid, ids in live if rid not in ends]
    clean, where = _finish(steps)
    return clean, where, peak


# --- replay -------------------------------------------------------------------

def replay_in_process(executor, steps) -> Dict[Tuple[int, int], np.ndarray]:
    """Run a trace on an Executor, as bin/trace_run does; (step, row) -> logits row."""
    from bare_cuda_4gib_amd.engine import StepEntry
    out = {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not executor.has(e["id"]):
                executor.admit(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = executor.step(entries)
        if logits is not None:
            rows = logits.float().cpu().numpy()
            for r in range(rows.shape[0]):
                out[(s["step"], r)] = rows[r]
        for rid in s["end"]:
            executor.release(rid)
    return out


def replay_subprocess(model_dir: str, dtype: str, steps, out_dir: str, max_tokens: int, vocab: int,
                      extra: Sequence[str] = ()) -> Dict[Tuple[int, int], np.ndarray]:
    """Run a trace through bin/trace_run itself."""
    os.makedirs(out_dir, exist_ok=True)
    text = "".join(json.dumps(s) + "\n" for s in steps)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
                           "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens), *extra],
                          input=text, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    dones = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert dones == [f"done {s['step']}" for s in steps], proc.stdout[-2000:]
    out = {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if n_want == 0:
            assert not os.path.exists(path)
            continue
        rows = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        for r in range(n_want):
            out[(s["step"], r)] = rows[r]
    return out


def compare_with_plain(got, where, plain_logits: Dict[str, np.ndarray], rtol: float, atol: float, label: str,
                       row_rms: float = 0.0):
    """Every logits row the replay produced against the plain implementation's row at the same
    request and position; reports the first wrong place.  ``row_rms`` (if not 0): moreover the root
    mean square of a row's errors may be at most this fraction of the root mean square of the row's
    logits -- rounding noise averages out over a vocabulary, a fault in a scale or a sum does not."""
    assert set(got) == set(where), f"{label}: rows produced {len(got)}, rows expected {len(where)}"
    worst = 0.0
    for key in sorted(where):
        rid, pos = where[key]
        ref = plain_logits[rid][pos]
        row = got[key]
        assert np.all(np.isfinite(row)), f"{label}: non-finite logits at step {key[0]} request {rid} position {pos}"
        err = np.abs(row - ref)
        if row_rms:
            e, r = float(np.sqrt(np.mean(err * err))), float(np.sqrt(np.mean(ref * ref)))
            assert e <= row_rms * r, (f"{label}: step {key[0]}, request {rid}, position {pos}: the row's errors have a "
                                      f"root mean square of {e:.3g}, {e / r:.3g} of the logits' {r:.3g} (limit {row_rms:.3g})")
        bound = atol + rtol * np.abs(ref)
        if np.any(err > bound):
            i = int(np.argmax(err - bound))
            raise AssertionError(f"{label}: first wrong row at step {key[0]}, request {rid}, position {pos}: "
                                 f"logit {i} is {row[i]:.6g}, plain {ref[i]:.6g} (|diff| {err[i]:.3g} > {bound[i]:.3g})")
        worst = max(worst, float(err.max()))
    return worst
