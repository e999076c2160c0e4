"""``llm-batch-check``: batched decoding against decoding one request at a time, on a model folder
(reference: bench/src/batch_check_main.cc:1-160 -- the same prompt lengths, more prompts than slots so
that queueing and retiring run too, the same verdict).

Each prompt is decoded greedily alone, then all together through the scheduler.  Alone and batched
steps have other numbers of rows, which may choose other kernels that add in another order, so a
near-tie between the two best logits may break the other way.  Where a request's ids differ, both
candidates are scored by a third, neutral path -- one fresh pass over the shared prefix -- and only a
gap between their logits above ``--tol`` counts as a failure.

The reference reads its prompts from an offline-tokenized text (``--ids``: flat little-endian int32);
without such a file the prompts are drawn uniformly from the vocabulary with ``--seed``.
"""
from __future__ import annotations

import argparse
import sys
from typing import List

PROMPT_LENGTHS = (5, 17, 64, 120, 300, 8, 200, 37)     # text ids; the reference puts BOS before them
PROMPT_SPACING = 1000                                  # ids between the starts of two prompts' slices
BOS_ID = 1


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="llm-batch-check", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="model folder (config.json + model.safetensors)")
    ap.add_argument("--ids", default=None, help="flat little-endian int32 token ids to cut the prompts from")
    ap.add_argument("--tokens", type=int, default=64, help="tokens to generate per prompt (default 64)")
    ap.add_argument("--batch", type=int, default=4, help="sequences decoded at once (default 4)")
    ap.add_argument("--tol", type=float, default=0.01,
                    help="largest logit gap a divergence may have and still pass (default 0.01)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--seed", type=int, default=0, help="without --ids: seed of the random prompts")
    ap.add_argument("--page-tokens", type=int, default=64)
    args = ap.parse_args(argv)
    if args.tokens <= 0 or args.batch <= 0:
        ap.print_usage(sys.stderr)
        return 1

    import numpy as np
    from ..config.registry import load_config
    from ..engine.engine import Engine, generate_batch
    from ..engine.executor import StepEntry
    from ..errors import EngineError

    try:
        _, cfg = load_config(args.model)
        vocab = cfg.vocab_size
        longest_allowed = cfg.max_seq_len - args.tokens
        lengths = [n for n in PROMPT_LENGTHS if n + 1 <= longest_allowed]
        if not lengths:
            print(f"[llm] the model's {cfg.max_seq_len} positions hold no prompt and {args.tokens} new tokens", file=sys.stderr)
            return 1
        prompts: List[List[int]] = []
        if args.ids:
            text = np.fromfile(args.ids, dtype="<i4")
            for p, n in enumerate(lengths):
                start = p * PROMPT_SPACING
                if start + n > text.size:
                    print(f"[llm] {args.ids} has {text.size} ids, too few for prompt {p}", file=sys.stderr)
                    return 1
                prompts.append([BOS_ID] + [int(t) for t in text[start:start + n]])
        else:
            rng = np.random.default_rng(args.seed)
            prompts = [[int(t) for t in rng.integers(0, vocab, size=n + 1)] for n in lengths]
        longest = max(len(p) for p in prompts)
        engine = Engine(args.model, max_tokens=longest + args.tokens, max_seqs=args.batch, kv_pages=0, dtype=args.dtype,
                        page_tokens=args.page_tokens)
        print(f"model      {args.model}")
        print(f"check      {len(prompts)} prompts of {min(len(p) for p in prompts)}-{longest} tokens, {args.tokens} new tokens "
              f"each, {args.batch} decoding at once, dtype {args.dtype}")
        print(f"kv pool    {engine.kv_pages} pages | max batch {engine.max_seqs} at {engine.max_tokens} tokens per sequence\n")

        alone = [generate_batch(engine, [p], args.tokens)[0] for p in prompts]
        together = generate_batch(engine, prompts, args.tokens)

        exact = near_ties = failures = 0
        for p, prompt in enumerate(prompts):
            step = next((i for i, (a, b) in enumerate(zip(alone[p], together[p])) if a != b), None)
            if step is None and len(alone[p]) == len(together[p]):
                exact += 1
                print(f"prompt {p}  {len(prompt):3d} tokens  match, {len(alone[p])} ids identical")
                continue
            step = min(len(alone[p]), len(together[p])) if step is None else step
            # both candidates scored by one fresh pass over the shared prefix: a third, neutral path
            prefix = prompt + alone[p][:step]
            row = engine.step([StepEntry("score", prefix, [len(prefix) - 1])])[0].float().cpu().numpy()
            engine.release("score")
            a = alone[p][step] if step < len(alone[p]) else -1
            b = together[p][step] if step < len(together[p]) else -1
            gap = abs(float(row[a]) - float(row[b])) if a >= 0 and b >= 0 else float("inf")
            tie = gap <= args.tol
            near_ties, failures = near_ties + tie, failures + (not tie)
            print(f"prompt {p}  {len(prompt):3d} tokens  {'near-tie' if tie else 'DIVERGES'} at step {step}: alone {a}, "
                  f"batched {b}, logit gap {gap:.5f}")
    except EngineError as e:
        print(f"[llm] {e}", file=sys.stderr)
        return 1

    print(f"\n{exact} match, {near_ties} split on a near-tie (gap <= {args.tol:.3g}), {failures} diverge")
    if failures:
        print("FAIL: batched decode disagrees with decoding alone beyond rounding")
        return 1
    print("PASS: batched decode agrees with decoding alone")
    return 0


if __name__ == "__main__":
    sys.exit(main())
