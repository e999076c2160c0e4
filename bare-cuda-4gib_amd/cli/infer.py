"""``llm-infer``: load a model folder, run a prompt of token ids through it,
print the generated ids.  Options as in the reference's program of the same
name (bench/src/main.cc:18-95): ``--model --prompt id,id,... [--tokens N]
[--max-seq N]``; ids in, ids out, no tokenizer.  Added here: ``--dtype``,
the sampling options of the Python entry point, ``--kv-pages`` /
``--page-tokens`` for the cache pool, and ``--random-weights`` to write the
model folder from a configuration and a seed first."""
from __future__ import annotations

import argparse
import sys
from typing import List


def parse_ids(text: str) -> List[int]:
    return [int(piece) for piece in text.split(",") if piece.strip()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="llm-infer", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="model folder (config.json + model.safetensors)")
    ap.add_argument("--prompt", required=True, help="comma-separated token ids")
    ap.add_argument("--tokens", type=int, default=16, help="number of tokens to generate (default 16)")
    ap.add_argument("--max-seq", type=int, default=0, help="cache size in tokens; must cover prompt + generated")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--seed", type=int, default=-1, help="sampling seed; -1 draws one")
    ap.add_argument("--kv-pages", type=int, default=0, help="pages in the cache pool; 0 sizes it for --max-seq")
    ap.add_argument("--page-tokens", type=int, default=64, help="tokens per cache page (a multiple of 16)")
    ap.add_argument("--random-weights", metavar="CONFIG_JSON", default=None,
                    help="first write --model from this config.json with random weights")
    ap.add_argument("--weights-seed", type=int, default=0)
    args = ap.parse_args(argv)

    prompt = parse_ids(args.prompt)
    if not prompt:
        print("[llm] no token ids parsed from --prompt", file=sys.stderr)
        return 1
    if args.random_weights:
        from ..config.base import read_config_json
        from ..weights import write_random_model
        write_random_model(read_config_json(args.random_weights), args.weights_seed, args.model, args.dtype)

    from ..engine.engine import Engine, generate_batch
    from ..errors import EngineError
    max_seq = args.max_seq if args.max_seq > 0 else len(prompt) + args.tokens
    try:
        engine = Engine(args.model, max_tokens=max_seq, max_seqs=1, kv_pages=args.kv_pages, dtype=args.dtype,
                        page_tokens=args.page_tokens)
        cache_mib = engine.executor.cache.storage_bytes() / 2**20
        print(f"[llm] {len(engine.model.layers)} layers, hidden {engine.model.hidden_size}, vocab "
              f"{engine.model.vocab_size} | weights {engine.model.weight_bytes / 2**20:.1f} MiB "
              f"({engine.model.device_weight_bytes / 2**20:.1f} on the device, as the kernels read them), cache "
              f"{cache_mib:.1f} MiB ({engine.kv_pages} pages, max batch {engine.max_seqs})")
        generated = generate_batch(engine, [prompt], args.tokens, temperature=args.temperature,
                                   top_p=args.top_p, top_k=args.top_k, seed=args.seed)[0]
    except EngineError as e:
        print(f"[llm] {e}", file=sys.stderr)
        return 1
    print("prompt:    " + " ".join(str(t) for t in prompt))
    print("generated: " + " ".join(str(t) for t in generated))
    return 0


if __name__ == "__main__":
    sys.exit(main())
