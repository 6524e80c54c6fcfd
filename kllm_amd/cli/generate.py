"""generate: decode from a checkpoint with raw token ids.

The options are the reference's (cmd/generate/main.go:15-21): ``--model`` (a
folder with config.json and safetensors), ``--device``, ``--ids``
(space-separated prompt ids), ``--steps`` (most new tokens), ``--max-seq`` (KV
capacity in tokens).  Its ``--backend`` named the CUDA library to load; here
it may name a prebuilt kernel library and is otherwise not needed.  Added:
``--dtype``, ``--temperature``, ``--seed``, ``--sample-seed``, ``--random
CONFIG.json`` for seeded random weights, ``--max-new-tokens`` (another name of
``--steps``), and the engine's sizes: ``--page-size``, ``--num-pages``,
``--max-step-tokens`` (the token budget of a step: longer prompts are cut
into portions) and ``--memory-gib`` (a byte budget that the cache is fitted
into).  What the cache was sized to is printed to standard error at start.
Output as the reference prints it:

    prompt:    [1 17 42 100 7]
    generated: [...]
"""

from __future__ import annotations

import argparse
import json
import sys


def parse_ids(text: str):
    ids = []
    for field in text.split():
        try:
            ids.append(int(field))
        except ValueError:
            raise SystemExit(f"error: bad token id {field!r}")
    return ids


def build_parser():
    ap = argparse.ArgumentParser(prog="generate", description="greedy or sampled decoding from raw token ids")
    ap.add_argument("--backend", default=None, help="path of a prebuilt kernel library (default: built in-tree)")
    ap.add_argument("--model", default="testmodels/tiny-llama", help="checkpoint folder (config.json + safetensors)")
    ap.add_argument("--random", default=None, metavar="CONFIG.json",
                    help="use seeded random weights for this config.json instead of --model")
    ap.add_argument("--device", type=int, default=0, help="GPU index")
    ap.add_argument("--ids", default="1 17 42 100 7", help="space-separated prompt token ids")
    ap.add_argument("--steps", "--max-new-tokens", dest="steps", type=int, default=16, help="max new tokens")
    ap.add_argument("--max-seq", type=int, default=256, help="KV capacity in tokens")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-pages", type=int, default=None, help="cache pages (default: --max-seq tokens' worth)")
    ap.add_argument("--max-step-tokens", type=int, default=None,
                    help="most tokens in one step; a longer prompt is cut into portions (default 2048)")
    ap.add_argument("--memory-gib", type=float, default=None, help="fit the cache into this many GiB")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--seed", type=int, default=0, help="seed of sampling (and of --random weights)")
    ap.add_argument("--sample-seed", type=int, default=None, help="seed of sampling alone (default: --seed)")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    prompt = parse_ids(args.ids)
    if args.backend:
        import os
        os.environ["KLLM_AMD_LIBRARY"] = args.backend
    from ..engine import Engine, EngineOptions
    opts = EngineOptions(device=args.device, dtype=args.dtype, page_size=args.page_size,
                         max_tokens=args.max_seq, num_pages=args.num_pages,
                         memory_bytes=None if args.memory_gib is None else int(args.memory_gib * 2**30),
                         max_model_len=args.max_seq, max_requests=4)
    try:
        if args.random:
            with open(args.random) as f:
                eng = Engine.from_random(json.load(f), args.seed, opts)
        else:
            eng = Engine.from_dir(args.model, opts)
        print(eng.capacity_report(), file=sys.stderr)
        out = eng.generate(prompt, args.steps, temperature=args.temperature,
                           seed=args.seed if args.sample_seed is None else args.sample_seed,
                           max_step_tokens=args.max_step_tokens)
    except Exception as e:  # the reference prints "error: ..." and exits 1
        print(f"error: {e}", file=sys.stderr)
        return 1
    fmt = lambda ids: "[" + " ".join(str(i) for i in ids) + "]"
    print(f"prompt:    {fmt(prompt)}\ngenerated: {fmt(out)}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
