"""bench: time to first token and decode rate of one checkpoint.

Options as in the reference (cmd/bench/main.go:16-27): ``--model``,
``--device``, ``--prompt`` (length of the synthetic prompt), ``--steps``
(decode steps to time), ``--reps`` (best reported), ``--max-seq`` (KV
capacity), ``--json``, ``--attn-kernel`` (-1 default kernels, 0 the kernel
that takes every size).  ``--fused`` is accepted and has no effect: the
residual add is always fused into the norm.  Added: ``--dtype``, ``--batch``
(one number or several, ``1,8,64``: one result each), ``--random CONFIG.json``,
``--page-size``, and ``--kernel NAME --shape a,b,...``, which times one kernel
alone and quotes it against the published and the measured peaks (the
reference's te_bench_matmul, backend/model.cu:800-863, for every hot kernel;
see ``kllm_amd.benchmark.bench_kernel`` for names and shapes).  As in the reference, TTFT is the mean of 16
prefills of the prompt and ITL the mean over the timed single-token steps
(cmd/bench/main.go:73-122); both are bracketed by device synchronisation.
"""

from __future__ import annotations

import argparse
import json
import sys
import time


def build_parser():
    ap = argparse.ArgumentParser(prog="bench", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--backend", default=None, help="path of a prebuilt kernel library")
    ap.add_argument("--model", default="testmodels/tiny-llama", help="checkpoint folder")
    ap.add_argument("--random", default=None, metavar="CONFIG.json", help="seeded random weights for this config")
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--prompt", type=int, default=32, help="prompt length (synthetic token ids)")
    ap.add_argument("--steps", type=int, default=128, help="decode steps to time")
    ap.add_argument("--reps", type=int, default=3, help="repetitions (best reported)")
    ap.add_argument("--fused", default="true", help="accepted for compatibility; always fused")
    ap.add_argument("--max-seq", type=int, default=512, help="KV capacity in tokens per request")
    ap.add_argument("--json", action="store_true", help="emit one JSON result object")
    ap.add_argument("--attn-kernel", type=int, default=-1, help="-1 default, 0 the generic kernel")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", default="1", help="requests decoded together; several values give a sweep: 1,8,64")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--kernel", default=None, help="time one kernel alone instead of the model")
    ap.add_argument("--shape", default="", help="comma-separated sizes for --kernel")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.backend:
        import os
        os.environ["KLLM_AMD_LIBRARY"] = args.backend
    import torch
    from .. import benchmark as B
    from ..engine import Engine, EngineOptions, StepEntry

    if args.kernel:
        try:
            res = B.bench_kernel(args.kernel, [int(v) for v in args.shape.replace("x", ",").split(",") if v],
                                 args.dtype, reps=max(1, args.steps), warmup=4)
        except Exception as e:
            print(f"error: {e}", file=sys.stderr)
            return 1
        if args.json:
            print(json.dumps(res))
        else:
            print("  ".join(f"{k} {v}" for k, v in res.items() if v != ""))
        return 0
    try:
        batches = [int(b) for b in str(args.batch).split(",") if b]
    except ValueError:
        print(f"error: bad --batch {args.batch!r}", file=sys.stderr)
        return 1
    if not batches or min(batches) < 1:
        print(f"error: bad --batch {args.batch!r}", file=sys.stderr)
        return 1
    opts = EngineOptions(device=args.device, dtype=args.dtype, page_size=args.page_size,
                         max_tokens=(args.max_seq + args.page_size) * max(batches), max_requests=max(64, max(batches)),
                         max_model_len=args.max_seq, attention="generic" if args.attn_kernel == 0 else "auto")
    results = []
    try:
        if args.random:
            with open(args.random) as f:
                eng = Engine.from_random(json.load(f), 0, opts)
            name = args.random
        else:
            eng = Engine.from_dir(args.model, opts)
            name = args.model
        if args.prompt + args.steps + 8 > args.max_seq:
            raise ValueError(f"--prompt {args.prompt} + --steps {args.steps} does not fit --max-seq {args.max_seq}")
        print(eng.capacity_report(), file=sys.stderr)
        vocab = eng.vocab_size
        eng.generate([B.synthetic_ids(args.prompt, vocab)], 8)            # warm-up, as the reference does
        for batch in batches:
            best_ttft, best_itl = None, None
            for _ in range(args.reps):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(16):
                    eng.step([StepEntry(("ttft", i), B.synthetic_ids(args.prompt, vocab, i), [args.prompt - 1])])
                    eng.release(("ttft", i))
                torch.cuda.synchronize()
                ttft = (time.perf_counter() - t0) * 1e3 / 16
                ms, _ = B.measure_decode(eng, batch, args.prompt + args.steps + 4, args.steps, 4)
                best_ttft = ttft if best_ttft is None else min(best_ttft, ttft)
                best_itl = ms if best_itl is None else min(best_itl, ms)
            results.append({"model": name, "fused": True, "prompt_len": args.prompt, "steps": args.steps,
                            "reps": args.reps, "ttft_ms": round(best_ttft, 4), "itl_ms": round(best_itl, 4),
                            "decode_tok_s": round(batch * 1e3 / best_itl, 1), "batch": batch,
                            "dtype": args.dtype})
    except Exception as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    for result in results:
        if args.json:
            print(json.dumps(result))
        else:
            print(f"model {name}  prompt {args.prompt}  steps {args.steps}  batch {result['batch']}  {args.dtype}")
            print(f"TTFT {result['ttft_ms']:.3f} ms   ITL {result['itl_ms']:.3f} ms   "
                  f"decode {result['decode_tok_s']:.1f} tok/s")
    return 0


if __name__ == "__main__":
    sys.exit(main())
