"""Headline benchmark: decode tokens a second of a TinyLlama-1.1B-sized model
with random weights on one MI355X (batch 8, contexts ending at 2,048 tokens),
plus prefill of 2,048 tokens and decode at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32]

Prints one JSON line.  A "step" is one decode step of the whole batch: the
forward pass over the cache, sampling on the device, the tokens read back.
"""

import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="context length the timed steps end at")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--gemm", default="hip", choices=["hip", "library"])
    ap.add_argument("--prefill-only", action="store_true", help="time the 2,048-token prefill only (for profiles)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--model", default="tinyllama-1.1b", choices=["tinyllama-1.1b", "llama2-7b", "llama3-8b"],
                    help="whose sizes to run (the default is the headline configuration)")
    args = ap.parse_args(argv)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not built")
        return 2

    import torch
    from kllm_amd import benchmark as B

    cfg = dict(B.PRESETS[args.model])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    elem = 2 if args.dtype == "bfloat16" else 4
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    eng = B.make_engine(cfg, args.dtype, max_tokens=max_batch * args.context + 4096,
                        max_model_len=args.context + 64, gemm=args.gemm, page_size=args.page_size)

    if args.prefill_only:
        pms = B.measure_prefill(eng, 2048, reps=max(1, args.steps), warmup=args.warmup)
        print(json.dumps({"prefill_ms": round(pms, 3), "tok_s": round(2048e3 / pms, 1)}))
        return 0
    ms, ctx = B.measure_decode(eng, args.batch, args.context, args.steps, args.warmup)
    value = args.batch * 1e3 / ms
    need = B.decode_step_bytes(cfg, args.batch, int(ctx), elem)
    achieved = need / (ms * 1e-3) / 1e9
    out = {
        "metric": "decode tok/s, %s sizes, random weights" % {"tinyllama-1.1b": "TinyLlama-1.1B", "llama2-7b": "Llama-2-7B",
                                                               "llama3-8b": "Llama-3-8B"}[args.model],
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": args.model + "-sizes", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
            "rope_theta": cfg["rope_theta"], "rms_eps": cfg["rms_norm_eps"],
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": 2048,
            "page_size": eng.options.page_size, "parallelism": "single-gpu", "weights": "random",
            "gemm": args.gemm,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": B.PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / B.PEAK_HBM_GBS, 4)},
    }
    if not args.no_points:
        T = 2048
        pms = B.measure_prefill(eng, T)
        flops = B.prefill_flops(cfg, T)
        out["prefill"] = {"value": round(T * 1e3 / pms, 1), "tokens": T, "ms": round(pms, 3),
                          "frac": round(flops / (pms * 1e-3) / B.PEAK_FLOPS[args.dtype], 4)}
        points = {}
        for b in (1, 64):
            k = max(16, args.steps // 2)
            bms, _ = B.measure_decode(eng, b, args.context, k, 8)
            points[f"decode_b{b}"] = round(b * 1e3 / bms, 1)
        out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
