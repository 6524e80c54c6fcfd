"""Headline benchmark: decode tokens a second of a TinyLlama-1.1B-sized model
with random weights on one MI355X (batch 8, contexts ending at 2,048 tokens),
plus prefill of 2,048 tokens and decode at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32]

Prints one JSON line.  A "step" is one decode step of the whole batch: the
forward pass over the cache, sampling on the device, the tokens read back.
``points`` of that line also holds, beside batch 1 and 64: the float32 path at the
same sizes, the 2,048-token prompt in portions of 512, the decode run from 512 to
2,048 tokens, Llama-3-8B sizes at batch 64 with contexts of 4,096, and the mixed
serving workload at Llama-2-7B sizes (``--no-extra`` leaves those out).

Other workloads, each printing one JSON line of its own (``--model`` chooses the sizes):

    --workload decode-run      prompts of 512 tokens decoded to 2,048: mean tok/s over the run
                               and at context lengths 512, 1280 and 2047 (--batch)
    --workload prefill-chunks  a prompt of --context tokens (2,048) in portions of --chunk tokens
    --workload mixed           --requests prompts of 128 to 2,048 tokens through the scheduler,
                               prefilled in portions of --chunk tokens beside decode tokens
    --kernel NAME --shape a,b,..   one kernel alone (gemm n,m,k; gemm_swiglu n,f,k; attn_prefill
                               tokens,H,KV,hd; attn_decode batch,context,H,KV,hd; add_rmsnorm n,d;
                               copy bytes), in microseconds and against nominal and measured peaks
    --calibrate                the box's own copy bandwidth and MFMA rates
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
    ap.add_argument("--no-extra", action="store_true", help="skip the points at other dtypes, sizes and workloads")
    ap.add_argument("--gemm", default="hip", choices=["hip", "library"])
    ap.add_argument("--prefill-only", action="store_true", help="time the 2,048-token prefill only (for profiles)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--model", default="tinyllama-1.1b", choices=["tinyllama-1.1b", "llama2-7b", "llama3-8b"],
                    help="whose sizes to run (the default is the headline configuration)")
    ap.add_argument("--extra", default="", help="engine options for experiments: key=value,key=value (ints or words)")
    ap.add_argument("--workload", default="headline", choices=["headline", "decode-run", "prefill-chunks", "mixed"])
    ap.add_argument("--chunk", type=int, default=512, help="tokens per prompt portion (prefill-chunks, mixed)")
    ap.add_argument("--requests", type=int, default=32, help="requests of the mixed workload")
    ap.add_argument("--new-tokens", type=int, default=64, help="tokens each request of the mixed workload generates")
    ap.add_argument("--kernel", default=None, help="time one kernel alone (see the module's text)")
    ap.add_argument("--shape", default="", help="comma-separated sizes for --kernel")
    ap.add_argument("--calibrate", action="store_true", help="measure the box's copy bandwidth and MFMA rates")
    args = ap.parse_args(argv)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not built")
        return 2

    import torch
    from kllm_amd import benchmark as B

    if args.calibrate:
        print(json.dumps({"calibration": B.calibrate(), "peak_hbm_GBs": B.PEAK_HBM_GBS,
                          "peak_TFLOPs": {k: v / 1e12 for k, v in B.PEAK_FLOPS.items()}}))
        return 0
    if args.kernel:
        shape = [int(v) for v in args.shape.replace("x", ",").split(",") if v]
        res = B.bench_kernel(args.kernel, shape, args.dtype, reps=max(1, args.steps), warmup=max(1, args.warmup))
        res["calibration"] = B.calibrate()
        print(json.dumps(res))
        return 0

    cfg = dict(B.PRESETS[args.model])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    elem = 2 if args.dtype == "bfloat16" else 4
    extra = {}
    for item in filter(None, args.extra.split(",")):
        key, _, val = item.partition("=")
        extra[key] = int(val) if val.lstrip("-").isdigit() else (val or True)
    if args.workload != "headline":
        return other_workload(args, cfg, full_layers, B, extra)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    eng = B.make_engine(cfg, args.dtype, max_tokens=max_batch * args.context + 4096, max_requests=max_batch,
                        max_model_len=args.context + 64, gemm=args.gemm, page_size=args.page_size, extra=extra)

    if args.prefill_only:
        pms = B.measure_prefill(eng, 2048, reps=max(1, args.steps), warmup=args.warmup)
        print(json.dumps({"prefill_ms": round(pms, 3), "tok_s": round(2048e3 / pms, 1)}))
        return 0
    ms, ctx = B.measure_decode(eng, args.batch, args.context, args.steps, args.warmup)
    value = args.batch * 1e3 / ms
    need = eng.step_read_bytes([int(ctx)] * args.batch)      # asked of the model's parts and the cache plan
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
    cal = B.calibrate()     # the box's own copy bandwidth and MFMA rate, beside the published peaks
    out["roofline"]["measured_copy"] = cal["copy_GBs"]
    out["roofline"]["frac_of_measured_copy"] = round(achieved / cal["copy_GBs"], 4)
    out["roofline"]["measured_read"] = cal["read_GBs"]      # a read-only stream: what a decode kernel does
    out["roofline"]["frac_of_measured_read"] = round(achieved / cal["read_GBs"], 4)
    if not args.no_points:
        T = 2048
        pms = B.measure_prefill(eng, T)
        flops = eng.model.step_flops(T, T * (T + 1) / 2.0, 1)
        out["prefill"] = {"value": round(T * 1e3 / pms, 1), "tokens": T, "ms": round(pms, 3),
                          "frac": round(flops / (pms * 1e-3) / B.PEAK_FLOPS[args.dtype], 4),
                          "frac_of_measured_mfma": round(flops / (pms * 1e-3) / 1e12 / cal[f"mfma_{args.dtype}_TFLOPs"], 4)}
        points = {}
        for b in (1, 64):
            k = max(16, args.steps // 2)
            bms, _ = B.measure_decode(eng, b, args.context, k, 8)
            points[f"decode_b{b}"] = round(b * 1e3 / bms, 1)
        if not args.no_extra and args.model == "tinyllama-1.1b" and not args.layers:
            import gc
            points.update(B.same_engine_points(eng))
            del eng                               # the larger models need its memory
            gc.collect()
            torch.cuda.empty_cache()
            points.update(B.other_engine_points(cfg, args.dtype, args.gemm, args.page_size))
        out["points"] = points
    print(json.dumps(out))
    return 0


def other_workload(args, cfg, full_layers, B, extra):
    import torch
    elem = 2 if args.dtype == "bfloat16" else 4
    base = {"workload": args.workload, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "model": args.model + "-sizes", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
            "page_size": args.page_size, "gemm": args.gemm}
    if args.workload == "decode-run":
        eng = B.make_engine(cfg, args.dtype, max_tokens=args.batch * args.context + 4096, max_requests=args.batch,
                            max_model_len=args.context + 64, gemm=args.gemm, page_size=args.page_size)
        res = B.measure_decode_run(eng, args.batch, prompt_len=512, total_len=args.context)
        base.update(batch=args.batch, prompt_len=512, total_len=args.context, unit="tok/s", **res)
        worst = eng.step_read_bytes([args.context - 1] * args.batch)
        base["frac_of_hbm_at_end"] = round(worst * res["at"][max(res["at"])] / args.batch / 1e9 / B.PEAK_HBM_GBS, 4)
    elif args.workload == "prefill-chunks":
        tokens = args.context                      # the prompt's length (2,048 unless --context says otherwise)
        eng = B.make_engine(cfg, args.dtype, max_tokens=2 * tokens + 4096, max_model_len=tokens + 64, gemm=args.gemm,
                            page_size=args.page_size, extra=extra)
        ms = B.measure_prefill_chunks(eng, tokens, args.chunk, reps=3 if tokens <= 8192 else 2, warmup=1)
        flops = eng.model.step_flops(tokens, tokens * (tokens + 1) / 2.0, 1)
        base.update(tokens=tokens, chunk=args.chunk, ms=round(ms, 3), tok_s=round(tokens * 1e3 / ms, 1),
                    frac=round(flops / (ms * 1e-3) / B.PEAK_FLOPS[args.dtype], 4))
        if tokens <= 8192:                         # (a longer prompt in one step wants scratch buffers of its own size)
            base["whole_prompt_ms"] = round(B.measure_prefill(eng, tokens), 3)
    else:
        # room for every request's prompt and new tokens at once (no preemption in the timed run)
        tokens = args.requests * (2048 + args.new_tokens + args.page_size)
        eng = B.make_engine(cfg, args.dtype, max_tokens=tokens, max_model_len=2048 + args.new_tokens + 64,
                            gemm=args.gemm, page_size=args.page_size, max_requests=max(64, args.requests))
        res = B.measure_mixed(eng, args.requests, 128, 2048, args.new_tokens, args.chunk)
        base.update(chunk=args.chunk, new_tokens=args.new_tokens, **res)
        # the products alone (attention's share depends on the lengths drawn)
        base["prefill_frac"] = round(res["prompt_tok_s"] * eng.model.step_flops(1, 0.0, 0) / B.PEAK_FLOPS[args.dtype], 4)
    print(json.dumps(base))
    return 0


if __name__ == "__main__":
    sys.exit(main())
