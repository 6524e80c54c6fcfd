"""Replaying a trace of steps through the engine's own step function.

A trace step names, per request, its next tokens and the places whose logits
are wanted, plus the requests that end after the step.  Nothing is sampled and
no scheduler is involved: the batch of each step is exactly what the trace
says.  This is the role the reference's oracle harness plays for its tests
(engine/oracle/oracle.go:47-137), made a program:

    python -m kllm_amd.replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

(``bin/trace_run`` is the same program.)  Standard input carries one JSON
object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, DIR/<step>.f32 receives the logits at
the wanted places, in the order of the entries and of ``want``, as
little-endian float32 [wanted, vocab].  After every step a line ``done <step>``
is printed and flushed.  It has no forward pass, cache or loader of its own.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional, Sequence

import numpy as np

from .engine import Engine, EngineOptions, StepEntry


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16,
                 device: int = 0, options: Optional[EngineOptions] = None):
        if options is None:
            # The pool holds max_tokens tokens; a request's count is rounded up
            # to whole pages (and to 64, which whole pages of 16 divide).
            options = EngineOptions(device=device, dtype=dtype, page_size=page_size,
                                    max_tokens=max_tokens, max_model_len=1 << 30,
                                    max_requests=64)
        self.engine = Engine.from_dir(model_dir, options)

    def step(self, entries: Sequence[dict], end: Sequence = ()) -> Optional[np.ndarray]:
        """Run one trace step; returns float32 logits [wanted, vocab] or None."""
        logits = None
        if entries:
            batch = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in entries]
            out = self.engine.step(batch)
            if out is not None:
                logits = out.detach().to("cpu").numpy().astype(np.float32, copy=False)
        for rid in end:
            if rid in self.engine.cache:
                self.engine.release(rid)
        return logits


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", type=int, default=0)
    args = ap.parse_args(argv)

    print("trace_run: loading (kernels are compiled at the first call)", file=sys.stderr, flush=True)
    rep = Replayer(args.model, args.dtype, args.max_tokens, page_size=args.page_size, device=args.device)
    os.makedirs(args.out, exist_ok=True)
    print("trace_run: ready", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        logits = rep.step(rec.get("entries", []), rec.get("end", []))
        if logits is not None:
            logits.astype("<f4").tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
